// CPU oracle: a restatement of LBANN's CPU (OpenMP) implementation of the
// forward/backward compute of the normalization, softmax and neighbouring layers
// listed below.  TEST INFRASTRUCTURE ONLY: this file
// is the checker that the HIP kernels are compared against and the timed CPU
// baseline of the benchmark; nothing in the product path may call it.
//
// Every function keeps the reference's loop order, accumulation type and
// operation order (sequential accumulation in the tensor data type, the same
// clamps, reciprocal-vs-divide choices), so that its rounding pattern is the
// reference's when built with -ffp-contract=off.  The `_f64` instantiations
// are the same code with TensorDataType=double (a data type the reference can
// also be built with) and serve as the "exact" answer where the fp32 reference
// is itself noisy.
//
// Matrices are column-major, element (r,c) at buf[r + c*ld], one column per
// sample, exactly like El::Matrix<T,CPU>.
//
// Pinning status (see tests/test_oracle_*.py): every function below is pinned
// by float64 closed forms taken from the reference's own unit tests, by
// invariants, by finite differences or by torch library routines; none is
// "parity unpinned".
//
// Followed reference code (file:line in LBANN v0.105.0):
//   layer norm      src/layers/regularizers/layer_norm.cpp:41-136 (fwd), :139-258 (bwd)
//   batch norm      src/layers/regularizers/batch_normalization.cpp:37-175 (fwd), :178-329 (bwd)
//   softmax         include/lbann/utils/dnn_lib/openmp/softmax.hpp:39-117 (fwd), :119-181 (bwd)
//   log-softmax     src/layers/activations/log_softmax.cpp:35-93 (fwd), :95-136 (bwd)
//   channelwise sm  src/layers/misc/channelwise_softmax.cpp:41-99 (fwd), :121-169 (bwd)
//   instance norm   src/layers/regularizers/instance_norm.cpp:47-113 (fwd), :137-231 (bwd)
//   entry-wise bn   src/layers/regularizers/entrywise_batch_normalization.cpp:52-202 (fwd),
//                   :210-414 (bwd)
//   cross entropy   src/layers/loss/cross_entropy.cpp:35-73 (fwd), :75-120 (bwd)
//   entry-wise scale/bias    src/layers/learning/entrywise_scale_bias.cpp:35-60, :62-113
//   channel-wise scale/bias  src/layers/learning/channelwise_scale_bias.cpp:33-73, :75-135
//   gradient buffer update   include/lbann/optimizers/optimizer_impl.hpp:207-217

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <limits>
#include <vector>
#ifdef _OPENMP
#include <omp.h>
#endif

namespace {

using idx = std::int64_t;

template <typename T>
struct CMat {  // const column-major view
  const T* p;
  idx ld;
  const T& operator()(idx r, idx c) const { return p[r + c * ld]; }
};
template <typename T>
struct Mat {  // mutable column-major view
  T* p;
  idx ld;
  T& operator()(idx r, idx c) const { return p[r + c * ld]; }
};

// ---------------------------------------------------------------- layer norm
// layer_norm.cpp:41-136.  stats is (2G x w): rows [0,G) means, [G,2G) variances.
template <typename T>
void ln_fwd(idx G, idx n, idx stride, idx w, T eps, CMat<T> x, Mat<T> y,
            Mat<T> stats, const T* gamma, const T* beta)
{
  // layer_norm.cpp:76  El::Zero(statistics)
  for (idx i = 0; i < w; ++i)
    for (idx j = 0; j < 2 * G; ++j) stats(j, i) = T(0);

  // layer_norm.cpp:77-88  running sums, accumulated in place in the stats matrix
#pragma omp parallel for collapse(2)
  for (idx i = 0; i < w; ++i) {
    for (idx j = 0; j < G; ++j) {
      T& sum = stats(j, i);
      T& sqsum = stats(G + j, i);
      for (idx k = 0; k < n; ++k) {
        const T v = x(k + j * stride, i);
        sum += v;
        sqsum += v * v;
      }
    }
  }

  // layer_norm.cpp:94-113
  if (n <= 1) {
    for (idx i = 0; i < w; ++i)
      for (idx j = 0; j < G; ++j) stats(G + j, i) = T(1);
  }
  else {
#pragma omp parallel for collapse(2)
    for (idx i = 0; i < w; ++i) {
      for (idx j = 0; j < G; ++j) {
        const T sum = stats(j, i);
        const T sqsum = stats(G + j, i);
        const T nn = static_cast<T>(n);
        const T mean = sum / nn;
        const T sqmean = sqsum / nn;
        const T var = sqmean - mean * mean;
        stats(j, i) = mean;
        stats(G + j, i) = std::max(var, T(0));
      }
    }
  }

  // layer_norm.cpp:117-135
#pragma omp parallel for collapse(2)
  for (idx i = 0; i < w; ++i) {
    for (idx j = 0; j < G; ++j) {
      const T mean = stats(j, i);
      const T var = stats(G + j, i);
      const T inv_stdev = T(1) / std::sqrt(var + eps);
      for (idx k = 0; k < n; ++k) {
        const T v = x(k + j * stride, i);
        T r = (v - mean) * inv_stdev;
        if (gamma) r *= gamma[k];
        if (beta) r += beta[k];
        y(k + j * stride, i) = r;
      }
    }
  }
}

// layer_norm.cpp:139-258 plus the zeroing of the weight-gradient buffers done by
// bp_compute (:300-309).  stats_grad is (2G x w): rows [0,G) dmean, [G,2G) dvar.
template <typename T>
void ln_bwd(idx G, idx n, idx stride, idx w, idx h, T eps, CMat<T> x, CMat<T> dy,
            Mat<T> dx, CMat<T> stats, Mat<T> sgrad, const T* gamma, T* dgamma,
            T* dbeta)
{
  if (dgamma) std::fill(dgamma, dgamma + n, T(0));
  if (dbeta) std::fill(dbeta, dbeta + n, T(0));

  // layer_norm.cpp:189-192
  if (n <= 1) {
    for (idx i = 0; i < w; ++i)
      for (idx r = 0; r < h; ++r) dx(r, i) = T(0);
    return;
  }

  for (idx i = 0; i < w; ++i)
    for (idx j = 0; j < 2 * G; ++j) sgrad(j, i) = T(0);

  // layer_norm.cpp:198-227
#pragma omp parallel for collapse(2)
  for (idx i = 0; i < w; ++i) {
    for (idx j = 0; j < G; ++j) {
      const T mean = stats(j, i);
      const T var = stats(G + j, i);
      const T inv_stdev = T(1) / std::sqrt(var + eps);
      T& dmean = sgrad(j, i);
      T& dvar = sgrad(G + j, i);
      for (idx k = 0; k < n; ++k) {
        const T v = x(k + j * stride, i);
        T g = dy(k + j * stride, i);
        if (dbeta) {
#pragma omp atomic
          dbeta[k] += g;
        }
        if (dgamma) {
          const T contrib = g * (v - mean) * inv_stdev;
#pragma omp atomic
          dgamma[k] += contrib;
          g *= gamma[k];
        }
        dmean += g;
        dvar += g * (v - mean);
      }
      dmean *= -inv_stdev;
      dvar *= -inv_stdev * inv_stdev * inv_stdev / 2;
    }
  }

  // layer_norm.cpp:236-257  (the code divides by n, not n-1)
#pragma omp parallel for collapse(2)
  for (idx i = 0; i < w; ++i) {
    for (idx j = 0; j < G; ++j) {
      const T mean = stats(j, i);
      const T var = stats(G + j, i);
      const T inv_stdev = T(1) / std::sqrt(var + eps);
      const T dmean = sgrad(j, i);
      const T dvar = sgrad(G + j, i);
      for (idx k = 0; k < n; ++k) {
        const T v = x(k + j * stride, i);
        T g = dy(k + j * stride, i);
        if (gamma) g *= gamma[k];
        dx(k + j * stride, i) =
          g * inv_stdev + dmean / n + dvar * (v - mean) * 2 / n;
      }
    }
  }
}

// ---------------------------------------------------------------- batch norm
// batch_normalization.cpp:37-175, local statistics (statistics_group_size==1), so
// num_per_sum = channel_size * local_width (:94-97).
template <typename T>
void bn_fwd(idx C, idx cs, idx w, int bessel, T eps, T decay, int training,
            CMat<T> x, Mat<T> y, T* mean_out, T* var_out, const T* gamma,
            const T* beta, T* running_mean, T* running_var)
{
  const int correction = bessel ? 1 : 0;
  if (training) {
    // :70-85
#pragma omp parallel for
    for (idx c = 0; c < C; ++c) {
      T sum = T(0), sqsum = T(0);
      const idx r0 = c * cs, r1 = (c + 1) * cs;
      for (idx col = 0; col < w; ++col) {
        for (idx r = r0; r < r1; ++r) {
          const T v = x(r, col);
          sum += v;
          sqsum += v * v;
        }
      }
      mean_out[c] = sum;
      var_out[c] = sqsum;
    }
    const idx num_per_sum = cs * w;
    // :118-138
    if (num_per_sum <= 1) {
      for (idx c = 0; c < C; ++c) var_out[c] = T(1);
    }
    else {
#pragma omp parallel for
      for (idx c = 0; c < C; ++c) {
        const T nn = static_cast<T>(num_per_sum);
        const T mean = mean_out[c] / nn;
        const T sqmean = var_out[c] / nn;
        T var = nn * (sqmean - mean * mean) / (nn - correction);
        var = std::max(var, eps);
        mean_out[c] = mean;
        var_out[c] = var;
        running_mean[c] = decay * running_mean[c] + (T(1) - decay) * mean;
        running_var[c] = decay * running_var[c] + (T(1) - decay) * var;
      }
    }
  }
  // :141-174  training uses the batch statistics, otherwise the running ones
  const T* use_mean = training ? mean_out : running_mean;
  const T* use_var = training ? var_out : running_var;
#pragma omp parallel for
  for (idx c = 0; c < C; ++c) {
    const T mean = use_mean[c];
    const T var = use_var[c];
    const T inv_stdev = static_cast<T>(1 / std::sqrt(var + eps));
    const T scale = gamma[c];
    const T bias = beta[c];
    const idx r0 = c * cs, r1 = (c + 1) * cs;
    for (idx col = 0; col < w; ++col) {
      for (idx r = r0; r < r1; ++r) {
        const T xhat = (x(r, col) - mean) * inv_stdev;
        y(r, col) = scale * xhat + bias;
      }
    }
  }
}

// batch_normalization.cpp:178-329.
template <typename T>
void bn_bwd(idx C, idx cs, idx w, int bessel, T eps, int training, CMat<T> x,
            CMat<T> dy, Mat<T> dx, const T* mean_in, const T* var_in,
            const T* running_mean, const T* running_var, const T* gamma,
            T* dgamma, T* dbeta, T* dmean_out, T* dvar_out)
{
  const int correction = bessel ? 1 : 0;
  const T* use_mean = training ? mean_in : running_mean;
  const T* use_var = training ? var_in : running_var;
  // :211-245
#pragma omp parallel for
  for (idx c = 0; c < C; ++c) {
    const T mean = use_mean[c];
    const T var = use_var[c];
    const T scale = gamma[c];
    const T inv_stdev = static_cast<T>(1 / std::sqrt(var + eps));
    const T dvar_factor = inv_stdev * inv_stdev * inv_stdev / 2;
    T dmean = T(0), dvar = T(0), dscale = T(0), dbias = T(0);
    const idx r0 = c * cs, r1 = (c + 1) * cs;
    for (idx col = 0; col < w; ++col) {
      for (idx r = r0; r < r1; ++r) {
        const T v = x(r, col);
        const T xhat = (v - mean) * inv_stdev;
        const T g = dy(r, col);
        dscale += g * xhat;
        dbias += g;
        const T dxhat = g * scale;
        dmean += -dxhat * inv_stdev;
        dvar += -dxhat * (v - mean) * dvar_factor;
      }
    }
    dmean_out[c] = dmean;
    dvar_out[c] = dvar;
    dgamma[c] = dscale;
    dbeta[c] = dbias;
  }
  // :248-267  outside training the statistics gradients are dropped
  if (!training) {
    for (idx c = 0; c < C; ++c) {
      dmean_out[c] = T(0);
      dvar_out[c] = T(0);
    }
  }
  // :282-328
  const idx num_per_sum = cs * w;
  if (num_per_sum <= 1) {
    for (idx col = 0; col < w; ++col)
      for (idx r = 0; r < C * cs; ++r) dx(r, col) = T(0);
    return;
  }
#pragma omp parallel for
  for (idx c = 0; c < C; ++c) {
    const T mean = use_mean[c];
    const T var = use_var[c];
    const T scale = gamma[c];
    const T dmean = dmean_out[c];
    const T dvar = dvar_out[c];
    const T inv_stdev = static_cast<T>(1 / std::sqrt(var + eps));
    const T dmean_term = dmean / num_per_sum;
    const T dvar_term = dvar * 2 / (num_per_sum - correction);
    const idx r0 = c * cs, r1 = (c + 1) * cs;
    for (idx col = 0; col < w; ++col) {
      for (idx r = r0; r < r1; ++r) {
        const T dxhat = dy(r, col) * scale;
        dx(r, col) = dxhat * inv_stdev + dmean_term + dvar_term * (x(r, col) - mean);
      }
    }
  }
}

// ------------------------------------------------------------------- softmax
// openmp/softmax.hpp:39-117
template <typename T>
void sm_fwd(idx h, idx w, CMat<T> x, Mat<T> y)
{
  std::vector<T> work(static_cast<size_t>(w), std::numeric_limits<T>::lowest());
  T* ws = work.data();
#pragma omp parallel for
  for (idx c = 0; c < w; ++c) {
    T& m = ws[c];
    for (idx r = 0; r < h; ++r) m = std::max(m, x(r, c));
  }
#pragma omp parallel for
  for (idx c = 0; c < w; ++c) {
    const T shift = ws[c];
    T sum = T(0);
    for (idx r = 0; r < h; ++r) {
      const T e = std::exp(x(r, c) - shift);
      y(r, c) = e;
      sum += e;
    }
    ws[c] = sum;
  }
#pragma omp parallel for
  for (idx c = 0; c < w; ++c) {
    const T scale = 1 / ws[c];
    for (idx r = 0; r < h; ++r) {
      const T t = scale * y(r, c);
      y(r, c) = std::isnormal(t) ? t : T(0);
    }
  }
}

// openmp/softmax.hpp:119-181
template <typename T>
void sm_bwd(idx h, idx w, CMat<T> y, CMat<T> dy, Mat<T> dx)
{
  std::vector<T> work(static_cast<size_t>(w), T(0));
  T* ws = work.data();
#pragma omp parallel for
  for (idx c = 0; c < w; ++c) {
    T& d = ws[c];
    for (idx r = 0; r < h; ++r) d += y(r, c) * dy(r, c);
  }
#pragma omp parallel for
  for (idx c = 0; c < w; ++c) {
    const T d = ws[c];
    for (idx r = 0; r < h; ++r) dx(r, c) = y(r, c) * (dy(r, c) - d);
  }
}

// --------------------------------------------------------------- log-softmax
// log_softmax.cpp:35-93
template <typename T>
void lsm_fwd(idx h, idx w, CMat<T> x, Mat<T> y)
{
  std::vector<T> work(static_cast<size_t>(w), std::numeric_limits<T>::lowest());
  T* ws = work.data();
#pragma omp parallel for
  for (idx c = 0; c < w; ++c) {
    T& m = ws[c];
    for (idx r = 0; r < h; ++r) m = std::max(m, x(r, c));
  }
#pragma omp parallel for
  for (idx c = 0; c < w; ++c) {
    const T shift = ws[c];
    T sum{0};
    for (idx r = 0; r < h; ++r) {
      const T v = x(r, c) - shift;
      y(r, c) = v;
      sum += std::exp(v);
    }
    ws[c] = sum;
  }
#pragma omp parallel for
  for (idx c = 0; c < w; ++c) {
    const T lse = static_cast<T>(std::log(ws[c]));
    for (idx r = 0; r < h; ++r) y(r, c) -= lse;
  }
}

// log_softmax.cpp:95-136
template <typename T>
void lsm_bwd(idx h, idx w, CMat<T> y, CMat<T> dy, Mat<T> dx)
{
  std::vector<T> work(static_cast<size_t>(w), T(0));
  T* ws = work.data();
#pragma omp parallel for
  for (idx c = 0; c < w; ++c) {
    T& s = ws[c];
    for (idx r = 0; r < h; ++r) s += dy(r, c);
  }
#pragma omp parallel for
  for (idx c = 0; c < w; ++c) {
    const T s = ws[c];
    for (idx r = 0; r < h; ++r) dx(r, c) = dy(r, c) - std::exp(y(r, c)) * s;
  }
}

// -------------------------------------------------------- channelwise softmax
// channelwise_softmax.cpp:41-99.  Only the max loop is parallel in the
// reference; the denominator and output loops (:75, :88) carry no pragma.
template <typename T>
void cws_fwd(idx C, idx cs, idx stride, idx w, CMat<T> x, Mat<T> y)
{
  std::vector<T> shifts(static_cast<size_t>(C * w), std::numeric_limits<T>::lowest());
  std::vector<T> denoms(static_cast<size_t>(C * w), T(0));
  T* sh = shifts.data();
  T* dn = denoms.data();
#pragma omp parallel for collapse(2)
  for (idx k = 0; k < w; ++k) {
    for (idx j = 0; j < C; ++j) {
      T& m = sh[j + k * C];
      for (idx i = 0; i < cs; ++i) m = std::max(m, x(i + j * stride, k));
    }
  }
  for (idx k = 0; k < w; ++k) {
    for (idx j = 0; j < C; ++j) {
      const T shift = sh[j + k * C];
      T& d = dn[j + k * C];
      for (idx i = 0; i < cs; ++i) d += std::exp(x(i + j * stride, k) - shift);
    }
  }
  for (idx k = 0; k < w; ++k) {
    for (idx j = 0; j < C; ++j) {
      const T shift = sh[j + k * C];
      const T d = dn[j + k * C];
      for (idx i = 0; i < cs; ++i)
        y(i + j * stride, k) = std::exp(x(i + j * stride, k) - shift) / d;
    }
  }
}

// channelwise_softmax.cpp:121-169
template <typename T>
void cws_bwd(idx C, idx cs, idx stride, idx w, CMat<T> y, CMat<T> dy, Mat<T> dx)
{
  std::vector<T> dots(static_cast<size_t>(C * w), T(0));
  T* dt = dots.data();
#pragma omp parallel for collapse(2)
  for (idx k = 0; k < w; ++k) {
    for (idx j = 0; j < C; ++j) {
      T& d = dt[j + k * C];
      for (idx i = 0; i < cs; ++i) d += y(i + j * stride, k) * dy(i + j * stride, k);
    }
  }
#pragma omp parallel for collapse(2)
  for (idx k = 0; k < w; ++k) {
    for (idx j = 0; j < C; ++j) {
      const T d = dt[j + k * C];
      for (idx i = 0; i < cs; ++i)
        dx(i + j * stride, k) = y(i + j * stride, k) * (dy(i + j * stride, k) - d);
    }
  }
}

// ------------------------------------------------------------ instance norm
// instance_norm.cpp:47-113.  sums is the layer's workspace, (2C x w): rows [0,C) hold
// sum(x), rows [C,2C) sum(x^2) of each (channel, sample).
template <typename T>
void in_fwd(idx C, idx cs, idx w, T eps, CMat<T> x, Mat<T> y, Mat<T> sums)
{
  if (cs <= 1) {  // :65-68: the output is constant
    for (idx k = 0; k < w; ++k)
      for (idx i = 0; i < C * cs; ++i) y(i, k) = T(0);
    return;
  }
  for (idx k = 0; k < w; ++k)
    for (idx j = 0; j < 2 * C; ++j) sums(j, k) = T(0);
#pragma omp parallel for collapse(2)
  for (idx k = 0; k < w; ++k) {
    for (idx j = 0; j < C; ++j) {
      T& sum = sums(j, k);
      T& sqsum = sums(C + j, k);
      for (idx i = 0; i < cs; ++i) {
        const T v = x(i + j * cs, k);
        sum += v;
        sqsum += v * v;
      }
    }
  }
  const T mean_scale = T(1.) / cs;
#pragma omp parallel for collapse(2)
  for (idx k = 0; k < w; ++k) {
    for (idx j = 0; j < C; ++j) {
      const T mean = sums(j, k) * mean_scale;
      const T sqmean = sums(C + j, k) * mean_scale;
      T var = sqmean - mean * mean;
      var = std::max(var, T(0.));
      const T inv_stdev = T(1.) / std::sqrt(var + eps);
      for (idx i = 0; i < cs; ++i) y(i + j * cs, k) = (x(i + j * cs, k) - mean) * inv_stdev;
    }
  }
}

// instance_norm.cpp:137-231.  The variance is recomputed from the sums WITHOUT the
// clamp at zero of the forward pass (:186, :211), and the last factor is 2/cs (:225-226).
template <typename T>
void in_bwd(idx C, idx cs, idx w, T eps, CMat<T> x, CMat<T> dy, Mat<T> dx, CMat<T> sums)
{
  if (cs <= 1) {  // :164-167
    for (idx k = 0; k < w; ++k)
      for (idx i = 0; i < C * cs; ++i) dx(i, k) = T(0);
    return;
  }
  std::vector<T> sgrad(static_cast<size_t>(2 * C * w), T(0));
  const T mean_scale = T(1.) / cs;
#pragma omp parallel for collapse(2)
  for (idx k = 0; k < w; ++k) {
    for (idx j = 0; j < C; ++j) {
      const T mean = sums(j, k) * mean_scale;
      const T sqmean = sums(C + j, k) * mean_scale;
      const T var = sqmean - mean * mean;
      const T inv_stdev = T(1.) / std::sqrt(var + eps);
      T& dmean = sgrad[j + k * 2 * C];
      T& dvar = sgrad[C + j + k * 2 * C];
      for (idx i = 0; i < cs; ++i) {
        const T g = dy(i + j * cs, k);
        dmean += g;
        dvar += g * (x(i + j * cs, k) - mean);
      }
      dmean *= -inv_stdev;
      dvar *= -inv_stdev * inv_stdev * inv_stdev / 2;
    }
  }
#pragma omp parallel for collapse(2)
  for (idx k = 0; k < w; ++k) {
    for (idx j = 0; j < C; ++j) {
      const T mean = sums(j, k) * mean_scale;
      const T sqmean = sums(C + j, k) * mean_scale;
      const T var = sqmean - mean * mean;
      const T inv_stdev = T(1.) / std::sqrt(var + eps);
      const T dmean = sgrad[j + k * 2 * C];
      const T dvar = sgrad[C + j + k * 2 * C];
      for (idx i = 0; i < cs; ++i)
        dx(i + j * cs, k) = (dy(i + j * cs, k) * inv_stdev + dmean / cs +
                             dvar * (x(i + j * cs, k) - mean) * 2 / cs);
    }
  }
}

// ------------------------------------------------- entry-wise batch norm
// entrywise_batch_normalization.cpp:52-202.  Statistics per entry (matrix row) over
// the mini-batch (matrix columns); stats is (h x 2): column 0 mean, column 1 variance
// (Bessel corrected, not clamped).  The reference walks the rows in blocks of one
// cache line (:44-45); within a block the column loop is outside the row loop, which
// fixes the order in which each row's sums are accumulated: ascending columns.
template <typename T>
void ebn_fwd(idx h, idx w, T decay, T eps, int training, CMat<T> x, Mat<T> y, Mat<T> stats,
             T* rmean, T* rvar)
{
  const idx bsize = std::max<idx>(64 / static_cast<idx>(sizeof(float)), 1);  // DataType is float
  const T* mean = rmean;
  const T* var = rvar;
  if (training) {
    for (idx r = 0; r < h; ++r) stats(r, 0) = stats(r, 1) = T(0);
#pragma omp parallel for
    for (idx r0 = 0; r0 < h; r0 += bsize) {
      const idx r1 = std::min(r0 + bsize, h);
      for (idx c = 0; c < w; ++c)
        for (idx r = r0; r < r1; ++r) {
          const T v = x(r, c);
          stats(r, 0) += v;
          stats(r, 1) += v * v;
        }
    }
    if (w <= 1) {  // :103-106: the means already hold x
      for (idx r = 0; r < h; ++r) stats(r, 1) = T(1);
    }
    else {
#pragma omp parallel for
      for (idx r = 0; r < h; ++r) {
        const T sum = stats(r, 0);
        const T sqsum = stats(r, 1);
        const T m = sum / w;
        const T sqmean = sqsum / w;
        const T v = (sqmean - m * m) * w / (w - 1);
        stats(r, 0) = m;
        stats(r, 1) = v;
        rmean[r] = decay * rmean[r] + (T(1) - decay) * m;
        rvar[r] = decay * rvar[r] + (T(1) - decay) * v;
      }
    }
    mean = &stats(0, 0);
    var = &stats(0, 1);
  }
  // apply_batchnorm, :128-157
#pragma omp parallel for
  for (idx r0 = 0; r0 < h; r0 += bsize) {
    const idx r1 = std::min(r0 + bsize, h);
    T inv_stdev[64];
    for (idx r = r0; r < r1; ++r) inv_stdev[r - r0] = 1 / std::sqrt(var[r] + eps);
    for (idx c = 0; c < w; ++c)
      for (idx r = r0; r < r1; ++r) y(r, c) = (x(r, c) - mean[r]) * inv_stdev[r - r0];
  }
}

// entrywise_batch_normalization.cpp:210-414.  sgrad is (h x 2): dL/dmean, dL/dvar
// (written in training mode only).
template <typename T>
void ebn_bwd(idx h, idx w, T eps, int training, CMat<T> x, CMat<T> dy, Mat<T> dx, CMat<T> stats,
             Mat<T> sgrad, const T* rvar)
{
  const idx bsize = std::max<idx>(64 / static_cast<idx>(sizeof(float)), 1);
  if (!training) {  // :352-392
#pragma omp parallel for
    for (idx r0 = 0; r0 < h; r0 += bsize) {
      const idx r1 = std::min(r0 + bsize, h);
      T inv_stdev[64];
      for (idx r = r0; r < r1; ++r) inv_stdev[r - r0] = 1 / std::sqrt(rvar[r] + eps);
      for (idx c = 0; c < w; ++c)
        for (idx r = r0; r < r1; ++r) dx(r, c) = dy(r, c) * inv_stdev[r - r0];
    }
    return;
  }
  if (w <= 1) {  // :257-261
    for (idx c = 0; c < w; ++c)
      for (idx r = 0; r < h; ++r) dx(r, c) = T(0);
    return;
  }
  for (idx r = 0; r < h; ++r) sgrad(r, 0) = sgrad(r, 1) = T(0);
#pragma omp parallel for
  for (idx r0 = 0; r0 < h; r0 += bsize) {
    const idx r1 = std::min(r0 + bsize, h);
    T inv_stdev[64];
    for (idx r = r0; r < r1; ++r) inv_stdev[r - r0] = 1 / std::sqrt(stats(r, 1) + eps);
    for (idx c = 0; c < w; ++c)
      for (idx r = r0; r < r1; ++r) {
        const T is = inv_stdev[r - r0];
        const T g = dy(r, c);
        sgrad(r, 0) += -g * is;
        sgrad(r, 1) += -g * (x(r, c) - stats(r, 0)) * is * is * is / 2;
      }
  }
  const T wt = static_cast<T>(w);
  const T inv_w = T(1) / wt;
  const T inv_wm1 = T(1) / (wt - T(1));
#pragma omp parallel for
  for (idx r0 = 0; r0 < h; r0 += bsize) {
    const idx r1 = std::min(r0 + bsize, h);
    T inv_stdev[64];
    for (idx r = r0; r < r1; ++r) inv_stdev[r - r0] = 1 / std::sqrt(stats(r, 1) + eps);
    for (idx c = 0; c < w; ++c)
      for (idx r = r0; r < r1; ++r)
        dx(r, c) = (dy(r, c) * inv_stdev[r - r0] + sgrad(r, 0) * inv_w +
                    sgrad(r, 1) * (x(r, c) - stats(r, 0)) * 2 * inv_wm1);
  }
}

// ----------------------------------------------------------- cross entropy
// cross_entropy.cpp:35-73 (local_fp_cpu).  loss(0,c) = sum over rows with xhat > 0 of
// -xhat*log(x), accumulated in row order.  With use_labels the ground truth holds one
// class index per spatial position (rows [0,spatial) of truth) and
// xhat(row) = (truth(row % spatial) == row / spatial).
template <typename T>
void ce_fwd(idx h, idx w, int use_labels, idx spatial, CMat<T> x, CMat<T> truth, T* loss)
{
#pragma omp parallel for
  for (idx c = 0; c < w; ++c) {
    T sum = T(0);
    for (idx r = 0; r < h; ++r) {
      T xhat;
      if (use_labels) {
        const idx channel = r / spatial;
        const idx offset = r % spatial;
        const int label = static_cast<int>(truth(offset, c));
        xhat = T(label == channel ? 1. : 0.);
      }
      else {
        xhat = truth(r, c);
      }
      if (xhat > T(0)) sum += -xhat * std::log(x(r, c));
    }
    loss[c] = sum;
  }
}

// cross_entropy.cpp:75-120 (local_bp_cpu).  dy is the (1 x w) gradient w.r.t. the loss.
// dtruth is written only without use_labels.
template <typename T>
void ce_bwd(idx h, idx w, int use_labels, idx spatial, CMat<T> x, CMat<T> truth, const T* dy,
            Mat<T> dx, Mat<T> dtruth)
{
#pragma omp parallel for collapse(2)
  for (idx c = 0; c < w; ++c) {
    for (idx r = 0; r < h; ++r) {
      const T g = dy[c];
      const T v = x(r, c);
      T xhat;
      if (use_labels) {
        const idx channel = r / spatial;
        const idx offset = r % spatial;
        const int label = static_cast<int>(truth(offset, c));
        xhat = T(label == channel ? 1. : 0.);
      }
      else {
        xhat = truth(r, c);
        dtruth(r, c) = -g * std::log(v);
      }
      dx(r, c) = (xhat > T(0)) ? -g * xhat / v : T(0);
    }
  }
}

// ----------------------------------------------------- entry-wise scale/bias
// entrywise_scale_bias.cpp:35-60 (fp_impl), :62-113 (bp_impl).  weights is (h x 2):
// column 0 scale, column 1 bias; wgrad likewise.  Row sums accumulate over ascending
// columns (rows are walked in blocks of one cache line, the column loop outside).
template <typename T>
void esb_fwd(idx h, idx w, CMat<T> x, Mat<T> y, CMat<T> weights)
{
#pragma omp parallel for collapse(2)
  for (idx c = 0; c < w; ++c)
    for (idx r = 0; r < h; ++r) y(r, c) = weights(r, 0) * x(r, c) + weights(r, 1);
}

template <typename T>
void esb_bwd(idx h, idx w, CMat<T> x, CMat<T> dy, Mat<T> dx, CMat<T> weights, Mat<T> wgrad)
{
  for (idx r = 0; r < h; ++r) wgrad(r, 0) = wgrad(r, 1) = T(0);
  const idx bsize = std::max<idx>(64 / static_cast<idx>(sizeof(float)), 1);  // DataType is float
#pragma omp parallel for
  for (idx r0 = 0; r0 < h; r0 += bsize) {
    const idx r1 = std::min(r0 + bsize, h);
    for (idx c = 0; c < w; ++c)
      for (idx r = r0; r < r1; ++r) {
        const T g = dy(r, c);
        dx(r, c) = weights(r, 0) * g;
        wgrad(r, 0) += x(r, c) * g;
        wgrad(r, 1) += g;
      }
  }
}

// --------------------------------------------------- channel-wise scale/bias
// channelwise_scale_bias.cpp:33-73 (fp_compute), :75-135 (bp_compute).  Channel ch is
// rows [ch*cs, (ch+1)*cs) of every column; weights is (C x 2): scale, bias.  Sums run
// over columns, then rows, in order.
template <typename T>
void csb_fwd(idx C, idx cs, idx w, CMat<T> x, Mat<T> y, CMat<T> weights)
{
#pragma omp parallel for
  for (idx ch = 0; ch < C; ++ch) {
    const T a = weights(ch, 0);
    const T b = weights(ch, 1);
    for (idx c = 0; c < w; ++c)
      for (idx r = ch * cs; r < (ch + 1) * cs; ++r) y(r, c) = a * x(r, c) + b;
  }
}

template <typename T>
void csb_bwd(idx C, idx cs, idx w, CMat<T> x, CMat<T> dy, Mat<T> dx, CMat<T> weights, Mat<T> wgrad)
{
#pragma omp parallel for
  for (idx ch = 0; ch < C; ++ch) {
    const T a = weights(ch, 0);
    T da = T(0), db = T(0);
    for (idx c = 0; c < w; ++c)
      for (idx r = ch * cs; r < (ch + 1) * cs; ++r) {
        const T g = dy(r, c);
        da += x(r, c) * g;
        db += g;
        dx(r, c) = a * g;
      }
    wgrad(ch, 0) = da;
    wgrad(ch, 1) = db;
  }
}

// ------------------------------------------------------- gradient buffer update
// optimizer::add_to_gradient (optimizer_impl.hpp:207-217): El::Scale(buf_scale, grad) then
// El::Axpy(alpha, contrib, grad), on local matrices.  Hydrogen (>= 1.5.0, not part of the
// reference tree) documents Scale by zero as zeroing the matrix whatever it held, and by
// one as a no-op; Axpy is y += alpha * x element by element.  Two statements, so that the
// scaled buffer is rounded before the sum as with the two calls.
template <typename T>
void grad_sink(idx h, idx w, T buf_scale, T alpha, CMat<T> contrib, Mat<T> grad)
{
  for (idx c = 0; c < w; ++c)
    for (idx r = 0; r < h; ++r) {
      if (buf_scale == T(0)) grad(r, c) = T(0);
      else if (buf_scale != T(1)) grad(r, c) = buf_scale * grad(r, c);
    }
  for (idx c = 0; c < w; ++c)
    for (idx r = 0; r < h; ++r) {
      const T t = alpha * contrib(r, c);
      grad(r, c) = grad(r, c) + t;
    }
}

}  // namespace

// C interface (one _f32 and one _f64 entry per function), bound by oracle/cpu_oracle.py.
#define ORC_INSTANTIATE(SUF, T)                                                          \
  extern "C" void orc_layer_norm_fwd_##SUF(idx G, idx n, idx stride, idx w, T eps,       \
      const T* x, idx ldx, T* y, idx ldy, T* stats, idx lds, const T* gamma,             \
      const T* beta)                                                                     \
  { ln_fwd<T>(G, n, stride, w, eps, {x, ldx}, {y, ldy}, {stats, lds}, gamma, beta); }    \
  extern "C" void orc_layer_norm_bwd_##SUF(idx G, idx n, idx stride, idx w, idx h,       \
      T eps, const T* x, idx ldx, const T* dy, idx lddy, T* dx, idx lddx,                \
      const T* stats, idx lds, T* sgrad, idx ldsg, const T* gamma, T* dgamma, T* dbeta)  \
  { ln_bwd<T>(G, n, stride, w, h, eps, {x, ldx}, {dy, lddy}, {dx, lddx}, {stats, lds},   \
              {sgrad, ldsg}, gamma, dgamma, dbeta); }                                    \
  extern "C" void orc_batch_norm_fwd_##SUF(idx C, idx cs, idx w, int bessel, T eps,      \
      T decay, int training, const T* x, idx ldx, T* y, idx ldy, T* mean, T* var,        \
      const T* gamma, const T* beta, T* rmean, T* rvar)                                  \
  { bn_fwd<T>(C, cs, w, bessel, eps, decay, training, {x, ldx}, {y, ldy}, mean, var,     \
              gamma, beta, rmean, rvar); }                                               \
  extern "C" void orc_batch_norm_bwd_##SUF(idx C, idx cs, idx w, int bessel, T eps,      \
      int training, const T* x, idx ldx, const T* dy, idx lddy, T* dx, idx lddx,         \
      const T* mean, const T* var, const T* rmean, const T* rvar, const T* gamma,        \
      T* dgamma, T* dbeta, T* dmean, T* dvar)                                            \
  { bn_bwd<T>(C, cs, w, bessel, eps, training, {x, ldx}, {dy, lddy}, {dx, lddx}, mean,   \
              var, rmean, rvar, gamma, dgamma, dbeta, dmean, dvar); }                    \
  extern "C" void orc_softmax_fwd_##SUF(idx h, idx w, const T* x, idx ldx, T* y, idx ldy)\
  { sm_fwd<T>(h, w, {x, ldx}, {y, ldy}); }                                               \
  extern "C" void orc_softmax_bwd_##SUF(idx h, idx w, const T* y, idx ldy, const T* dy,  \
      idx lddy, T* dx, idx lddx)                                                         \
  { sm_bwd<T>(h, w, {y, ldy}, {dy, lddy}, {dx, lddx}); }                                 \
  extern "C" void orc_log_softmax_fwd_##SUF(idx h, idx w, const T* x, idx ldx, T* y,     \
      idx ldy)                                                                           \
  { lsm_fwd<T>(h, w, {x, ldx}, {y, ldy}); }                                              \
  extern "C" void orc_log_softmax_bwd_##SUF(idx h, idx w, const T* y, idx ldy,           \
      const T* dy, idx lddy, T* dx, idx lddx)                                            \
  { lsm_bwd<T>(h, w, {y, ldy}, {dy, lddy}, {dx, lddx}); }                                \
  extern "C" void orc_channelwise_softmax_fwd_##SUF(idx C, idx cs, idx stride, idx w,    \
      const T* x, idx ldx, T* y, idx ldy)                                                \
  { cws_fwd<T>(C, cs, stride, w, {x, ldx}, {y, ldy}); }                                  \
  extern "C" void orc_channelwise_softmax_bwd_##SUF(idx C, idx cs, idx stride, idx w,    \
      const T* y, idx ldy, const T* dy, idx lddy, T* dx, idx lddx)                       \
  { cws_bwd<T>(C, cs, stride, w, {y, ldy}, {dy, lddy}, {dx, lddx}); }                    \
  extern "C" void orc_instance_norm_fwd_##SUF(idx C, idx cs, idx w, T eps, const T* x,   \
      idx ldx, T* y, idx ldy, T* sums, idx lds)                                          \
  { in_fwd<T>(C, cs, w, eps, {x, ldx}, {y, ldy}, {sums, lds}); }                         \
  extern "C" void orc_instance_norm_bwd_##SUF(idx C, idx cs, idx w, T eps, const T* x,   \
      idx ldx, const T* dy, idx lddy, T* dx, idx lddx, const T* sums, idx lds)           \
  { in_bwd<T>(C, cs, w, eps, {x, ldx}, {dy, lddy}, {dx, lddx}, {sums, lds}); }          \
  extern "C" void orc_entrywise_batch_norm_fwd_##SUF(idx h, idx w, T decay, T eps,       \
      int training, const T* x, idx ldx, T* y, idx ldy, T* stats, idx lds, T* rmean,     \
      T* rvar)                                                                           \
  { ebn_fwd<T>(h, w, decay, eps, training, {x, ldx}, {y, ldy}, {stats, lds}, rmean,      \
               rvar); }                                                                  \
  extern "C" void orc_entrywise_batch_norm_bwd_##SUF(idx h, idx w, T eps, int training,  \
      const T* x, idx ldx, const T* dy, idx lddy, T* dx, idx lddx, const T* stats,       \
      idx lds, T* sgrad, idx ldsg, const T* rvar)                                        \
  { ebn_bwd<T>(h, w, eps, training, {x, ldx}, {dy, lddy}, {dx, lddx}, {stats, lds},      \
               {sgrad, ldsg}, rvar); }                                                   \
  extern "C" void orc_cross_entropy_fwd_##SUF(idx h, idx w, int use_labels, idx spatial, \
      const T* x, idx ldx, const T* truth, idx ldt, T* loss)                             \
  { ce_fwd<T>(h, w, use_labels, spatial, {x, ldx}, {truth, ldt}, loss); }                \
  extern "C" void orc_cross_entropy_bwd_##SUF(idx h, idx w, int use_labels, idx spatial, \
      const T* x, idx ldx, const T* truth, idx ldt, const T* dy, T* dx, idx lddx,        \
      T* dtruth, idx lddt)                                                               \
  { ce_bwd<T>(h, w, use_labels, spatial, {x, ldx}, {truth, ldt}, dy, {dx, lddx},         \
              {dtruth, lddt}); }                                                         \
  extern "C" void orc_entrywise_scale_bias_fwd_##SUF(idx h, idx w, const T* x, idx ldx,  \
      T* y, idx ldy, const T* weights, idx ldw)                                          \
  { esb_fwd<T>(h, w, {x, ldx}, {y, ldy}, {weights, ldw}); }                              \
  extern "C" void orc_entrywise_scale_bias_bwd_##SUF(idx h, idx w, const T* x, idx ldx,  \
      const T* dy, idx lddy, T* dx, idx lddx, const T* weights, idx ldw, T* wgrad,       \
      idx ldwg)                                                                          \
  { esb_bwd<T>(h, w, {x, ldx}, {dy, lddy}, {dx, lddx}, {weights, ldw}, {wgrad, ldwg}); } \
  extern "C" void orc_channelwise_scale_bias_fwd_##SUF(idx C, idx cs, idx w, const T* x, \
      idx ldx, T* y, idx ldy, const T* weights, idx ldw)                                 \
  { csb_fwd<T>(C, cs, w, {x, ldx}, {y, ldy}, {weights, ldw}); }                          \
  extern "C" void orc_channelwise_scale_bias_bwd_##SUF(idx C, idx cs, idx w, const T* x, \
      idx ldx, const T* dy, idx lddy, T* dx, idx lddx, const T* weights, idx ldw,        \
      T* wgrad, idx ldwg)                                                                \
  { csb_bwd<T>(C, cs, w, {x, ldx}, {dy, lddy}, {dx, lddx}, {weights, ldw},               \
               {wgrad, ldwg}); }                                                         \
  extern "C" void orc_gradient_sink_##SUF(idx h, idx w, T buf_scale, T alpha,             \
      const T* contrib, idx ldc, T* grad, idx ldg)                                       \
  { grad_sink<T>(h, w, buf_scale, alpha, {contrib, ldc}, {grad, ldg}); }

ORC_INSTANTIATE(f32, float)
ORC_INSTANTIATE(f64, double)

extern "C" int orc_max_threads()
{
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}
