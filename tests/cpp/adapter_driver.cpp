// Test driver for the C++ adapter (lbann_amd/adapter/lbnorm_layers.hpp): plays the
// part of data_type_layer::forward_prop / back_prop_impl_ -- attaches the framework's
// matrices, calls fp_compute() / bp_compute() -- on device buffers handed in by the
// Python tests.  Exceptions are turned into a non-zero return and a message.
#include <cstdio>
#include <cstring>
#include <string>

#include "../../lbann_amd/adapter/lbnorm_layers.hpp"

using namespace lbnorm;

namespace {

int fail(const std::exception& e, char* err, int errlen)
{
  if (err && errlen > 0) {
    std::strncpy(err, e.what(), static_cast<size_t>(errlen) - 1);
    err[errlen - 1] = 0;
  }
  return 1;
}

template <typename T>
void attach(device_matrix<T>& m, int64_t h, int64_t w, void* p, int64_t ld)
{
  m.Attach(h, w, static_cast<T*>(p), ld);
}

template <typename W>
void copy_out(void* dst, const device_matrix<W>& src, hipStream_t st)
{
  if (!dst || src.IsEmpty()) return;
  check_hip(hipMemcpy2DAsync(dst, static_cast<size_t>(src.Height()) * sizeof(W), src.LockedBuffer(),
                             static_cast<size_t>(src.LDim()) * sizeof(W), static_cast<size_t>(src.Height()) * sizeof(W),
                             static_cast<size_t>(src.Width()), hipMemcpyDeviceToDevice, st),
            "copy_out");
}

template <typename T>
int run_layer_norm(const int64_t* dims, int nd, int start_dim, int scale, int bias, double eps, int64_t h,
                   int64_t w, int64_t ld, void* x, void* y, void* dy, void* dx, const void* gw,
                   const void* bw, void* dg, void* db, void* stats_out, void* sgrad_out, void* stream)
{
  using W = typename layer_norm_layer<T>::weight_t;  // float, or double for a layer of doubles
  layer_norm_layer<T> layer(eps, scale != 0, bias != 0, start_dim);
  layer.setup(std::vector<int64_t>(dims, dims + nd));
  device_matrix<T> mx, my, mdy, mdx;
  attach(mx, h, w, x, ld); attach(my, h, w, y, ld); attach(mdy, h, w, dy, ld); attach(mdx, h, w, dx, ld);
  layer.io.prev_activations = &mx; layer.io.activations = &my;
  layer.io.prev_error_signals = &mdy; layer.io.error_signals = &mdx;
  layer.io.stream = static_cast<hipStream_t>(stream);
  layer.set_weights(static_cast<const W*>(gw), static_cast<const W*>(bw));
  layer.set_weight_gradients(static_cast<W*>(dg), static_cast<W*>(db));
  layer.fp_compute();
  layer.bp_compute();
  copy_out(stats_out, layer.m_statistics, layer.io.stream);
  copy_out(sgrad_out, layer.m_statistics_gradient, layer.io.stream);
  check_hip(hipStreamSynchronize(layer.io.stream), "sync");  // owned statistics die with the layer
  return 0;
}

}  // namespace

template <typename T>
static int run_batch_norm(const int64_t* dims, int nd, double decay, double eps, int bessel, int training,
                          int64_t h, int64_t w, int64_t ld, void* x, void* y, void* dy, void* dx,
                          const void* gw, const void* bw, void* rmean, void* rvar, void* dg, void* db,
                          void* mean_var_out, void* mean_var_grad_out, void* stream)
{
  using W = typename batch_normalization_layer<T>::weight_t;
  batch_normalization_layer<T> layer(decay, eps, 1, bessel != 0);
  layer.setup(std::vector<int64_t>(dims, dims + nd));
  layer.is_training = training != 0;
  device_matrix<T> mx, my, mdy, mdx;
  attach(mx, h, w, static_cast<T*>(x), ld); attach(my, h, w, static_cast<T*>(y), ld);
  attach(mdy, h, w, static_cast<T*>(dy), ld); attach(mdx, h, w, static_cast<T*>(dx), ld);
  layer.io.prev_activations = &mx; layer.io.activations = &my;
  layer.io.prev_error_signals = &mdy; layer.io.error_signals = &mdx;
  layer.io.stream = static_cast<hipStream_t>(stream);
  layer.set_weights(static_cast<const W*>(gw), static_cast<const W*>(bw), static_cast<W*>(rmean), static_cast<W*>(rvar));
  layer.set_weight_gradients(static_cast<W*>(dg), static_cast<W*>(db));
  layer.fp_compute();
  layer.bp_compute();
  copy_out(mean_var_out, layer.m_mean_and_var, layer.io.stream);
  copy_out(mean_var_grad_out, layer.m_mean_and_var_gradient, layer.io.stream);
  check_hip(hipStreamSynchronize(layer.io.stream), "sync");
  return 0;
}

extern "C" {

// half: 0 fp32, 1 fp16 storage, 2 double (weights, statistics and gradients are doubles then)
int drv_layer_norm(int half, const int64_t* dims, int nd, int start_dim, int scale, int bias, double eps,
                   int64_t h, int64_t w, int64_t ld, void* x, void* y, void* dy, void* dx, const void* gw,
                   const void* bw, void* dg, void* db, void* stats_out, void* sgrad_out, void* stream,
                   char* err, int errlen)
{
  try {
    if (half == 2)
      return run_layer_norm<double>(dims, nd, start_dim, scale, bias, eps, h, w, ld, x, y, dy, dx, gw, bw,
                                    dg, db, stats_out, sgrad_out, stream);
    if (half)
      return run_layer_norm<uint16_t>(dims, nd, start_dim, scale, bias, eps, h, w, ld, x, y, dy, dx, gw, bw,
                                      dg, db, stats_out, sgrad_out, stream);
    return run_layer_norm<float>(dims, nd, start_dim, scale, bias, eps, h, w, ld, x, y, dy, dx, gw, bw, dg, db,
                                 stats_out, sgrad_out, stream);
  }
  catch (const std::exception& e) {
    return fail(e, err, errlen);
  }
}

int drv_batch_norm(int half, const int64_t* dims, int nd, double decay, double eps, int bessel, int training,
                   int64_t h, int64_t w, int64_t ld, void* x, void* y, void* dy, void* dx, const void* gw,
                   const void* bw, void* rmean, void* rvar, void* dg, void* db, void* mean_var_out,
                   void* mean_var_grad_out, void* stream, char* err, int errlen)
{
  try {
    if (half == 2)
      return run_batch_norm<double>(dims, nd, decay, eps, bessel, training, h, w, ld, x, y, dy, dx, gw, bw,
                                    rmean, rvar, dg, db, mean_var_out, mean_var_grad_out, stream);
    if (half)
      return run_batch_norm<uint16_t>(dims, nd, decay, eps, bessel, training, h, w, ld, x, y, dy, dx, gw, bw,
                                      rmean, rvar, dg, db, mean_var_out, mean_var_grad_out, stream);
    return run_batch_norm<float>(dims, nd, decay, eps, bessel, training, h, w, ld, x, y, dy, dx, gw, bw, rmean,
                                 rvar, dg, db, mean_var_out, mean_var_grad_out, stream);
  }
  catch (const std::exception& e) {
    return fail(e, err, errlen);
  }
}

// kind: 0 softmax, 1 log-softmax, 2 channelwise softmax (dims/dim/single_dim_mode used)
int drv_softmax_family(int kind, const int64_t* dims, int nd, int64_t dim, int single_dim_mode, int64_t h,
                       int64_t w, int64_t ld, float* x, float* y, float* dy, float* dx, void* stream,
                       char* err, int errlen)
{
  try {
    device_matrix<float> mx, my, mdy, mdx;
    attach(mx, h, w, x, ld); attach(my, h, w, y, ld); attach(mdy, h, w, dy, ld); attach(mdx, h, w, dx, ld);
    auto bind = [&](auto& layer) {
      layer.io.prev_activations = &mx; layer.io.activations = &my;
      layer.io.prev_error_signals = &mdy; layer.io.error_signals = &mdx;
      layer.io.stream = static_cast<hipStream_t>(stream);
      layer.fp_compute();
      layer.bp_compute();
      check_hip(hipStreamSynchronize(layer.io.stream), "sync");  // the layer's scratch dies with it
    };
    if (kind == 0) { softmax_layer<> l; bind(l); }
    else if (kind == 1) { log_softmax_layer<> l; bind(l); }
    else {
      channelwise_softmax_layer<> l(dim, single_dim_mode != 0);
      l.setup(std::vector<int64_t>(dims, dims + nd));
      bind(l);
    }
    return 0;
  }
  catch (const std::exception& e) {
    return fail(e, err, errlen);
  }
}

// The softmax family on matrices of doubles (kind as above).
int drv_softmax_family_f64(int kind, const int64_t* dims, int nd, int64_t dim, int single_dim_mode, int64_t h,
                           int64_t w, int64_t ld, double* x, double* y, double* dy, double* dx, void* stream,
                           char* err, int errlen)
{
  try {
    using M = device_matrix<double>;
    M mx, my, mdy, mdx;
    attach(mx, h, w, x, ld); attach(my, h, w, y, ld); attach(mdy, h, w, dy, ld); attach(mdx, h, w, dx, ld);
    auto bind = [&](auto& layer) {
      layer.io.prev_activations = &mx; layer.io.activations = &my;
      layer.io.prev_error_signals = &mdy; layer.io.error_signals = &mdx;
      layer.io.stream = static_cast<hipStream_t>(stream);
      layer.fp_compute();
      layer.bp_compute();
      check_hip(hipStreamSynchronize(layer.io.stream), "sync");
    };
    if (kind == 0) { softmax_layer<M> l; bind(l); }
    else if (kind == 1) { log_softmax_layer<M> l; bind(l); }
    else {
      channelwise_softmax_layer<M> l(dim, single_dim_mode != 0);
      l.setup(std::vector<int64_t>(dims, dims + nd));
      bind(l);
    }
    return 0;
  }
  catch (const std::exception& e) {
    return fail(e, err, errlen);
  }
}

int drv_instance_norm(const int64_t* dims, int nd, double eps, int64_t h, int64_t w, int64_t ld, float* x,
                      float* y, float* dy, float* dx, void* stream, char* err, int errlen)
{
  try {
    instance_norm_layer<> layer(eps);
    layer.setup(std::vector<int64_t>(dims, dims + nd));
    device_matrix<float> mx, my, mdy, mdx;
    attach(mx, h, w, x, ld); attach(my, h, w, y, ld); attach(mdy, h, w, dy, ld); attach(mdx, h, w, dx, ld);
    layer.io.prev_activations = &mx; layer.io.activations = &my;
    layer.io.prev_error_signals = &mdy; layer.io.error_signals = &mdx;
    layer.io.stream = static_cast<hipStream_t>(stream);
    layer.fp_compute();
    layer.bp_compute();
    check_hip(hipStreamSynchronize(layer.io.stream), "sync");
    return 0;
  }
  catch (const std::exception& e) {
    return fail(e, err, errlen);
  }
}

int drv_entrywise_batch_norm(const int64_t* dims, int nd, double decay, double eps, int training, int64_t h,
                             int64_t w, int64_t ld, float* x, float* y, float* dy, float* dx, float* rmean,
                             float* rvar, float* stats_out, float* sgrad_out, void* stream, char* err,
                             int errlen)
{
  try {
    entrywise_batch_normalization_layer<> layer(decay, eps);
    layer.setup(std::vector<int64_t>(dims, dims + nd));
    layer.is_training = training != 0;
    layer.set_weights(rmean, rvar);
    device_matrix<float> mx, my, mdy, mdx;
    attach(mx, h, w, x, ld); attach(my, h, w, y, ld); attach(mdy, h, w, dy, ld); attach(mdx, h, w, dx, ld);
    layer.io.prev_activations = &mx; layer.io.activations = &my;
    layer.io.prev_error_signals = &mdy; layer.io.error_signals = &mdx;
    layer.io.stream = static_cast<hipStream_t>(stream);
    layer.fp_compute();
    layer.bp_compute();
    copy_out(stats_out, layer.m_batch_statistics, layer.io.stream);
    copy_out(sgrad_out, layer.m_batch_statistics_gradient, layer.io.stream);
    check_hip(hipStreamSynchronize(layer.io.stream), "sync");
    return 0;
  }
  catch (const std::exception& e) {
    return fail(e, err, errlen);
  }
}

// One mini-batch of w columns held by two ranks (columns [0, w0) and [w0, w)), each with its
// own layer object and running statistics (rmean2 / rvar2: two vectors of h floats each).  The
// all-reduce hook of a rank computes the other rank's local sums through the C ABI and adds
// them with the gradient-buffer kernel, which is what the collective would leave behind.
int drv_entrywise_batch_norm_two_ranks(const int64_t* dims, int nd, double decay, double eps, int64_t h,
                                       int64_t w, int64_t w0, int64_t ld, float* x, float* y, float* dy,
                                       float* dx, float* rmean2, float* rvar2, float* stats_out, void* stream,
                                       char* err, int errlen)
{
  try {
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int64_t first[2] = {0, w0}, count[2] = {w0, w - w0};
    for (int me = 0; me < 2; ++me) {
      const int other = 1 - me;
      entrywise_batch_normalization_layer<> layer(decay, eps);
      layer.setup(std::vector<int64_t>(dims, dims + nd));
      layer.set_weights(rmean2 + me * h, rvar2 + me * h);
      device_matrix<float> mx, my, mdy, mdx, peer(h, 2);
      attach(mx, h, count[me], x + first[me] * ld, ld); attach(my, h, count[me], y + first[me] * ld, ld);
      attach(mdy, h, count[me], dy + first[me] * ld, ld); attach(mdx, h, count[me], dx + first[me] * ld, ld);
      layer.io.prev_activations = &mx; layer.io.activations = &my;
      layer.io.prev_error_signals = &mdy; layer.io.error_signals = &mdx;
      layer.io.stream = st;
      int phase = 0;
      layer.set_statistics_allreduce(
        [&](device_matrix<float>& m) {
          const float* px = x + first[other] * ld;
          const float* pdy = dy + first[other] * ld;
          if (phase == 0)
            check_status(lbn_entrywise_batch_norm_fwd_sums_f32(st, h, count[other], px, ld, peer.Buffer(), peer.LDim()),
                         "peer sums");
          else
            check_status(lbn_entrywise_batch_norm_bwd_sums_f32(st, h, count[other], static_cast<float>(eps), px, ld, pdy,
                                                               ld, layer.m_batch_statistics.LockedBuffer(),
                                                               layer.m_batch_statistics.LDim(), peer.Buffer(),
                                                               peer.LDim()),
                         "peer gradient sums");
          check_status(lbn_gradient_sink_f32(st, h, 2, 1.f, 1.f, peer.LockedBuffer(), peer.LDim(), m.Buffer(), m.LDim()),
                       "sum over ranks");
          ++phase;
        },
        w);
      layer.fp_compute();
      layer.bp_compute();
      if (phase != (w > 1 ? 2 : 1)) throw exception("all-reduce hook called an unexpected number of times");
      if (me == 0) copy_out(stats_out, layer.m_batch_statistics, st);
      check_hip(hipStreamSynchronize(st), "sync");
    }
    return 0;
  }
  catch (const std::exception& e) {
    return fail(e, err, errlen);
  }
}

int drv_cross_entropy(const int64_t* pred_dims, const int64_t* truth_dims, int nd, int use_labels, int64_t h,
                      int64_t ht, int64_t w, float* x, float* truth, float* loss, float* dloss, float* dx,
                      float* dtruth, void* stream, char* err, int errlen)
{
  try {
    cross_entropy_layer<> layer(use_labels != 0);
    layer.setup(std::vector<int64_t>(pred_dims, pred_dims + nd), std::vector<int64_t>(truth_dims, truth_dims + nd));
    device_matrix<float> mx, mt, ml, mdl, mdx, mdt;
    attach(mx, h, w, x, h); attach(mt, ht, w, truth, ht); attach(ml, 1, w, loss, 1); attach(mdl, 1, w, dloss, 1);
    attach(mdx, h, w, dx, h); attach(mdt, ht, w, dtruth, ht);
    layer.io.prev_activations = &mx; layer.prev_ground_truth = &mt; layer.io.activations = &ml;
    layer.io.prev_error_signals = &mdl; layer.io.error_signals = &mdx; layer.ground_truth_error_signals = &mdt;
    layer.io.stream = static_cast<hipStream_t>(stream);
    layer.fp_compute();
    layer.bp_compute();
    check_hip(hipStreamSynchronize(layer.io.stream), "sync");
    return 0;
  }
  catch (const std::exception& e) {
    return fail(e, err, errlen);
  }
}

// softmax followed by cross entropy through the fused forward, then both layers' backward
// (fused_bwd: as one call, which leaves dy untouched)
int drv_softmax_cross_entropy(const int64_t* pred_dims, const int64_t* truth_dims, int nd, int use_labels, int64_t h,
                              int64_t ht, int64_t w, float* x, float* y, float* truth, float* loss, float* dloss,
                              float* dy, float* dx, float* dtruth, int fused_bwd, void* stream, char* err, int errlen)
{
  try {
    softmax_layer<> sm;
    cross_entropy_layer<> ce(use_labels != 0);
    ce.setup(std::vector<int64_t>(pred_dims, pred_dims + nd), std::vector<int64_t>(truth_dims, truth_dims + nd));
    device_matrix<float> mx, my, mt, ml, mdl, mdy, mdx, mdt;
    attach(mx, h, w, x, h); attach(my, h, w, y, h); attach(mt, ht, w, truth, ht); attach(ml, 1, w, loss, 1);
    attach(mdl, 1, w, dloss, 1); attach(mdy, h, w, dy, h); attach(mdx, h, w, dx, h); attach(mdt, ht, w, dtruth, ht);
    sm.io.prev_activations = &mx; sm.io.activations = &my; sm.io.prev_error_signals = &mdy; sm.io.error_signals = &mdx;
    ce.io.prev_activations = &my; ce.prev_ground_truth = &mt; ce.io.activations = &ml;
    ce.io.prev_error_signals = &mdl; ce.io.error_signals = &mdy; ce.ground_truth_error_signals = &mdt;
    sm.io.stream = ce.io.stream = static_cast<hipStream_t>(stream);
    ce.fp_compute_with(sm);
    if (fused_bwd) {
      ce.bp_compute_with(sm);
    }
    else {
      ce.bp_compute();
      sm.bp_compute();
    }
    sm.check_cluster_waits();
    check_hip(hipStreamSynchronize(sm.io.stream), "sync");
    return 0;
  }
  catch (const std::exception& e) {
    return fail(e, err, errlen);
  }
}

// kind: 0 entry-wise, 1 channel-wise.  weights: (n x 2) column-major, n = h resp. dims[0].
int drv_scale_bias(int kind, const int64_t* dims, int nd, int64_t h, int64_t w, int64_t ld, float* x, float* y,
                   float* dy, float* dx, const float* weights, int64_t ld_weights, float* wgrad_out,
                   void* stream, char* err, int errlen)
{
  try {
    device_matrix<float> mx, my, mdy, mdx;
    attach(mx, h, w, x, ld); attach(my, h, w, y, ld); attach(mdy, h, w, dy, ld); attach(mdx, h, w, dx, ld);
    auto run = [&](auto& layer) {
      layer.setup(std::vector<int64_t>(dims, dims + nd));
      layer.set_weights(weights, ld_weights);
      layer.io.prev_activations = &mx; layer.io.activations = &my;
      layer.io.prev_error_signals = &mdy; layer.io.error_signals = &mdx;
      layer.io.stream = static_cast<hipStream_t>(stream);
      layer.fp_compute();
      layer.bp_compute();
      copy_out(wgrad_out, layer.m_weights_gradient, layer.io.stream);
      check_hip(hipStreamSynchronize(layer.io.stream), "sync");
    };
    if (kind == 0) { entrywise_scale_bias_layer<> l; run(l); }
    else { channelwise_scale_bias_layer<> l; run(l); }
    return 0;
  }
  catch (const std::exception& e) {
    return fail(e, err, errlen);
  }
}


// Host-only checks of the error behaviour the reference has: returns the number of
// cases that did NOT throw as they should.
// Channel-wise scale/bias backward twice on the same inputs, the weight gradient handed to an
// attached gradient buffer each time with factors `scale0`, `scale1`: gradient_out (C x 2)
// ends as scale0 * dW + scale1 * dW, statuses[k] the buffer's status after step k.
int drv_gradient_buffer(const int64_t* dims, int nd, int64_t h, int64_t w, const float* x, const float* dy,
                        float* dx, const float* weights, float* gradient_out, int64_t ld_gradient, float scale0,
                        float scale1, int* statuses, void* stream, char* err, int errlen)
{
  try {
    channelwise_scale_bias_layer<> layer;
    layer.setup(std::vector<int64_t>(dims, dims + nd));
    layer.set_weights(weights, dims[0]);
    device_matrix<float> mx, mdy, mdx;
    mx.Attach(h, w, const_cast<float*>(x), h);
    mdy.Attach(h, w, const_cast<float*>(dy), h);
    mdx.Attach(h, w, dx, h);
    layer.io.stream = static_cast<hipStream_t>(stream);
    layer.io.prev_activations = &mx;
    layer.io.prev_error_signals = &mdy;
    layer.io.error_signals = &mdx;
    gradient_buffer sink;
    sink.attach(dims[0], 2, gradient_out, ld_gradient);
    const float scales[2] = {scale0, scale1};
    for (int k = 0; k < 2; ++k) {
      layer.bp_compute();
      sink.add_to_gradient(stream, layer.m_weights_gradient, scales[k], k == 1);
      statuses[k] = static_cast<int>(sink.get_status());
    }
    return 0;
  } catch (const std::exception& e) {
    return fail(e, err, errlen);
  }
}

// fp16 storage through the adapter: a matrix type with 2-byte elements selects the _f16 entry
// points.  kind: 0 softmax, 1 log-softmax.
int drv_softmax_family_f16(int kind, int64_t h, int64_t w, int64_t ld, void* x, void* y, void* dy, void* dx,
                           void* stream, char* err, int errlen)
{
  try {
    using half_bits = unsigned short;
    device_matrix<half_bits> mx, my, mdy, mdx;
    attach(mx, h, w, x, ld); attach(my, h, w, y, ld); attach(mdy, h, w, dy, ld); attach(mdx, h, w, dx, ld);
    auto bind = [&](auto& layer) {
      layer.io.prev_activations = &mx; layer.io.activations = &my;
      layer.io.prev_error_signals = &mdy; layer.io.error_signals = &mdx;
      layer.io.stream = static_cast<hipStream_t>(stream);
      layer.fp_compute();
      layer.bp_compute();
      check_hip(hipStreamSynchronize(layer.io.stream), "sync");
    };
    if (kind == 0) { softmax_layer<device_matrix<half_bits>> l; bind(l); }
    else { log_softmax_layer<device_matrix<half_bits>> l; bind(l); }
    return 0;
  }
  catch (const std::exception& e) {
    return fail(e, err, errlen);
  }
}

// Cross entropy with fp16 storage (dense ground truth): 2-byte elements select the _f16 entry points.
int drv_cross_entropy_f16(const int64_t* dims, int nd, int64_t h, int64_t w, void* x, void* truth, void* loss,
                          void* dloss, void* dx, void* dtruth, void* stream, char* err, int errlen)
{
  try {
    using half_bits = unsigned short;
    using M = device_matrix<half_bits>;
    cross_entropy_layer<M> layer(false);
    layer.setup(std::vector<int64_t>(dims, dims + nd), std::vector<int64_t>(dims, dims + nd));
    M mx, mt, ml, mdl, mdx, mdt;
    attach(mx, h, w, x, h); attach(mt, h, w, truth, h); attach(ml, 1, w, loss, 1); attach(mdl, 1, w, dloss, 1);
    attach(mdx, h, w, dx, h); attach(mdt, h, w, dtruth, h);
    layer.io.prev_activations = &mx; layer.prev_ground_truth = &mt; layer.io.activations = &ml;
    layer.io.prev_error_signals = &mdl; layer.io.error_signals = &mdx; layer.ground_truth_error_signals = &mdt;
    layer.io.stream = static_cast<hipStream_t>(stream);
    layer.fp_compute();
    layer.bp_compute();
    check_hip(hipStreamSynchronize(layer.io.stream), "sync");
    return 0;
  }
  catch (const std::exception& e) {
    return fail(e, err, errlen);
  }
}

// A softmax layer on a (h x w) problem that uses scratch: forward, then the wait check, which
// must pass; then the designed give-up exit is run on the layer's own scratch buffer and
// the next check must throw (returns 0 only if it did, with the message in err), after which
// the word is clear again and a further forward + check pass.
int drv_cluster_wait_check(int64_t h, int64_t w, float* x, float* y, float* out4, void* stream, char* err,
                           int errlen)
{
  try {
    device_matrix<float> mx, my;
    attach(mx, h, w, x, h); attach(my, h, w, y, h);
    softmax_layer<> layer;
    layer.io.prev_activations = &mx; layer.io.activations = &my;
    layer.io.stream = static_cast<hipStream_t>(stream);
    layer.fp_compute();
    layer.check_cluster_waits();
    if (layer.scratch().bytes() < 128) throw exception("the test shape was expected to use scratch");
    check_status(lbn_selftest_cluster_wait_gives_up(stream, layer.scratch().reserve(0), layer.scratch().bytes(), 32,
                                                    out4), "selftest");
    bool thrown = false;
    try {
      layer.check_cluster_waits();
    }
    catch (const exception& e) {
      thrown = true;
      std::snprintf(err, errlen, "%s", e.what());
    }
    if (!thrown) throw exception("check_cluster_waits() did not report the wait that gave up");
    layer.fp_compute();
    layer.check_cluster_waits();
    check_hip(hipStreamSynchronize(layer.io.stream), "sync");
    return 0;
  }
  catch (const std::exception& e) {
    return fail(e, err, errlen);
  }
}

int drv_error_cases(void)
{
  int missed = 0;
  {
    // the gradient buffer's status machine (optimizer_impl.hpp:262-287), no device touched
    gradient_buffer b;
    float bs = -1.f, is = -1.f;
    using S = optimizer_gradient_status;
    if (b.get_status() != S::cleared) ++missed;
    b.get_gradient_scales(bs, is, false);
    if (bs != 0.f || is != 1.f || b.get_status() != S::ready) ++missed;
    b.get_gradient_scales(bs, is, true);
    if (bs != 1.f || is != 1.f || b.get_status() != S::sync_needed) ++missed;
    b.get_gradient_scales(bs, is, false);
    if (bs != 1.f || is != 1.f || b.get_status() != S::sync_needed) ++missed;
    b.clear();
    b.get_gradient_scales(bs, is, true);
    if (bs != 0.f || b.get_status() != S::sync_needed) ++missed;
    b.set_status(S::sync_started);
    try { b.get_gradient_scales(bs, is, false); ++missed; } catch (const exception&) {}
    device_matrix<float> wrong;
    wrong.Attach(3, 1, nullptr, 3);
    gradient_buffer c;
    c.attach(4, 1, nullptr, 4);
    try { c.add_to_gradient(nullptr, wrong); ++missed; } catch (const exception&) {}
  }
  try { softmax_layer<> l(softmax_mode::CHANNEL); ++missed; } catch (const exception&) {}
  try { layer_norm_layer<float> l(1e-5, false, false, 2); l.setup({4, 4}); ++missed; } catch (const exception&) {}
  try { layer_norm_layer<float> l(1e-5, false, false, -3); l.setup({4, 4}); ++missed; } catch (const exception&) {}
  try { channelwise_softmax_layer<> l(3, false); l.setup({2, 3, 4}); ++missed; } catch (const exception&) {}
  try { channelwise_softmax_layer<> l(1, false); l.setup({2, 3, 4}); ++missed; } catch (const exception&) {}
  try { batch_normalization_layer<> l(0.9, 1e-5, 0, true); ++missed; } catch (const exception&) {}
  { batch_normalization_layer<uint16_t> half_storage(0.9, 1e-5, 1, true); (void)half_storage; }
  // cross entropy with labels: ground truth must be (1, spatial...) matching the prediction's spatial dims
  try { cross_entropy_layer<> l(true); l.setup({3, 8, 8}, {2, 8, 8}); ++missed; } catch (const exception&) {}
  try { cross_entropy_layer<> l(true); l.setup({3}, {1}); ++missed; } catch (const exception&) {}
  try { cross_entropy_layer<> l(true); l.setup({3, 8, 8}, {1, 8, 4}); ++missed; } catch (const exception&) {}
  try { cross_entropy_layer<> l(false); l.setup({3, 8}, {3, 4}); ++missed; } catch (const exception&) {}
  { cross_entropy_layer<> l(true); l.setup({3, 4, 4, 4}, {1, 4, 4, 4}); }
  {
    layer_norm_layer<float> l(1e-5, true, true, -1);
    l.setup({31, 2, 5});
    int64_t n, gn, G, s;
    l.get_normdims(n, gn, G, s);
    if (n != 5 || G != 62 || s != 5 || gn != 5) ++missed;
    channelwise_softmax_layer<> c(-1, true);
    c.setup({5, 2, 7});
    int64_t cs, st, C;
    c.get_channel_size_and_stride(cs, st, C);
    if (cs != 7 || st != 7 || C != 10) ++missed;
  }
  return missed;
}

}  // extern "C"
