// Header-only C++ adapter: the five LBANN layer classes' fp_compute()/bp_compute()
// bodies, written against the C ABI of include/lbnorm.h.
//
// The classes keep the reference's names, constructor parameters, member matrices
// and error behaviour (a thrown exception where the reference calls LBANN_ERROR), so
// that each body can replace the corresponding GPU specialisation in LBANN:
//   layer_norm_layer            src/layers/regularizers/layer_norm.cu  (fp_compute/bp_compute)
//   batch_normalization_layer   src/layers/regularizers/batch_normalization.cu
//   softmax_layer               src/layers/activations/softmax.cu      (data-parallel branch)
//   log_softmax_layer           src/layers/activations/log_softmax.cu
//   channelwise_softmax_layer   src/layers/misc/channelwise_softmax.cu
// and, beyond those five, instance_norm_layer, entrywise_batch_normalization_layer,
// cross_entropy_layer, entrywise_scale_bias_layer and channelwise_scale_bias_layer,
// and gradient_buffer, where their weight gradients go (optimizer::add_to_gradient).
//
// `Mat` is any local-matrix type with the El::Matrix<T, El::Device::GPU> accessors
//   Height(), Width(), LDim(), Buffer(), LockedBuffer()
// (El::Matrix itself inside LBANN; lbnorm::device_matrix below elsewhere).  The
// adapter never touches matrix contents on the host and never synchronises.
#pragma once

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdint>
#include <cstdlib>
#include <functional>
#include <numeric>
#include <stdexcept>
#include <string>
#include <type_traits>
#include <utility>
#include <vector>

#include "../../include/lbnorm.h"

namespace lbnorm {

/// Thrown where the reference throws lbann::exception through LBANN_ERROR.
struct exception : std::runtime_error {
  using std::runtime_error::runtime_error;
};

inline void check_status(int status, const char* where)
{
  if (status != LBN_OK)
    throw exception(std::string(where) + ": " + lbn_status_string(status) + " (status " +
                    std::to_string(status) + ")");
}

inline void check_hip(hipError_t e, const char* where)
{
  if (e != hipSuccess) throw exception(std::string(where) + ": " + hipGetErrorString(e));
}

/// Column-major device matrix with El::Matrix's accessor names.  Owns its memory
/// unless attached to an existing buffer.
template <typename T>
class device_matrix {
public:
  device_matrix() = default;
  device_matrix(int64_t height, int64_t width) { Resize(height, width); }
  device_matrix(const device_matrix&) = delete;
  device_matrix& operator=(const device_matrix&) = delete;
  ~device_matrix() { release(); }

  /// View of memory owned by someone else (El::Matrix::Attach / LockedAttach).
  void Attach(int64_t height, int64_t width, T* buffer, int64_t ldim)
  {
    release();
    m_h = height; m_w = width; m_ld = ldim; m_buf = buffer; m_owned = false;
  }
  void Resize(int64_t height, int64_t width)
  {
    if (m_owned && m_buf && height * width <= m_capacity) {
      m_h = height; m_w = width; m_ld = height > 0 ? height : 1;
      return;
    }
    release();
    m_h = height; m_w = width; m_ld = height > 0 ? height : 1;
    m_capacity = height * width;
    if (m_capacity > 0) {
      void* p = nullptr;
      check_hip(hipMalloc(&p, static_cast<size_t>(m_capacity) * sizeof(T)), "device_matrix::Resize");
      m_buf = static_cast<T*>(p);
      m_owned = true;
    }
  }
  int64_t Height() const { return m_h; }
  int64_t Width() const { return m_w; }
  int64_t LDim() const { return m_ld; }
  T* Buffer() { return m_buf; }
  const T* LockedBuffer() const { return m_buf; }
  bool IsEmpty() const { return m_h < 1 || m_w < 1; }

private:
  void release()
  {
    if (m_owned && m_buf) (void)hipFree(m_buf);
    m_buf = nullptr; m_owned = false; m_capacity = 0;
  }
  int64_t m_h = 0, m_w = 0, m_ld = 1, m_capacity = 0;
  T* m_buf = nullptr;
  bool m_owned = false;
};

namespace detail {
/// LBN_CHECK_CLUSTER_WAITS=1 in the environment: every compute hook checks its workspace's
/// error word right after the call (this waits for the stream: a debugging mode).
inline bool check_every_call()
{
  static const bool on = [] {
    const char* v = std::getenv("LBN_CHECK_CLUSTER_WAITS");
    return v && *v && *v != '0';
  }();
  return on;
}
inline bool stream_is_capturing(hipStream_t st)
{
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(st, &status) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  return status != hipStreamCaptureStatusNone;
}
}  // namespace detail

/// Scratch buffer a layer owns (the role of the reference's m_workspace members).
///
/// The compute hooks only enqueue kernels as long as the buffer is large enough; it grows
/// (hipFree + hipMalloc, which wait for the device) when a larger mini-batch arrives.  A
/// caller that must not hit that inside a step, or that records its step into a HIP graph,
/// sizes it up front: `layer.scratch().reserve(bytes, stream)` with the *_workspace_bytes()
/// of its largest mini-batch.  Growing while the stream records is refused.
///
/// The first 64 bytes hold the error word of the kernels that wait across workgroups; they
/// are cleared when the buffer is allocated, and check() turns a raised word into an
/// exception: call it (through the layer's check_cluster_waits()) where a step's results are
/// consumed; it waits for the stream.
class workspace {
public:
  workspace() = default;
  workspace(const workspace&) = delete;
  workspace& operator=(const workspace&) = delete;
  ~workspace() { if (m_buf) (void)hipFree(m_buf); }
  void* reserve(size_t bytes, hipStream_t stream = nullptr)
  {
    if (bytes > m_bytes) {
      if (detail::stream_is_capturing(stream))
        throw exception("workspace::reserve: the scratch buffer would have to grow (" + std::to_string(m_bytes) +
                        " -> " + std::to_string(bytes) + " bytes) while the stream records a graph; "
                        "reserve it before recording");
      if (m_buf) (void)hipFree(m_buf);
      m_buf = nullptr;
      m_bytes = 0;
      const size_t alloc = bytes < 64 ? 64 : bytes;
      check_hip(hipMalloc(&m_buf, alloc), "workspace::reserve");
      check_hip(hipMemsetAsync(m_buf, 0, 64, stream), "workspace::reserve (clearing the header)");
      m_bytes = alloc;
    }
    return m_buf;
  }
  size_t bytes() const { return m_bytes; }
  /// Throws if a wait between workgroups ran out in a call that used this buffer; clears the
  /// word so that the next call starts clean.  Waits for `stream`.
  void check(hipStream_t stream, const char* where)
  {
    if (!m_buf) return;
    int timed_out = 0;
    check_status(lbn_workspace_timed_out(stream, m_buf, &timed_out), where);
    if (timed_out) {
      check_hip(hipMemsetAsync(m_buf, 0, 64, stream), where);
      throw exception(std::string(where) + ": a bounded wait between workgroups ran out; the results of that "
                      "call are undefined");
    }
  }
  /// The debugging mode's check after every call (not while the stream is being captured into
  /// a HIP graph: the check waits for the device).
  void after_call(hipStream_t stream, const char* where)
  {
    if (detail::check_every_call() && !detail::stream_is_capturing(stream)) check(stream, where);
  }

private:
  void* m_buf = nullptr;
  size_t m_bytes = 0;
};

/// What data_type_layer hands to the compute hooks: the four local matrices and the
/// stream of their SyncInfo.
template <typename Mat>
struct layer_io {
  const Mat* prev_activations = nullptr;    // get_prev_activations().LockedMatrix()
  Mat* activations = nullptr;               // get_activations().Matrix()
  const Mat* prev_error_signals = nullptr;  // get_prev_error_signals().LockedMatrix()
  Mat* error_signals = nullptr;             // get_error_signals().Matrix()
  hipStream_t stream = nullptr;
};

namespace detail {
inline int64_t product(const std::vector<int64_t>& d, size_t from, size_t to)
{
  int64_t p = 1;
  for (size_t i = from; i < to; ++i) p *= d[i];
  return p;
}
template <typename T> struct is_half : std::false_type {};
/// Element type of a matrix class (what Buffer() points to): 2-byte elements select the
/// fp16-storage entry points.
template <typename Mat>
using element_t = std::remove_cv_t<std::remove_pointer_t<decltype(std::declval<Mat&>().Buffer())>>;
}  // namespace detail

// ------------------------------------------------------------------ layer norm
/// include/lbann/layers/regularizers/layer_norm.hpp:53-143.  T is float, a 16-bit
/// storage type (any 2-byte IEEE binary16 type) for the fp16-storage kernels, or double
/// (TensorDataType = double: statistics, weights and their gradients are doubles too).
template <typename T, typename Mat = device_matrix<T>>
class layer_norm_layer {
public:
  /// Type of statistics, weights and weight gradients: float unless the layer is one of doubles.
  using weight_t = std::conditional_t<sizeof(T) == 8, double, float>;
  layer_norm_layer(double epsilon = 1e-5, bool scale = false, bool bias = false, int start_dim = 0)
    : m_epsilon(epsilon), m_scale(scale), m_bias(bias), m_start_dim(start_dim) {}

  /// setup_dims + setup_data: fixes the normalised dimensions (layer_norm.hpp:259-290).
  void setup(const std::vector<int64_t>& dims)
  {
    m_dims = dims;
    const int nd = static_cast<int>(dims.size());
    const int sd = m_start_dim >= 0 ? m_start_dim : nd + m_start_dim;
    if (sd < 0 || sd >= nd)
      throw exception("Layer normalization start dimension " + std::to_string(m_start_dim) +
                      " does not match the input tensor dimensionality of " + std::to_string(nd));
    m_sd = sd;
  }
  /// get_normdims (layer_norm.hpp:362-405), data-parallel layout.
  void get_normdims(int64_t& normalization_size, int64_t& global_normalization_size,
                    int64_t& num_normalized, int64_t& normalization_stride) const
  {
    num_normalized = detail::product(m_dims, 0, m_sd);
    normalization_size = detail::product(m_dims, m_sd, m_dims.size());
    normalization_stride = normalization_size;
    global_normalization_size = normalization_size;
  }
  /// Weight values (weights_values(i).LockedMatrix().LockedBuffer()) and gradient sinks.
  void set_weights(const weight_t* scale, const weight_t* bias) { m_scale_w = scale; m_bias_w = bias; }
  void set_weight_gradients(weight_t* dscale, weight_t* dbias) { m_scale_grad = dscale; m_bias_grad = dbias; }

  layer_io<Mat> io;
  device_matrix<weight_t> m_statistics;           // 2*num_normalized x width: means, then variances
  device_matrix<weight_t> m_statistics_gradient;  // same shape: dL/dmean, dL/dvar
  int stats_mode = LBN_STATS_TWO_PASS;

  /// layer_norm.cpp:263-290 / layer_norm.cu fp_compute.
  void fp_compute()
  {
    const Mat& x = *io.prev_activations;
    Mat& y = *io.activations;
    int64_t n, gn, G, stride;
    get_normdims(n, gn, G, stride);
    m_statistics.Resize(2 * G, x.Width());
    const weight_t* sw = m_scale ? m_scale_w : nullptr;
    const weight_t* bw = m_bias ? m_bias_w : nullptr;
    int st;
    if constexpr (sizeof(T) == 8) {
      st = lbn_layer_norm_fwd_f64(io.stream, G, n, stride, x.Width(), m_epsilon,
                                  reinterpret_cast<const double*>(x.LockedBuffer()), x.LDim(),
                                  reinterpret_cast<double*>(y.Buffer()), y.LDim(), m_statistics.Buffer(),
                                  m_statistics.LDim(), sw, bw, stats_mode);
    }
    else {
      // scratch is only needed (and only non-zero) for groups of tens of thousands of entries
      const size_t bytes = lbn_layer_norm_fwd_workspace_bytes(G, n, x.Width(), static_cast<int>(sizeof(T)));
      void* ws = m_ws.reserve(bytes, io.stream);
      const float eps = static_cast<float>(m_epsilon);
      if constexpr (sizeof(T) == 2)
        st = lbn_layer_norm_fwd_f16(io.stream, G, n, stride, x.Width(), eps, x.LockedBuffer(), x.LDim(),
                                    y.Buffer(), y.LDim(), m_statistics.Buffer(), m_statistics.LDim(), sw, bw,
                                    ws, bytes, stats_mode);
      else
        st = lbn_layer_norm_fwd_f32(io.stream, G, n, stride, x.Width(), eps,
                                    reinterpret_cast<const float*>(x.LockedBuffer()), x.LDim(),
                                    reinterpret_cast<float*>(y.Buffer()), y.LDim(), m_statistics.Buffer(),
                                    m_statistics.LDim(), sw, bw, ws, bytes, stats_mode);
    }
    check_status(st, "layer_norm_layer::fp_compute");
    m_ws.after_call(io.stream, "layer_norm_layer::fp_compute");
  }

  /// layer_norm.cpp:292-348 / layer_norm.cu bp_compute.  The weight gradients are
  /// overwritten (the reference zeroes them first, :300-309); handing them to the
  /// optimizer (add_to_gradient, :330-347) stays with the caller.
  void bp_compute()
  {
    const Mat& x = *io.prev_activations;
    const Mat& dy = *io.prev_error_signals;
    Mat& dx = *io.error_signals;
    int64_t n, gn, G, stride;
    get_normdims(n, gn, G, stride);
    m_statistics_gradient.Resize(2 * G, x.Width());
    const weight_t* sw = m_scale ? m_scale_w : nullptr;
    weight_t* dsw = m_scale ? m_scale_grad : nullptr;
    weight_t* dbw = m_bias ? m_bias_grad : nullptr;
    int st;
    if constexpr (sizeof(T) == 8) {
      const size_t bytes = lbn_layer_norm_bwd_workspace_bytes_f64(G, n, x.Width(), (dsw || dbw) ? 1 : 0);
      void* ws = m_ws.reserve(bytes, io.stream);
      st = lbn_layer_norm_bwd_f64(io.stream, G, n, stride, x.Width(), m_epsilon,
                                  reinterpret_cast<const double*>(x.LockedBuffer()), x.LDim(),
                                  reinterpret_cast<const double*>(dy.LockedBuffer()), dy.LDim(),
                                  reinterpret_cast<double*>(dx.Buffer()), dx.LDim(),
                                  m_statistics.LockedBuffer(), m_statistics.LDim(),
                                  m_statistics_gradient.Buffer(), m_statistics_gradient.LDim(), sw, dsw, dbw,
                                  ws, bytes);
    }
    else {
      const size_t bytes = lbn_layer_norm_bwd_workspace_bytes(G, n, x.Width(), (dsw || dbw) ? 1 : 0,
                                                              static_cast<int>(sizeof(T)));
      void* ws = m_ws.reserve(bytes, io.stream);
      const float eps = static_cast<float>(m_epsilon);
      if constexpr (sizeof(T) == 2)
        st = lbn_layer_norm_bwd_f16(io.stream, G, n, stride, x.Width(), eps, x.LockedBuffer(), x.LDim(),
                                    dy.LockedBuffer(), dy.LDim(), dx.Buffer(), dx.LDim(),
                                    m_statistics.LockedBuffer(), m_statistics.LDim(),
                                    m_statistics_gradient.Buffer(), m_statistics_gradient.LDim(), sw, dsw, dbw,
                                    ws, bytes);
      else
        st = lbn_layer_norm_bwd_f32(io.stream, G, n, stride, x.Width(), eps,
                                    reinterpret_cast<const float*>(x.LockedBuffer()), x.LDim(),
                                    reinterpret_cast<const float*>(dy.LockedBuffer()), dy.LDim(),
                                    reinterpret_cast<float*>(dx.Buffer()), dx.LDim(),
                                    m_statistics.LockedBuffer(), m_statistics.LDim(),
                                    m_statistics_gradient.Buffer(), m_statistics_gradient.LDim(), sw, dsw, dbw,
                                    ws, bytes);
    }
    check_status(st, "layer_norm_layer::bp_compute");
    m_ws.after_call(io.stream, "layer_norm_layer::bp_compute");
  }

  /// The layer's scratch buffer (reserve it up front to keep the hooks free of allocation).
  workspace& scratch() { return m_ws; }
  /// Throws if a wait between workgroups ran out in a call of this layer since the last
  /// check; waits for the stream.  Call where a step's results are consumed.
  void check_cluster_waits()
  {
    m_ws.check(io.stream, "check_cluster_waits");
  }

private:
  double m_epsilon;
  bool m_scale, m_bias;
  int m_start_dim, m_sd = 0;
  std::vector<int64_t> m_dims;
  const weight_t* m_scale_w = nullptr;
  const weight_t* m_bias_w = nullptr;
  weight_t* m_scale_grad = nullptr;
  weight_t* m_bias_grad = nullptr;
  workspace m_ws;
};

// ------------------------------------------------------------------ batch norm
/// include/lbann/layers/regularizers/batch_normalization.hpp:130-199 with local
/// statistics (statistics_group_size == 1).  T is the storage type of the activations
/// and error signals: float, or a 2-byte type holding IEEE binary16 (statistics and
/// weights are float for both), or double (statistics and weights are doubles as well).
template <typename T = float, typename Mat = device_matrix<T>>
class batch_normalization_layer {
  static_assert(sizeof(T) == 8 || sizeof(T) == 4 || sizeof(T) == 2, "fp64, fp32 or fp16 storage");
public:
  using weight_t = std::conditional_t<sizeof(T) == 8, double, float>;
  batch_normalization_layer(double decay = 0.9, double epsilon = 1e-5, int statistics_group_size = 1,
                            bool bessel_correction = true)
    : m_decay(decay), m_epsilon(epsilon),
      m_statistics_group_size(statistics_group_size), m_bessel_correction(bessel_correction)
  {
    if (statistics_group_size != 1)
      throw exception("batch_normalization_layer: only local statistics (statistics_group_size == 1) "
                      "run on one GPU; aggregate with the lbn_batch_norm_*_sums/_stats/_apply entry points");
  }
  void setup(const std::vector<int64_t>& dims)
  {
    m_dims = dims;
    m_num_channels = dims.at(0);
    m_channel_size = detail::product(dims, 1, dims.size());
    m_mean_and_var.Resize(m_num_channels, 2);
    m_mean_and_var_gradient.Resize(m_num_channels, 2);
  }
  /// weights 0..3: scale, bias, running mean, running variance (all device pointers).
  void set_weights(const weight_t* scale, const weight_t* bias, weight_t* running_mean, weight_t* running_var)
  {
    m_w[0] = const_cast<weight_t*>(scale); m_w[1] = const_cast<weight_t*>(bias);
    m_w[2] = running_mean; m_w[3] = running_var;
  }
  void set_weight_gradients(weight_t* dscale, weight_t* dbias) { m_scale_grad = dscale; m_bias_grad = dbias; }

  layer_io<Mat> io;
  bool is_training = true;                           // execution_mode::training
  device_matrix<weight_t> m_mean_and_var;            // C x 2: column 0 mean, column 1 variance
  device_matrix<weight_t> m_mean_and_var_gradient;   // C x 2
  int stats_mode = LBN_STATS_TWO_PASS;

  void fp_compute()
  {
    const Mat& x = *io.prev_activations;
    Mat& y = *io.activations;
    const size_t bytes = workspace_bytes(x.Width());
    void* ws = m_ws.reserve(bytes, io.stream);
    weight_t* mv = m_mean_and_var.Buffer();
    int st;
    if constexpr (sizeof(T) == 8) {
      st = lbn_batch_norm_fwd_f64(io.stream, m_num_channels, m_channel_size, x.Width(),
                                  m_bessel_correction ? 1 : 0, m_epsilon, m_decay, is_training ? 1 : 0,
                                  reinterpret_cast<const double*>(x.LockedBuffer()), x.LDim(),
                                  reinterpret_cast<double*>(y.Buffer()), y.LDim(), mv,
                                  mv + m_mean_and_var.LDim(), m_w[0], m_w[1], m_w[2], m_w[3], ws, bytes,
                                  stats_mode);
    }
    else {
      const float eps = static_cast<float>(m_epsilon), decay = static_cast<float>(m_decay);
      if constexpr (sizeof(T) == 2)
        st = lbn_batch_norm_fwd_f16(io.stream, m_num_channels, m_channel_size, x.Width(),
                                    m_bessel_correction ? 1 : 0, eps, decay, is_training ? 1 : 0,
                                    x.LockedBuffer(), x.LDim(), y.Buffer(), y.LDim(), mv,
                                    mv + m_mean_and_var.LDim(), m_w[0], m_w[1], m_w[2], m_w[3], ws, bytes,
                                    stats_mode);
      else
        st = lbn_batch_norm_fwd_f32(io.stream, m_num_channels, m_channel_size, x.Width(),
                                    m_bessel_correction ? 1 : 0, eps, decay, is_training ? 1 : 0,
                                    reinterpret_cast<const float*>(x.LockedBuffer()), x.LDim(),
                                    reinterpret_cast<float*>(y.Buffer()), y.LDim(), mv,
                                    mv + m_mean_and_var.LDim(), m_w[0], m_w[1], m_w[2], m_w[3], ws, bytes,
                                    stats_mode);
    }
    check_status(st, "batch_normalization_layer::fp_compute");
    m_ws.after_call(io.stream, "batch_normalization_layer::fp_compute");
  }
  void bp_compute()
  {
    const Mat& x = *io.prev_activations;
    const Mat& dy = *io.prev_error_signals;
    Mat& dx = *io.error_signals;
    const size_t bytes = workspace_bytes(x.Width());
    void* ws = m_ws.reserve(bytes, io.stream);
    const weight_t* mv = m_mean_and_var.LockedBuffer();
    weight_t* mvg = m_mean_and_var_gradient.Buffer();
    int st;
    if constexpr (sizeof(T) == 8) {
      st = lbn_batch_norm_bwd_f64(io.stream, m_num_channels, m_channel_size, x.Width(),
                                  m_bessel_correction ? 1 : 0, m_epsilon, is_training ? 1 : 0,
                                  reinterpret_cast<const double*>(x.LockedBuffer()), x.LDim(),
                                  reinterpret_cast<const double*>(dy.LockedBuffer()), dy.LDim(),
                                  reinterpret_cast<double*>(dx.Buffer()), dx.LDim(), mv,
                                  mv + m_mean_and_var.LDim(), m_w[2], m_w[3], m_w[0], m_scale_grad,
                                  m_bias_grad, mvg, mvg + m_mean_and_var_gradient.LDim(), ws, bytes);
    }
    else {
      const float eps = static_cast<float>(m_epsilon);
      if constexpr (sizeof(T) == 2)
        st = lbn_batch_norm_bwd_f16(io.stream, m_num_channels, m_channel_size, x.Width(),
                                    m_bessel_correction ? 1 : 0, eps, is_training ? 1 : 0,
                                    x.LockedBuffer(), x.LDim(), dy.LockedBuffer(), dy.LDim(), dx.Buffer(),
                                    dx.LDim(), mv, mv + m_mean_and_var.LDim(), m_w[2], m_w[3], m_w[0],
                                    m_scale_grad, m_bias_grad, mvg, mvg + m_mean_and_var_gradient.LDim(), ws,
                                    bytes);
      else
        st = lbn_batch_norm_bwd_f32(io.stream, m_num_channels, m_channel_size, x.Width(),
                                    m_bessel_correction ? 1 : 0, eps, is_training ? 1 : 0,
                                    reinterpret_cast<const float*>(x.LockedBuffer()), x.LDim(),
                                    reinterpret_cast<const float*>(dy.LockedBuffer()), dy.LDim(),
                                    reinterpret_cast<float*>(dx.Buffer()), dx.LDim(), mv,
                                    mv + m_mean_and_var.LDim(), m_w[2], m_w[3], m_w[0], m_scale_grad,
                                    m_bias_grad, mvg, mvg + m_mean_and_var_gradient.LDim(), ws, bytes);
    }
    check_status(st, "batch_normalization_layer::bp_compute");
    m_ws.after_call(io.stream, "batch_normalization_layer::bp_compute");
  }

  /// The layer's scratch buffer (reserve it up front to keep the hooks free of allocation).
  workspace& scratch() { return m_ws; }
  /// Throws if a wait between workgroups ran out in a call of this layer since the last
  /// check; waits for the stream.  Call where a step's results are consumed.
  void check_cluster_waits()
  {
    m_ws.check(io.stream, "check_cluster_waits");
  }

private:
  size_t workspace_bytes(int64_t width) const
  {
    return sizeof(T) == 8 ? lbn_batch_norm_workspace_bytes_f64(m_num_channels, m_channel_size, width)
                          : lbn_batch_norm_workspace_bytes(m_num_channels, m_channel_size, width);
  }
  double m_decay, m_epsilon;
  int m_statistics_group_size;
  bool m_bessel_correction;
  std::vector<int64_t> m_dims;
  int64_t m_num_channels = 0, m_channel_size = 0;
  weight_t* m_w[4] = {nullptr, nullptr, nullptr, nullptr};
  weight_t* m_scale_grad = nullptr;
  weight_t* m_bias_grad = nullptr;
  workspace m_ws;
};

// --------------------------------------------------------- softmax / log-softmax
enum class softmax_mode { INVALID, INSTANCE, CHANNEL };

/// include/lbann/layers/activations/softmax.hpp:85-262, data-parallel layout.
template <typename Mat = device_matrix<float>>
class softmax_layer {
public:
  explicit softmax_layer(softmax_mode mode = softmax_mode::INSTANCE) : m_mode(mode)
  {
    // the CPU reference rejects everything else (dnn_lib/openmp/softmax.hpp:61-63)
    if (mode != softmax_mode::INSTANCE) throw exception("Unsupported softmax mode");
  }
  layer_io<Mat> io;
  void fp_compute()
  {
    const Mat& x = *io.prev_activations;
    Mat& y = *io.activations;
    if constexpr (sizeof(detail::element_t<Mat>) == 8) {  // TensorDataType = double: no scratch
      check_status(lbn_softmax_fwd_f64(io.stream, x.Height(), x.Width(),
                                       reinterpret_cast<const double*>(x.LockedBuffer()), x.LDim(),
                                       reinterpret_cast<double*>(y.Buffer()), y.LDim()),
                   "softmax_layer::fp_compute");
      return;
    }
    const size_t bytes = lbn_softmax_workspace_bytes(x.Height(), x.Width());
    const auto fwd = sizeof(detail::element_t<Mat>) == 2 ? &lbn_softmax_fwd_f16 : &call_f32_fwd;
    check_status(fwd(io.stream, x.Height(), x.Width(), x.LockedBuffer(), x.LDim(), y.Buffer(), y.LDim(),
                     m_ws.reserve(bytes, io.stream), bytes),
                 "softmax_layer::fp_compute");
    m_ws.after_call(io.stream, "softmax_layer::fp_compute");
  }
  void bp_compute()
  {
    const Mat& y = *io.activations;
    const Mat& dy = *io.prev_error_signals;
    Mat& dx = *io.error_signals;
    if constexpr (sizeof(detail::element_t<Mat>) == 8) {
      check_status(lbn_softmax_bwd_f64(io.stream, y.Height(), y.Width(),
                                       reinterpret_cast<const double*>(y.LockedBuffer()), y.LDim(),
                                       reinterpret_cast<const double*>(dy.LockedBuffer()), dy.LDim(),
                                       reinterpret_cast<double*>(dx.Buffer()), dx.LDim()),
                   "softmax_layer::bp_compute");
      return;
    }
    const size_t bytes = lbn_softmax_workspace_bytes(y.Height(), y.Width());
    const auto bwd = sizeof(detail::element_t<Mat>) == 2 ? &lbn_softmax_bwd_f16 : &call_f32_bwd;
    check_status(bwd(io.stream, y.Height(), y.Width(), y.LockedBuffer(), y.LDim(), dy.LockedBuffer(), dy.LDim(),
                     dx.Buffer(), dx.LDim(), m_ws.reserve(bytes, io.stream), bytes),
                 "softmax_layer::bp_compute");
    m_ws.after_call(io.stream, "softmax_layer::bp_compute");
  }
  /// The layer's scratch buffer (reserve it up front to keep the hooks free of allocation).
  workspace& scratch() { return m_ws; }
  /// Throws if a wait between workgroups ran out in a call of this layer since the last
  /// check; waits for the stream.  Call where a step's results are consumed.
  void check_cluster_waits()
  {
    m_ws.check(io.stream, "check_cluster_waits");
  }

private:
  // the fp32 entry points behind the pointer types of the fp16 ones
  static int call_f32_fwd(lbn_stream_t st, int64_t h, int64_t w, const void* x, int64_t ldx, void* y, int64_t ldy,
                          void* ws, size_t bytes)
  {
    return lbn_softmax_fwd_f32(st, h, w, static_cast<const float*>(x), ldx, static_cast<float*>(y), ldy, ws, bytes);
  }
  static int call_f32_bwd(lbn_stream_t st, int64_t h, int64_t w, const void* y, int64_t ldy, const void* dy,
                          int64_t lddy, void* dx, int64_t lddx, void* ws, size_t bytes)
  {
    return lbn_softmax_bwd_f32(st, h, w, static_cast<const float*>(y), ldy, static_cast<const float*>(dy), lddy,
                               static_cast<float*>(dx), lddx, ws, bytes);
  }
  softmax_mode m_mode;
  workspace m_ws;
};

/// include/lbann/layers/activations/log_softmax.hpp.
template <typename Mat = device_matrix<float>>
class log_softmax_layer {
public:
  layer_io<Mat> io;
  void fp_compute()
  {
    const Mat& x = *io.prev_activations;
    Mat& y = *io.activations;
    if constexpr (sizeof(detail::element_t<Mat>) == 8) {  // TensorDataType = double: no scratch
      check_status(lbn_log_softmax_fwd_f64(io.stream, x.Height(), x.Width(),
                                       reinterpret_cast<const double*>(x.LockedBuffer()), x.LDim(),
                                       reinterpret_cast<double*>(y.Buffer()), y.LDim()),
                   "log_softmax_layer::fp_compute");
      return;
    }
    const size_t bytes = lbn_softmax_workspace_bytes(x.Height(), x.Width());
    const auto fwd = sizeof(detail::element_t<Mat>) == 2 ? &lbn_log_softmax_fwd_f16 : &call_f32_fwd;
    check_status(fwd(io.stream, x.Height(), x.Width(), x.LockedBuffer(), x.LDim(), y.Buffer(), y.LDim(),
                     m_ws.reserve(bytes, io.stream), bytes),
                 "log_softmax_layer::fp_compute");
    m_ws.after_call(io.stream, "log_softmax_layer::fp_compute");
  }
  void bp_compute()
  {
    const Mat& y = *io.activations;
    const Mat& dy = *io.prev_error_signals;
    Mat& dx = *io.error_signals;
    if constexpr (sizeof(detail::element_t<Mat>) == 8) {
      check_status(lbn_log_softmax_bwd_f64(io.stream, y.Height(), y.Width(),
                                       reinterpret_cast<const double*>(y.LockedBuffer()), y.LDim(),
                                       reinterpret_cast<const double*>(dy.LockedBuffer()), dy.LDim(),
                                       reinterpret_cast<double*>(dx.Buffer()), dx.LDim()),
                   "log_softmax_layer::bp_compute");
      return;
    }
    const size_t bytes = lbn_softmax_workspace_bytes(y.Height(), y.Width());
    const auto bwd = sizeof(detail::element_t<Mat>) == 2 ? &lbn_log_softmax_bwd_f16 : &call_f32_bwd;
    check_status(bwd(io.stream, y.Height(), y.Width(), y.LockedBuffer(), y.LDim(), dy.LockedBuffer(), dy.LDim(),
                     dx.Buffer(), dx.LDim(), m_ws.reserve(bytes, io.stream), bytes),
                 "log_softmax_layer::bp_compute");
    m_ws.after_call(io.stream, "log_softmax_layer::bp_compute");
  }
  /// The layer's scratch buffer (reserve it up front to keep the hooks free of allocation).
  workspace& scratch() { return m_ws; }
  /// Throws if a wait between workgroups ran out in a call of this layer since the last
  /// check; waits for the stream.  Call where a step's results are consumed.
  void check_cluster_waits()
  {
    m_ws.check(io.stream, "check_cluster_waits");
  }

private:
  static int call_f32_fwd(lbn_stream_t st, int64_t h, int64_t w, const void* x, int64_t ldx, void* y, int64_t ldy,
                          void* ws, size_t bytes)
  {
    return lbn_log_softmax_fwd_f32(st, h, w, static_cast<const float*>(x), ldx, static_cast<float*>(y), ldy, ws, bytes);
  }
  static int call_f32_bwd(lbn_stream_t st, int64_t h, int64_t w, const void* y, int64_t ldy, const void* dy,
                          int64_t lddy, void* dx, int64_t lddx, void* ws, size_t bytes)
  {
    return lbn_log_softmax_bwd_f32(st, h, w, static_cast<const float*>(y), ldy, static_cast<const float*>(dy), lddy,
                                   static_cast<float*>(dx), lddx, ws, bytes);
  }
  workspace m_ws;
};

// --------------------------------------------------------- channelwise softmax
/// include/lbann/layers/misc/channelwise_softmax.hpp:50-107.
template <typename Mat = device_matrix<float>>
class channelwise_softmax_layer {
public:
  channelwise_softmax_layer(int64_t dim = 0, bool single_dim_mode = false)
    : m_dim(dim), m_single_dim_mode(single_dim_mode) {}

  /// setup_dims (channelwise_softmax_impl.hpp:33-56)
  void setup(const std::vector<int64_t>& dims)
  {
    const int64_t nd = static_cast<int64_t>(dims.size());
    if (m_dim < -nd || m_dim >= nd)
      throw exception("Dimension " + std::to_string(m_dim) + " is out of bounds for Channelwise Softmax layer on tensor with " +
                      std::to_string(nd) + " dimensions.");
    if (!m_single_dim_mode && m_dim != 0 && m_dim != -nd && m_dim != nd - 1 && m_dim != -1)
      throw exception("Channelwise softmax with all dimensions is only supported for the first or last tensor dimensions. Got dimension " +
                      std::to_string(m_dim));
    m_dims = dims;
  }
  /// channelwise_softmax_impl.hpp:58-104
  void get_channel_size_and_stride(int64_t& channel_size, int64_t& channel_stride, int64_t& num_channels) const
  {
    const int64_t nd = static_cast<int64_t>(m_dims.size());
    const int64_t dim = m_dim < 0 ? m_dim + nd : m_dim;
    const int64_t total = detail::product(m_dims, 0, m_dims.size());
    if (m_single_dim_mode) {
      channel_size = m_dims[dim];
      num_channels = total / channel_size;
      channel_stride = detail::product(m_dims, dim, m_dims.size());
    }
    else {
      channel_size = total / m_dims[dim];
      num_channels = m_dims[dim];
      channel_stride = dim == 0 ? channel_size : 1;
    }
  }
  layer_io<Mat> io;
  void fp_compute()
  {
    const Mat& x = *io.prev_activations;
    Mat& y = *io.activations;
    int64_t cs, stride, C;
    get_channel_size_and_stride(cs, stride, C);
    if constexpr (sizeof(detail::element_t<Mat>) == 8) {  // TensorDataType = double: no scratch
      check_status(lbn_channelwise_softmax_fwd_f64(io.stream, C, cs, stride, x.Width(), x.LockedBuffer(), x.LDim(),
                                                   y.Buffer(), y.LDim()),
                   "channelwise_softmax_layer::fp_compute");
      return;
    }
    else {
      const size_t bytes = lbn_channelwise_softmax_workspace_bytes(C, cs, x.Width());
      check_status(lbn_channelwise_softmax_fwd_f32(io.stream, C, cs, stride, x.Width(), x.LockedBuffer(), x.LDim(),
                                                   y.Buffer(), y.LDim(), m_ws.reserve(bytes, io.stream), bytes),
                   "channelwise_softmax_layer::fp_compute");
    }
    m_ws.after_call(io.stream, "channelwise_softmax_layer::fp_compute");
  }
  void bp_compute()
  {
    const Mat& y = *io.activations;
    const Mat& dy = *io.prev_error_signals;
    Mat& dx = *io.error_signals;
    int64_t cs, stride, C;
    get_channel_size_and_stride(cs, stride, C);
    if constexpr (sizeof(detail::element_t<Mat>) == 8) {
      check_status(lbn_channelwise_softmax_bwd_f64(io.stream, C, cs, stride, y.Width(), y.LockedBuffer(), y.LDim(),
                                                   dy.LockedBuffer(), dy.LDim(), dx.Buffer(), dx.LDim()),
                   "channelwise_softmax_layer::bp_compute");
      return;
    }
    else {
      const size_t bytes = lbn_channelwise_softmax_workspace_bytes(C, cs, y.Width());
      check_status(lbn_channelwise_softmax_bwd_f32(io.stream, C, cs, stride, y.Width(), y.LockedBuffer(), y.LDim(),
                                                   dy.LockedBuffer(), dy.LDim(), dx.Buffer(), dx.LDim(),
                                                   m_ws.reserve(bytes, io.stream), bytes),
                   "channelwise_softmax_layer::bp_compute");
    }
    m_ws.after_call(io.stream, "channelwise_softmax_layer::bp_compute");
  }
  /// The layer's scratch buffer (reserve it up front to keep the hooks free of allocation).
  workspace& scratch() { return m_ws; }
  /// Throws if a wait between workgroups ran out in a call of this layer since the last
  /// check; waits for the stream.  Call where a step's results are consumed.
  void check_cluster_waits()
  {
    m_ws.check(io.stream, "check_cluster_waits");
  }

private:
  int64_t m_dim;
  bool m_single_dim_mode;
  std::vector<int64_t> m_dims;
  workspace m_ws;
};

// ------------------------------------------------------------------ instance norm
/// include/lbann/layers/regularizers/instance_norm.hpp:52-100.
template <typename Mat = device_matrix<float>>
class instance_norm_layer {
public:
  explicit instance_norm_layer(double epsilon = 1e-5) : m_epsilon(static_cast<float>(epsilon)) {}

  /// setup_dims (instance_norm.hpp:163-168): output dims = input dims, channels first
  void setup(const std::vector<int64_t>& dims)
  {
    if (dims.empty()) throw exception("instance norm layer needs at least one tensor dimension");
    m_dims = dims;
  }
  int64_t num_channels() const { return m_dims.front(); }
  int64_t channel_size() const { return detail::product(m_dims, 0, m_dims.size()) / m_dims.front(); }

  layer_io<Mat> io;
  /// means in rows [0,C), variances in rows [C,2C) of every column
  device_matrix<float> m_workspace;

  void fp_compute()
  {
    const Mat& x = *io.prev_activations;
    Mat& y = *io.activations;
    m_workspace.Resize(2 * num_channels(), x.Width());
    const size_t bytes = lbn_instance_norm_fwd_workspace_bytes(num_channels(), channel_size(), x.Width());
    check_status(lbn_instance_norm_fwd_f32(io.stream, num_channels(), channel_size(), x.Width(), m_epsilon,
                                           x.LockedBuffer(), x.LDim(), y.Buffer(), y.LDim(),
                                           m_workspace.Buffer(), m_workspace.LDim(), m_ws_fwd.reserve(bytes, io.stream), bytes),
                 "instance_norm_layer::fp_compute");
    m_ws_fwd.after_call(io.stream, "instance_norm_layer::fp_compute");
  }
  void bp_compute()
  {
    const Mat& x = *io.prev_activations;
    const Mat& dy = *io.prev_error_signals;
    Mat& dx = *io.error_signals;
    const size_t bytes = lbn_instance_norm_bwd_workspace_bytes(num_channels(), channel_size(), x.Width());
    check_status(lbn_instance_norm_bwd_f32(io.stream, num_channels(), channel_size(), x.Width(), m_epsilon,
                                           x.LockedBuffer(), x.LDim(), dy.LockedBuffer(), dy.LDim(),
                                           dx.Buffer(), dx.LDim(), m_workspace.LockedBuffer(),
                                           m_workspace.LDim(), m_ws.reserve(bytes, io.stream), bytes),
                 "instance_norm_layer::bp_compute");
    m_ws.after_call(io.stream, "instance_norm_layer::bp_compute");
  }
  /// The layer's scratch buffer (reserve it up front to keep the hooks free of allocation).
  workspace& scratch() { return m_ws; }
  /// Throws if a wait between workgroups ran out in a call of this layer since the last
  /// check; waits for the stream.  Call where a step's results are consumed.
  void check_cluster_waits()
  {
    m_ws_fwd.check(io.stream, "instance_norm_layer (forward scratch)");
    m_ws.check(io.stream, "check_cluster_waits");
  }

private:
  float m_epsilon;
  std::vector<int64_t> m_dims;
  workspace m_ws;      // backward: statistics gradients, then the cluster kernels' slots
  workspace m_ws_fwd;  // forward scratch (long channels only)
};

// ---------------------------------------------------------- entry-wise batch norm
/// include/lbann/layers/regularizers/entrywise_batch_normalization.hpp: statistics of
/// every tensor entry over the mini-batch; weights 0/1 are the running mean/variance.
template <typename Mat = device_matrix<float>>
class entrywise_batch_normalization_layer {
public:
  entrywise_batch_normalization_layer(double decay = 0.9, double epsilon = 1e-5)
    : m_decay(static_cast<float>(decay)), m_epsilon(static_cast<float>(epsilon)) {}

  void setup(const std::vector<int64_t>& dims)
  {
    m_size = detail::product(dims, 0, dims.size());
    m_batch_statistics.Resize(m_size, 2);
    m_batch_statistics_gradient.Resize(m_size, 2);
  }
  /// device pointers to `size` floats each
  void set_weights(float* running_mean, float* running_var) { m_w[0] = running_mean; m_w[1] = running_var; }

  /// The mini-batch spread over several ranks: `allreduce` stands for comm.allreduce(...,
  /// El::mpi::SUM) of the reference (entrywise_batch_normalization.cpp:97-100, :301-303) and
  /// must replace the (size x 2) matrix of local sums by its sum over the ranks, ordered on
  /// io.stream; `statistics_count` is the global mini-batch size (input.Width() there).
  void set_statistics_allreduce(std::function<void(device_matrix<float>&)> allreduce, int64_t statistics_count)
  {
    m_allreduce = std::move(allreduce);
    m_statistics_count = statistics_count;
  }

  layer_io<Mat> io;
  bool is_training = true;                             // execution_mode::training
  device_matrix<float> m_batch_statistics;             // size x 2: mean, variance
  device_matrix<float> m_batch_statistics_gradient;    // size x 2

  void fp_compute()
  {
    const Mat& x = *io.prev_activations;
    Mat& y = *io.activations;
    if (!m_w[0] || !m_w[1]) throw exception("entrywise_batch_normalization_layer: weights are not set");
    if (m_allreduce) {
      const char* where = "entrywise_batch_normalization_layer::fp_compute";
      device_matrix<float>& st = m_batch_statistics;
      const float* mean = m_w[0];
      const float* var = m_w[1];
      if (is_training) {
        check_status(lbn_entrywise_batch_norm_fwd_sums_f32(io.stream, x.Height(), x.Width(), x.LockedBuffer(),
                                                           x.LDim(), st.Buffer(), st.LDim()), where);
        m_allreduce(st);
        check_status(lbn_entrywise_batch_norm_fwd_stats_f32(io.stream, x.Height(), m_statistics_count, m_decay,
                                                            st.Buffer(), st.LDim(), m_w[0], m_w[1]), where);
        mean = st.LockedBuffer();
        var = st.LockedBuffer() + st.LDim();
      }
      check_status(lbn_entrywise_batch_norm_fwd_apply_f32(io.stream, x.Height(), x.Width(), m_epsilon,
                                                          x.LockedBuffer(), x.LDim(), y.Buffer(), y.LDim(), mean, var),
                   where);
      return;
    }
    const size_t bytes = lbn_entrywise_batch_norm_workspace_bytes(x.Height(), x.Width());
    check_status(lbn_entrywise_batch_norm_fwd_f32(io.stream, x.Height(), x.Width(), m_decay, m_epsilon,
                                                  is_training ? 1 : 0, x.LockedBuffer(), x.LDim(), y.Buffer(),
                                                  y.LDim(), m_batch_statistics.Buffer(),
                                                  m_batch_statistics.LDim(), m_w[0], m_w[1],
                                                  bytes ? m_ws.reserve(bytes, io.stream) : nullptr, bytes),
                 "entrywise_batch_normalization_layer::fp_compute");
  }
  void bp_compute()
  {
    const Mat& x = *io.prev_activations;
    const Mat& dy = *io.prev_error_signals;
    Mat& dx = *io.error_signals;
    if (m_allreduce && is_training) {
      const char* where = "entrywise_batch_normalization_layer::bp_compute";
      device_matrix<float>& st = m_batch_statistics;
      device_matrix<float>& sg = m_batch_statistics_gradient;
      if (m_statistics_count > 1) {
        check_status(lbn_entrywise_batch_norm_bwd_sums_f32(io.stream, x.Height(), x.Width(), m_epsilon,
                                                           x.LockedBuffer(), x.LDim(), dy.LockedBuffer(), dy.LDim(),
                                                           st.LockedBuffer(), st.LDim(), sg.Buffer(), sg.LDim()),
                     where);
        m_allreduce(sg);
      }
      check_status(lbn_entrywise_batch_norm_bwd_apply_f32(io.stream, x.Height(), x.Width(), m_statistics_count,
                                                          m_epsilon, x.LockedBuffer(), x.LDim(), dy.LockedBuffer(),
                                                          dy.LDim(), dx.Buffer(), dx.LDim(), st.LockedBuffer(),
                                                          st.LDim(), sg.LockedBuffer(), sg.LDim()),
                   where);
      return;
    }
    const size_t bytes = lbn_entrywise_batch_norm_workspace_bytes(x.Height(), x.Width());
    check_status(lbn_entrywise_batch_norm_bwd_f32(io.stream, x.Height(), x.Width(), m_epsilon,
                                                  is_training ? 1 : 0, x.LockedBuffer(), x.LDim(),
                                                  dy.LockedBuffer(), dy.LDim(), dx.Buffer(), dx.LDim(),
                                                  m_batch_statistics.LockedBuffer(), m_batch_statistics.LDim(),
                                                  m_batch_statistics_gradient.Buffer(),
                                                  m_batch_statistics_gradient.LDim(), m_w[1],
                                                  bytes ? m_ws.reserve(bytes, io.stream) : nullptr, bytes),
                 "entrywise_batch_normalization_layer::bp_compute");
  }
  /// The layer's scratch buffer (partial sums of wide mini-batches; reserve it up front to
  /// keep the hooks free of allocation).
  workspace& scratch() { return m_ws; }
private:
  workspace m_ws;
  float m_decay, m_epsilon;
  int64_t m_size = 0;
  float* m_w[2] = {nullptr, nullptr};
  std::function<void(device_matrix<float>&)> m_allreduce;
  int64_t m_statistics_count = 0;
};

// ------------------------------------------------------------------ cross entropy
/// include/lbann/layers/loss/cross_entropy.hpp:75-190.  Two parents: the prediction
/// (io.prev_activations) and the ground truth (prev_ground_truth); the output is the
/// layer's 1 x width workspace matrix, which the reference sums across ranks and copies
/// into its activations (cross_entropy_impl.hpp:186-201).  bp_compute() reads the
/// gradient w.r.t. that row from io.prev_error_signals and writes io.error_signals
/// (w.r.t. the prediction) and, without use_labels, ground_truth_error_signals.
template <typename Mat = device_matrix<float>>
class cross_entropy_layer {
public:
  explicit cross_entropy_layer(bool use_labels = false) : m_use_labels(use_labels) {}

  /// setup_dims (cross_entropy_impl.hpp:39-155): the two inputs' dimensions
  void setup(const std::vector<int64_t>& prediction_dims, const std::vector<int64_t>& ground_truth_dims)
  {
    if (m_use_labels) {
      if (ground_truth_dims.empty() || ground_truth_dims[0] != 1)
        throw exception("cross entropy layer expects the 0-th dimension of the tensor to be 1 when use labels is enabled.");
      if (prediction_dims.size() != ground_truth_dims.size() || prediction_dims.size() < 2)
        throw exception("cross entropy layer expects both input tensors to have the same number of dimensions and have >2 "
                        "dimensions when use_labels is enabled.");
      if (!std::equal(prediction_dims.begin() + 1, prediction_dims.end(), ground_truth_dims.begin() + 1))
        throw exception("cross entropy layer expects both input tensors to have the same shape after the 0-th dimesion when "
                        "use_labels is enabled.");
    }
    else if (prediction_dims != ground_truth_dims) {
      throw exception("cross entropy layer has input tensors with different dimensions");
    }
    m_spatial_sample_size = detail::product(prediction_dims, 1, prediction_dims.size());
  }

  layer_io<Mat> io;
  const Mat* prev_ground_truth = nullptr;       // get_local_prev_activations(1)
  Mat* ground_truth_error_signals = nullptr;    // get_local_error_signals(1); unused with use_labels

  void fp_compute()
  {
    const Mat& x = *io.prev_activations;
    const Mat& t = *prev_ground_truth;
    Mat& loss = *io.activations;
    const size_t bytes = lbn_cross_entropy_fwd_workspace_bytes(x.Height(), x.Width());
    // the reference instantiates the layer for half precision too (cross_entropy.cpp:157-166)
    int status;
    if constexpr (sizeof(detail::element_t<Mat>) == 2)
      status = lbn_cross_entropy_fwd_f16(io.stream, x.Height(), x.Width(), m_use_labels ? 1 : 0,
                                         m_spatial_sample_size, x.LockedBuffer(), x.LDim(), t.LockedBuffer(),
                                         t.LDim(), loss.Buffer(), loss.LDim(), m_ws.reserve(bytes, io.stream), bytes);
    else
      status = lbn_cross_entropy_fwd_f32(io.stream, x.Height(), x.Width(), m_use_labels ? 1 : 0,
                                         m_spatial_sample_size, x.LockedBuffer(), x.LDim(), t.LockedBuffer(),
                                         t.LDim(), loss.Buffer(), loss.LDim(), m_ws.reserve(bytes, io.stream), bytes);
    check_status(status, "cross_entropy_layer::fp_compute");
  }
  /// fp_compute() of `sm`, a softmax layer whose output is this layer's prediction
  /// (sm.io.activations == io.prev_activations), and this layer's own, as one call: the
  /// results of sm.fp_compute() followed by fp_compute().  fp32 storage.
  void fp_compute_with(softmax_layer<Mat>& sm)
  {
    static_assert(sizeof(detail::element_t<Mat>) == 4, "the fused forward takes fp32 matrices");
    if (sm.io.activations != io.prev_activations)
      throw exception("cross_entropy_layer::fp_compute_with: the softmax layer's output is not this layer's prediction");
    const Mat& x = *sm.io.prev_activations;
    Mat& y = *sm.io.activations;
    const Mat& t = *prev_ground_truth;
    Mat& loss = *io.activations;
    const size_t bytes = lbn_softmax_cross_entropy_fwd_workspace_bytes(x.Height(), x.Width());
    check_status(lbn_softmax_cross_entropy_fwd_f32(sm.io.stream, x.Height(), x.Width(), m_use_labels ? 1 : 0,
                                                   m_spatial_sample_size, x.LockedBuffer(), x.LDim(),
                                                   t.LockedBuffer(), t.LDim(), y.Buffer(), y.LDim(), loss.Buffer(),
                                                   loss.LDim(), sm.scratch().reserve(bytes, sm.io.stream), bytes),
                 "cross_entropy_layer::fp_compute_with");
    sm.scratch().after_call(sm.io.stream, "cross_entropy_layer::fp_compute_with");
  }
  /// bp_compute() of this layer and of `sm` as one call: sm.io.error_signals receives what
  /// sm.bp_compute() would write after this layer's bp_compute(), and the gradient with respect
  /// to the prediction (io.error_signals) is never written.  ground_truth_error_signals is
  /// written when it is set (dense ground truth).  fp32 storage.
  void bp_compute_with(softmax_layer<Mat>& sm)
  {
    static_assert(sizeof(detail::element_t<Mat>) == 4, "the fused backward takes fp32 matrices");
    if (sm.io.activations != io.prev_activations)
      throw exception("cross_entropy_layer::bp_compute_with: the softmax layer's output is not this layer's prediction");
    const Mat& y = *io.prev_activations;
    const Mat& t = *prev_ground_truth;
    const Mat& dloss = *io.prev_error_signals;
    Mat& dx = *sm.io.error_signals;
    Mat* dt = m_use_labels ? nullptr : ground_truth_error_signals;
    const size_t bytes = lbn_softmax_workspace_bytes(y.Height(), y.Width());
    check_status(lbn_softmax_cross_entropy_bwd_f32(sm.io.stream, y.Height(), y.Width(), m_use_labels ? 1 : 0,
                                                   m_spatial_sample_size, y.LockedBuffer(), y.LDim(),
                                                   t.LockedBuffer(), t.LDim(), dloss.LockedBuffer(), dloss.LDim(),
                                                   dx.Buffer(), dx.LDim(), dt ? dt->Buffer() : nullptr,
                                                   dt ? dt->LDim() : 0, sm.scratch().reserve(bytes, sm.io.stream), bytes),
                 "cross_entropy_layer::bp_compute_with");
    sm.scratch().after_call(sm.io.stream, "cross_entropy_layer::bp_compute_with");
  }
  void bp_compute()
  {
    const Mat& x = *io.prev_activations;
    const Mat& t = *prev_ground_truth;
    const Mat& dy = *io.prev_error_signals;
    Mat& dx = *io.error_signals;
    Mat* dt = m_use_labels ? nullptr : ground_truth_error_signals;
    int status;
    if constexpr (sizeof(detail::element_t<Mat>) == 2)
      status = lbn_cross_entropy_bwd_f16(io.stream, x.Height(), x.Width(), m_use_labels ? 1 : 0,
                                         m_spatial_sample_size, x.LockedBuffer(), x.LDim(), t.LockedBuffer(),
                                         t.LDim(), dy.LockedBuffer(), dy.LDim(), dx.Buffer(), dx.LDim(),
                                         dt ? dt->Buffer() : nullptr, dt ? dt->LDim() : 0);
    else
      status = lbn_cross_entropy_bwd_f32(io.stream, x.Height(), x.Width(), m_use_labels ? 1 : 0,
                                         m_spatial_sample_size, x.LockedBuffer(), x.LDim(), t.LockedBuffer(),
                                         t.LDim(), dy.LockedBuffer(), dy.LDim(), dx.Buffer(), dx.LDim(),
                                         dt ? dt->Buffer() : nullptr, dt ? dt->LDim() : 0);
    check_status(status, "cross_entropy_layer::bp_compute");
  }
private:
  bool m_use_labels;
  int64_t m_spatial_sample_size = 1;
  workspace m_ws;
};

// ---------------------------------------------------------- scale and bias layers
/// include/lbann/layers/learning/entrywise_scale_bias.hpp:57-203.  One weights matrix
/// (size x 2: scale, bias; the framework owns it) and m_weights_gradient of that shape.
template <typename Mat = device_matrix<float>>
class entrywise_scale_bias_layer {
public:
  void setup(const std::vector<int64_t>& dims)
  {
    m_size = detail::product(dims, 0, dims.size());
    m_weights_gradient.Resize(m_size, 2);
  }
  /// device pointer to the (size x 2) column-major weights values and their leading dimension
  void set_weights(const float* values, int64_t ldim) { m_weights = values; m_ld_weights = ldim; }

  layer_io<Mat> io;
  device_matrix<float> m_weights_gradient;

  void fp_compute()
  {
    const Mat& x = *io.prev_activations;
    Mat& y = *io.activations;
    if (!m_weights) throw exception("entrywise_scale_bias_layer: weights are not set");
    check_status(lbn_entrywise_scale_bias_fwd_f32(io.stream, x.Height(), x.Width(), x.LockedBuffer(), x.LDim(),
                                                  y.Buffer(), y.LDim(), m_weights, m_ld_weights),
                 "entrywise_scale_bias_layer::fp_compute");
  }
  void bp_compute()
  {
    const Mat& x = *io.prev_activations;
    const Mat& dy = *io.prev_error_signals;
    Mat& dx = *io.error_signals;
    if (!m_weights) throw exception("entrywise_scale_bias_layer: weights are not set");
    const size_t bytes = lbn_entrywise_scale_bias_bwd_workspace_bytes(x.Height(), x.Width());
    check_status(lbn_entrywise_scale_bias_bwd_f32(io.stream, x.Height(), x.Width(), x.LockedBuffer(), x.LDim(),
                                                  dy.LockedBuffer(), dy.LDim(), dx.Buffer(), dx.LDim(), m_weights,
                                                  m_ld_weights, m_weights_gradient.Buffer(),
                                                  m_weights_gradient.LDim(), m_ws.reserve(bytes, io.stream), bytes),
                 "entrywise_scale_bias_layer::bp_compute");
  }
private:
  int64_t m_size = 0;
  const float* m_weights = nullptr;
  int64_t m_ld_weights = 0;
  workspace m_ws;
};

/// include/lbann/layers/learning/channelwise_scale_bias.hpp:60-206.  Weights are
/// (num_channels x 2), num_channels = dims[0].
template <typename Mat = device_matrix<float>>
class channelwise_scale_bias_layer {
public:
  void setup(const std::vector<int64_t>& dims)
  {
    if (dims.empty()) throw exception("channelwise_scale_bias_layer: empty dimensions");
    m_num_channels = dims[0];
    m_channel_size = detail::product(dims, 1, dims.size());
    m_weights_gradient.Resize(m_num_channels, 2);
  }
  void set_weights(const float* values, int64_t ldim) { m_weights = values; m_ld_weights = ldim; }

  layer_io<Mat> io;
  device_matrix<float> m_weights_gradient;

  void fp_compute()
  {
    const Mat& x = *io.prev_activations;
    Mat& y = *io.activations;
    if (!m_weights) throw exception("channelwise_scale_bias_layer: weights are not set");
    check_status(lbn_channelwise_scale_bias_fwd_f32(io.stream, m_num_channels, m_channel_size, x.Width(),
                                                    x.LockedBuffer(), x.LDim(), y.Buffer(), y.LDim(), m_weights,
                                                    m_ld_weights),
                 "channelwise_scale_bias_layer::fp_compute");
  }
  void bp_compute()
  {
    const Mat& x = *io.prev_activations;
    const Mat& dy = *io.prev_error_signals;
    Mat& dx = *io.error_signals;
    if (!m_weights) throw exception("channelwise_scale_bias_layer: weights are not set");
    const size_t bytes = lbn_channelwise_scale_bias_bwd_workspace_bytes(m_num_channels, m_channel_size, x.Width());
    check_status(lbn_channelwise_scale_bias_bwd_f32(io.stream, m_num_channels, m_channel_size, x.Width(),
                                                    x.LockedBuffer(), x.LDim(), dy.LockedBuffer(), dy.LDim(),
                                                    dx.Buffer(), dx.LDim(), m_weights, m_ld_weights,
                                                    m_weights_gradient.Buffer(), m_weights_gradient.LDim(),
                                                    m_ws.reserve(bytes, io.stream), bytes),
                 "channelwise_scale_bias_layer::bp_compute");
  }
private:
  int64_t m_num_channels = 0, m_channel_size = 0;
  const float* m_weights = nullptr;
  int64_t m_ld_weights = 0;
  workspace m_ws;
};

/// Where the layers' weight gradients go: optimizer::add_to_gradient and
/// get_gradient_buffer (include/lbann/optimizers/optimizer_impl.hpp:207-288) with the
/// status values of include/lbann/optimizers/optimizer.hpp:54-70, for one process: the
/// buffer's RedundantSize is 1, so needing a synchronisation changes the status only.
/// The buffer starts cleared; the first contribution overwrites it without reading it.
enum class optimizer_gradient_status { ready, cleared, sync_needed, sync_started };

class gradient_buffer {
public:
  gradient_buffer() = default;
  gradient_buffer(int64_t height, int64_t width) { setup(height, width); }
  void setup(int64_t height, int64_t width)
  {
    m_gradient.Resize(height, width);
    m_status = optimizer_gradient_status::cleared;
  }
  /// View of a gradient matrix owned by someone else.
  void attach(int64_t height, int64_t width, float* buffer, int64_t ldim)
  {
    m_gradient.Attach(height, width, buffer, ldim);
    m_status = optimizer_gradient_status::cleared;
  }
  void clear() { m_status = optimizer_gradient_status::cleared; }
  optimizer_gradient_status get_status() const { return m_status; }
  void set_status(optimizer_gradient_status s) { m_status = s; }
  device_matrix<float>& local_gradient() { return m_gradient; }

  /// The factors for the buffer and for the contribution, and the status transition.
  void get_gradient_scales(float& buf_scale, float& in_scale, bool sync_needed)
  {
    switch (m_status) {
    case optimizer_gradient_status::ready:
      buf_scale = 1.f; in_scale = 1.f;
      if (sync_needed) m_status = optimizer_gradient_status::sync_needed;
      break;
    case optimizer_gradient_status::cleared:
      buf_scale = 0.f; in_scale = 1.f;
      m_status = sync_needed ? optimizer_gradient_status::sync_needed : optimizer_gradient_status::ready;
      break;
    case optimizer_gradient_status::sync_needed:
      buf_scale = 1.f; in_scale = 1.f;
      break;
    default:
      throw exception("unexpected gradient status (sync_started)");
    }
  }

  /// contrib: height x width values with leading dimension ldim, in device memory.
  void add_to_gradient(lbn_stream_t stream, const float* contrib, int64_t ldim, float scale = 1.f,
                       bool sync_needed = false)
  {
    float buf_scale, in_scale;
    get_gradient_scales(buf_scale, in_scale, sync_needed);
    check_status(lbn_gradient_sink_f32(stream, m_gradient.Height(), m_gradient.Width(), buf_scale,
                                       in_scale * scale, contrib, ldim, m_gradient.Buffer(), m_gradient.LDim()),
                 "gradient_buffer::add_to_gradient");
  }
  template <typename Mat>
  void add_to_gradient(lbn_stream_t stream, const Mat& contrib, float scale = 1.f, bool sync_needed = false)
  {
    if (contrib.Height() != m_gradient.Height() || contrib.Width() != m_gradient.Width())
      throw exception("gradient_buffer::add_to_gradient: contribution has the wrong shape");
    add_to_gradient(stream, contrib.LockedBuffer(), contrib.LDim(), scale, sync_needed);
  }
private:
  device_matrix<float> m_gradient;
  optimizer_gradient_status m_status = optimizer_gradient_status::cleared;
};

}  // namespace lbnorm
