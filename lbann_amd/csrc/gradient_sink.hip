// Where the weight gradients of these layers go: the optimizer's gradient buffer.
// Reference: optimizer::add_to_gradient (include/lbann/optimizers/optimizer_impl.hpp:207-217)
// does Scale(buf_scale, gradient) and then Axpy(in_scale * scale, contribution, gradient),
// with the two factors chosen from the buffer's status by get_gradient_buffer (:219-288):
// a cleared buffer is overwritten (buf_scale = 0: its old contents, possibly never
// initialised, are not read), a ready one accumulates.  One kernel does both steps:
//   gradient = buf_scale * gradient + in_scale * contribution,
// each product and the sum rounded on its own as the two library calls do.
#include "device_utils.hpp"
#include "host_utils.hpp"

namespace lbn {

constexpr int kSinkThreads = 256;

struct SinkArgs {
  int64_t h, w;
  float buf_scale, in_scale;
  const float* contrib;
  float* grad;
  int64_t ldc, ldg;
};

// Contraction is switched off in both helpers: the intrinsics are plain operators to the
// compiler, which would otherwise fuse a product into the sum and round once.
__device__ __forceinline__ float sink_value(float g, float c, float bs, float is)
{
#pragma clang fp contract(off)
  const float a = bs * g;
  const float b = is * c;
  return a + b;
}

// The zeroed buffer plus the contribution: 0 + t, so that a product of -0 is stored as +0
// as after the two library calls.
__device__ __forceinline__ float sink_fresh(float c, float is)
{
#pragma clang fp contract(off)
  const float t = is * c;
  return 0.f + t;
}

// OVERWRITE: buf_scale == 0, the gradient buffer is write-only.
template <bool OVERWRITE>
__global__ void __launch_bounds__(kSinkThreads)
grad_sink_quads(SinkArgs a)  // h % 4 == 0, 16-byte aligned columns
{
  const int64_t qh = a.h / 4;
  const int64_t total = qh * a.w;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kSinkThreads + threadIdx.x; i < total;
       i += static_cast<int64_t>(gridDim.x) * kSinkThreads) {
    const int64_t c = i / qh;
    const int64_t r = 4 * (i - c * qh);
    const float4 v = *reinterpret_cast<const float4*>(a.contrib + r + c * a.ldc);
    float4* gp = reinterpret_cast<float4*>(a.grad + r + c * a.ldg);
    float4 g = make_float4(0.f, 0.f, 0.f, 0.f);
    if (!OVERWRITE) g = *gp;
    float4 o;
    if (OVERWRITE) {
      o.x = sink_fresh(v.x, a.in_scale);
      o.y = sink_fresh(v.y, a.in_scale);
      o.z = sink_fresh(v.z, a.in_scale);
      o.w = sink_fresh(v.w, a.in_scale);
    } else {
      o.x = sink_value(g.x, v.x, a.buf_scale, a.in_scale);
      o.y = sink_value(g.y, v.y, a.buf_scale, a.in_scale);
      o.z = sink_value(g.z, v.z, a.buf_scale, a.in_scale);
      o.w = sink_value(g.w, v.w, a.buf_scale, a.in_scale);
    }
    *gp = o;
  }
}

template <bool OVERWRITE>
__global__ void __launch_bounds__(kSinkThreads)
grad_sink_scalar(SinkArgs a)
{
  const int64_t total = a.h * a.w;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kSinkThreads + threadIdx.x; i < total;
       i += static_cast<int64_t>(gridDim.x) * kSinkThreads) {
    const int64_t c = i / a.h;
    const int64_t r = i - c * a.h;
    const float v = a.contrib[r + c * a.ldc];
    float* gp = a.grad + r + c * a.ldg;
    *gp = OVERWRITE ? sink_fresh(v, a.in_scale) : sink_value(*gp, v, a.buf_scale, a.in_scale);
  }
}

}  // namespace lbn

using namespace lbn;

extern "C" int lbn_gradient_sink_f32(lbn_stream_t stream, int64_t height, int64_t width, float buf_scale,
                                     float in_scale, const float* contribution, int64_t ld_contribution,
                                     float* gradient, int64_t ld_gradient)
{
  if (height < 0 || width < 0) return LBN_ERR_INVALID_ARGUMENT;
  if (width > 1 && (ld_contribution < height || ld_gradient < height)) return LBN_ERR_INVALID_ARGUMENT;
  if (height == 0 || width == 0) return LBN_OK;
  if (!contribution || !gradient) return LBN_ERR_INVALID_ARGUMENT;
  if (height > (int64_t(1) << 40) / width) return LBN_ERR_UNSUPPORTED;
  hipStream_t st = as_stream(stream);
  SinkArgs a{height, width, buf_scale, in_scale, contribution, gradient, ld_contribution, ld_gradient};
  const bool quads = height % 4 == 0 && aligned16(contribution) && aligned16(gradient) &&
                     (width == 1 || (ld_contribution % 4 == 0 && ld_gradient % 4 == 0));
  const int64_t items = quads ? height / 4 * width : height * width;
  int64_t blocks = ceil_div(items, kSinkThreads);
  if (blocks > 4096) blocks = 4096;  // grid-stride beyond
  const dim3 grid(static_cast<unsigned>(blocks));
  const bool overwrite = buf_scale == 0.f;
  if (quads) {
    if (overwrite) hipLaunchKernelGGL(grad_sink_quads<true>, grid, dim3(kSinkThreads), 0, st, a);
    else hipLaunchKernelGGL(grad_sink_quads<false>, grid, dim3(kSinkThreads), 0, st, a);
  } else {
    if (overwrite) hipLaunchKernelGGL(grad_sink_scalar<true>, grid, dim3(kSinkThreads), 0, st, a);
    else hipLaunchKernelGGL(grad_sink_scalar<false>, grid, dim3(kSinkThreads), 0, st, a);
  }
  return launch_status();
}
