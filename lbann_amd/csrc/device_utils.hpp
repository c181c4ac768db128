// Device-side building blocks shared by every kernel: 128-bit coalesced row I/O,
// wave64 shuffle reductions, LDS cross-wave reductions, and the row -> address map
// of LBANN's column-major local matrices.  gfx950 only (64-wide wavefronts).
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cfloat>
#include <cstdint>
#include <type_traits>

namespace lbn {

constexpr int kWave = 64;

typedef float v4f __attribute__((ext_vector_type(4)));
typedef unsigned int v4u __attribute__((ext_vector_type(4)));

// Outputs are streamed with non-temporal stores: they are not read again by the kernel
// that writes them, and keeping them out of the caches leaves the Infinity Cache to the
// inputs (measured on a 196 MiB -> 196 MiB copy: 7.0 TB/s against 5.7 TB/s with plain
// stores; never slower at any footprint tried).
#ifndef LBN_NT_STORE
#define LBN_NT_STORE 1
#endif
#ifndef LBN_NT_LOAD
#define LBN_NT_LOAD 0
#endif

__device__ __forceinline__ int64_t imin64(int64_t a, int64_t b) { return a < b ? a : b; }

// ---------------------------------------------------------------------------
// A "row" is one contiguous run of n entries that is normalised on its own: a
// whole matrix column (softmax), one group of a column (layer norm with
// start_dim > 0) or one channel window (channelwise softmax).  Row r lives at
// (r % groups) * stride + (r / groups) * ld.
struct RowMap {
  int64_t groups;
  int64_t stride;
  // Column and group of a row.  Row and group counts stay below 2^31 (checked on the
  // host), so the division is a 32-bit one; whole-column rows skip it altogether.
  __device__ __forceinline__ void split(int64_t row, int64_t& col, int64_t& g) const
  {
    if (groups == 1) {
      col = row;
      g = 0;
    }
    else {
      const unsigned c = static_cast<unsigned>(row) / static_cast<unsigned>(groups);
      col = c;
      g = static_cast<unsigned>(row) - c * static_cast<unsigned>(groups);
    }
  }
  __device__ __forceinline__ int64_t offset(int64_t row, int64_t ld) const
  {
    int64_t col, g;
    split(row, col, g);
    return g * stride + col * ld;
  }
};

// Index of the calling wave inside its block, as a wave-uniform (scalar) value: row
// indices and row base addresses derived from it stay in scalar registers.
__device__ __forceinline__ int wave_index()
{
  return __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x) / kWave);
}

// ---------------------------------------------------------------------------
// 16-byte vector access for the two storage types.  Values are always widened to
// fp32 registers.
template <typename T>
struct Vec16;

template <>
struct Vec16<float> {
  static constexpr int N = 4;
  static __device__ __forceinline__ void load(const float* p, float (&v)[4])
  {
    const v4f r = LBN_NT_LOAD ? __builtin_nontemporal_load(reinterpret_cast<const v4f*>(p))
                              : *reinterpret_cast<const v4f*>(p);
    v[0] = r.x; v[1] = r.y; v[2] = r.z; v[3] = r.w;
  }
  static __device__ __forceinline__ void store(float* p, const float (&v)[4])
  {
    v4f r;
    r.x = v[0]; r.y = v[1]; r.z = v[2]; r.w = v[3];
    if (LBN_NT_STORE) __builtin_nontemporal_store(r, reinterpret_cast<v4f*>(p));
    else *reinterpret_cast<v4f*>(p) = r;
  }
  // streaming load: the line is not kept in the caches (for tensors read exactly once)
  static __device__ __forceinline__ void load_stream(const float* p, float (&v)[4])
  {
    const v4f r = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(p));
    v[0] = r.x; v[1] = r.y; v[2] = r.z; v[3] = r.w;
  }
  static __device__ __forceinline__ float load1(const float* p) { return *p; }
  static __device__ __forceinline__ void store1(float* p, float v) { *p = v; }
  // raw 16-byte register image of a vector (for software prefetch) and its widening
  using raw_t = v4f;
  static __device__ __forceinline__ raw_t load_raw(const float* p)
  {
    return LBN_NT_LOAD ? __builtin_nontemporal_load(reinterpret_cast<const v4f*>(p))
                       : *reinterpret_cast<const v4f*>(p);
  }
  static __device__ __forceinline__ void unpack(const raw_t& r, float (&v)[4])
  {
    v[0] = r.x; v[1] = r.y; v[2] = r.z; v[3] = r.w;
  }
};

// fp32 storage accessed one element at a time: for matrices whose rows start on 4-byte
// but not 16-byte boundaries (odd row lengths).  Consecutive lanes then take consecutive
// floats, so a wave instruction still reads 256 contiguous bytes.
struct f32x1 {
  float v;
};

template <>
struct Vec16<f32x1> {
  static constexpr int N = 1;
  using raw_t = float;
  static __device__ __forceinline__ raw_t load_raw(const f32x1* p) { return p->v; }
  static __device__ __forceinline__ void unpack(const raw_t& r, float (&v)[1]) { v[0] = r; }
  static __device__ __forceinline__ void load(const f32x1* p, float (&v)[1]) { v[0] = p->v; }
  static __device__ __forceinline__ void store(f32x1* p, const float (&v)[1]) { p->v = v[0]; }
  static __device__ __forceinline__ float load1(const f32x1* p) { return p->v; }
  static __device__ __forceinline__ void store1(f32x1* p, float v) { p->v = v; }
};

// fp32 storage in 16-byte accesses at addresses that are only 4-byte aligned: the hardware
// takes them (measured on a 256 MiB copy shifted by one or three floats: 5.1 TB/s against 5.5
// aligned and 4.2 with one float per access), so long rows off the 16-byte grid need no cut at
// 16-byte boundaries, only their last n % 4 entries apart.
struct f32u {
  float v;
};

template <>
struct Vec16<f32u> {
  static constexpr int N = 4;
  using raw_t = v4f;
  static __device__ __forceinline__ raw_t load_raw(const f32u* p)
  {
    v4f r;
    __builtin_memcpy(&r, p, 16);
    return r;
  }
  static __device__ __forceinline__ void unpack(const raw_t& r, float (&v)[4]) { Vec16<float>::unpack(r, v); }
  static __device__ __forceinline__ void load(const f32u* p, float (&v)[4]) { __builtin_memcpy(v, p, 16); }
  static __device__ __forceinline__ void store(f32u* p, const float (&v)[4]) { __builtin_memcpy(p, v, 16); }
  static __device__ __forceinline__ float load1(const f32u* p) { return p->v; }
  static __device__ __forceinline__ void store1(f32u* p, float v) { p->v = v; }
};

// Four consecutive floats of a weight vector beside data of storage type T: aligned like the
// data, except beside f32u data.
template <typename T>
__device__ __forceinline__ void load_weights4(const float* p, float (&w)[4])
{
  if constexpr (std::is_same<T, f32u>::value) __builtin_memcpy(w, p, 16);
  else Vec16<float>::load(p, w);
}

// fp16 storage accessed one pair (4 bytes) at a time: for rows whose length is even but
// not a multiple of 8, or that start on 4-byte but not 16-byte boundaries.  The type has
// the size of one half, so pointer offsets count halves like those of __half.
struct f16x2 {
  unsigned short bits;
};

template <>
struct Vec16<f16x2> {
  static constexpr int N = 2;
  using raw_t = unsigned int;
  static __device__ __forceinline__ raw_t load_raw(const f16x2* p)
  {
    return *reinterpret_cast<const unsigned int*>(p);
  }
  static __device__ __forceinline__ void unpack(const raw_t& r, float (&v)[2])
  {
    __half2 h;
    __builtin_memcpy(&h, &r, 4);
    const float2 f = __half22float2(h);
    v[0] = f.x;
    v[1] = f.y;
  }
  static __device__ __forceinline__ void load(const f16x2* p, float (&v)[2]) { unpack(load_raw(p), v); }
  static __device__ __forceinline__ void store(f16x2* p, const float (&v)[2])
  {
    const __half2 h = __floats2half2_rn(v[0], v[1]);
    unsigned int w;
    __builtin_memcpy(&w, &h, 4);
    *reinterpret_cast<unsigned int*>(p) = w;
  }
};

// fp16 storage accessed one value at a time: channels of odd sizes (7 x 7 maps) held by one
// workgroup.  Consecutive lanes take consecutive halves.  Sized like one half.
struct f16x1 {
  unsigned short bits;
};

template <>
struct Vec16<f16x1> {
  static constexpr int N = 1;
  using raw_t = unsigned short;
  static __device__ __forceinline__ raw_t load_raw(const f16x1* p) { return p->bits; }
  static __device__ __forceinline__ void unpack(const raw_t& r, float (&v)[1])
  {
    __half h;
    __builtin_memcpy(&h, &r, 2);
    v[0] = __half2float(h);
  }
  static __device__ __forceinline__ void load(const f16x1* p, float (&v)[1]) { unpack(load_raw(p), v); }
  static __device__ __forceinline__ void store(f16x1* p, const float (&v)[1])
  {
    const __half h = __float2half_rn(v[0]);
    __builtin_memcpy(&p->bits, &h, 2);
  }
  static __device__ __forceinline__ float load1(const f16x1* p)
  {
    float v[1];
    load(p, v);
    return v[0];
  }
  static __device__ __forceinline__ void store1(f16x1* p, float v)
  {
    const float a[1] = {v};
    store(p, a);
  }
};

// fp16 storage accessed four values (8 bytes) at a time: for channels and rows whose length
// is a multiple of 4 but not of 8 (14 x 14 feature maps: 196 entries).  Sized like one half,
// so pointer offsets count halves.
struct f16x4 {
  unsigned short bits;
};

template <>
struct Vec16<f16x4> {
  static constexpr int N = 4;
  using raw_t = uint2;
  static __device__ __forceinline__ raw_t load_raw(const f16x4* p) { return *reinterpret_cast<const uint2*>(p); }
  static __device__ __forceinline__ void unpack(const raw_t& r, float (&v)[4])
  {
    __half2 lo, hi;
    __builtin_memcpy(&lo, &r.x, 4);
    __builtin_memcpy(&hi, &r.y, 4);
    const float2 a = __half22float2(lo), b = __half22float2(hi);
    v[0] = a.x; v[1] = a.y; v[2] = b.x; v[3] = b.y;
  }
  static __device__ __forceinline__ void load(const f16x4* p, float (&v)[4]) { unpack(load_raw(p), v); }
  static __device__ __forceinline__ void store(f16x4* p, const float (&v)[4])
  {
    const __half2 lo = __floats2half2_rn(v[0], v[1]), hi = __floats2half2_rn(v[2], v[3]);
    uint2 r;
    __builtin_memcpy(&r.x, &lo, 4);
    __builtin_memcpy(&r.y, &hi, 4);
    *reinterpret_cast<uint2*>(p) = r;
  }
  static __device__ __forceinline__ float load1(const f16x4* p)
  {
    return __half2float(*reinterpret_cast<const __half*>(p));
  }
  static __device__ __forceinline__ void store1(f16x4* p, float v)
  {
    *reinterpret_cast<__half*>(p) = __float2half_rn(v);
  }
};

// VE consecutive fp32 weights (scale, bias, their partial gradients) at p: 16-byte accesses
// when a thread owns at least four of them, single floats otherwise.
template <int VE>
__device__ __forceinline__ void load_f32_run(const float* p, float (&out)[VE])
{
  if constexpr (VE >= 4) {
#pragma unroll
    for (int k4 = 0; k4 < VE; k4 += 4) {
      float q4[4];
      Vec16<float>::load(p + k4, q4);
#pragma unroll
      for (int k = 0; k < 4; ++k) out[k4 + k] = q4[k];
    }
  }
  else {
#pragma unroll
    for (int k = 0; k < VE; ++k) out[k] = p[k];
  }
}

template <int VE>
__device__ __forceinline__ void store_f32_run(float* p, const float (&in)[VE])
{
  if constexpr (VE >= 4) {
#pragma unroll
    for (int k4 = 0; k4 < VE; k4 += 4) {
      float q4[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) q4[k] = in[k4 + k];
      Vec16<float>::store(p + k4, q4);
    }
  }
  else {
#pragma unroll
    for (int k = 0; k < VE; ++k) p[k] = in[k];
  }
}

template <>
struct Vec16<__half> {
  static constexpr int N = 8;
  using raw_t = v4u;
  static __device__ __forceinline__ raw_t load_raw(const __half* p)
  {
    return LBN_NT_LOAD ? __builtin_nontemporal_load(reinterpret_cast<const v4u*>(p))
                       : *reinterpret_cast<const v4u*>(p);
  }
  static __device__ __forceinline__ void unpack(const raw_t& r, float (&v)[8])
  {
    const unsigned int w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      __half2 h;
      __builtin_memcpy(&h, &w[i], 4);
      const float2 f = __half22float2(h);
      v[2 * i] = f.x;
      v[2 * i + 1] = f.y;
    }
  }
  static __device__ __forceinline__ void load(const __half* p, float (&v)[8])
  {
    const v4u r = load_raw(p);
    const unsigned int w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      __half2 h;
      __builtin_memcpy(&h, &w[i], 4);
      const float2 f = __half22float2(h);
      v[2 * i] = f.x;
      v[2 * i + 1] = f.y;
    }
  }
  static __device__ __forceinline__ void store(__half* p, const float (&v)[8])
  {
    unsigned int w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const __half2 h = __floats2half2_rn(v[2 * i], v[2 * i + 1]);
      __builtin_memcpy(&w[i], &h, 4);
    }
    v4u r;
    r.x = w[0]; r.y = w[1]; r.z = w[2]; r.w = w[3];
    if (LBN_NT_STORE) __builtin_nontemporal_store(r, reinterpret_cast<v4u*>(p));
    else *reinterpret_cast<v4u*>(p) = r;
  }
  static __device__ __forceinline__ float load1(const __half* p) { return __half2float(*p); }
  static __device__ __forceinline__ void store1(__half* p, float v) { *p = __float2half_rn(v); }
};

// fp16 storage in 16-byte accesses at addresses that are only 2-byte aligned (rows of odd
// length): the hardware takes those too (256 MiB copy: 5.2 TB/s against 5.4 aligned).
struct f16u {
  __half v;
};

template <>
struct Vec16<f16u> {
  static constexpr int N = 8;
  using raw_t = v4u;
  static __device__ __forceinline__ raw_t load_raw(const f16u* p)
  {
    v4u r;
    __builtin_memcpy(&r, p, 16);
    return r;
  }
  static __device__ __forceinline__ void unpack(const raw_t& r, float (&v)[8]) { Vec16<__half>::unpack(r, v); }
  static __device__ __forceinline__ void load(const f16u* p, float (&v)[8]) { unpack(load_raw(p), v); }
  static __device__ __forceinline__ void store(f16u* p, const float (&v)[8])
  {
    unsigned int w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const __half2 h = __floats2half2_rn(v[2 * i], v[2 * i + 1]);
      __builtin_memcpy(&w[i], &h, 4);
    }
    __builtin_memcpy(p, w, 16);
  }
  static __device__ __forceinline__ float load1(const f16u* p) { return __half2float(p->v); }
  static __device__ __forceinline__ void store1(f16u* p, float v) { p->v = __float2half_rn(v); }
};

// Aligned fp32 / fp16 storage read with streaming (non-temporal) loads, for calls that move more
// than the last-level cache holds: lines that are read once then do not displace each other
// (layer norm backward over 256 MiB tensors that are not in any cache: 68 -> 76 % of 8 TB/s).
// Tensors that fit that cache lose as much when they are found there, so the host chooses by size.
struct f32s {
  float v;
};

template <>
struct Vec16<f32s> {
  static constexpr int N = 4;
  using raw_t = v4f;
  static __device__ __forceinline__ raw_t load_raw(const f32s* p)
  {
    return __builtin_nontemporal_load(reinterpret_cast<const v4f*>(p));
  }
  static __device__ __forceinline__ void unpack(const raw_t& r, float (&v)[4]) { Vec16<float>::unpack(r, v); }
  static __device__ __forceinline__ void load(const f32s* p, float (&v)[4]) { unpack(load_raw(p), v); }
  static __device__ __forceinline__ void store(f32s* p, const float (&v)[4])
  {
    Vec16<float>::store(reinterpret_cast<float*>(p), v);
  }
  static __device__ __forceinline__ float load1(const f32s* p) { return p->v; }
  static __device__ __forceinline__ void store1(f32s* p, float v) { p->v = v; }
};

struct f16s {
  __half v;
};

template <>
struct Vec16<f16s> {
  static constexpr int N = 8;
  using raw_t = v4u;
  static __device__ __forceinline__ raw_t load_raw(const f16s* p)
  {
    return __builtin_nontemporal_load(reinterpret_cast<const v4u*>(p));
  }
  static __device__ __forceinline__ void unpack(const raw_t& r, float (&v)[8]) { Vec16<__half>::unpack(r, v); }
  static __device__ __forceinline__ void load(const f16s* p, float (&v)[8]) { unpack(load_raw(p), v); }
  static __device__ __forceinline__ void store(f16s* p, const float (&v)[8])
  {
    Vec16<__half>::store(reinterpret_cast<__half*>(p), v);
  }
  static __device__ __forceinline__ float load1(const f16s* p) { return __half2float(p->v); }
  static __device__ __forceinline__ void store1(f16s* p, float v) { p->v = __float2half_rn(v); }
};

// float -> f32s, __half -> f16s
template <typename T>
struct Streamed;
template <>
struct Streamed<float> {
  using type = f32s;
};
template <>
struct Streamed<__half> {
  using type = f16s;
};

// Storage type for a tensor beside streamed data that goes through ordinary loads (the upstream
// gradient in a backward call: the next layer has just written it).
template <typename T>
struct FreshInput {
  using type = T;
};
template <>
struct FreshInput<f32s> {
  using type = float;
};
template <>
struct FreshInput<f16s> {
  using type = __half;
};

template <typename T>
struct StreamedVec : std::integral_constant<bool, std::is_same<T, f16s>::value || std::is_same<T, f32s>::value> {};

// Storage types whose 16-byte accesses need no alignment beyond that of one entry.
template <typename T>
struct UnalignedVec : std::integral_constant<bool, std::is_same<T, f16u>::value || std::is_same<T, f32u>::value> {};

// ---------------------------------------------------------------------------
// exp(x) for x <= ~0 (softmax arguments after max-subtraction) in 6 VALU operations
// and one v_exp_f32: exp(x) = 2^t * 2^r with t = fl(x*log2e) and r the exact
// rounding error of that product plus x*(log2e - fl(log2e)), 2^r ~ 1 + r*ln2.
// Error stays below 2 ulp for x <= 88, against ~20 operations for the library expf.
// Results below the smallest normal float come out as 0 (v_exp_f32 has no denormal
// support); exp_keep_denormals() rescales to keep them.
__device__ __forceinline__ float exp_fast(float x)
{
  constexpr float kLog2e = 1.44269502162933349609375f;        // fl(log2(e))
  constexpr float kLog2eLo = 1.925963033500011e-08f;          // log2(e) - fl(log2(e))
  constexpr float kLn2 = 0.693147182464599609375f;
  x = x < -104.0f ? -104.0f : x;  // exp underflows to 0 there; keeps t finite and NaN a NaN
  const float t = x * kLog2e;
  float r = __builtin_fmaf(x, kLog2e, -t);
  r = __builtin_fmaf(x, kLog2eLo, r);
  const float e = __builtin_amdgcn_exp2f(t);
  return __builtin_fmaf(e, r * kLn2, e);
}

// exp(x) in two operations (one multiply, one v_exp_f32): relative error up to about
// |x| * 3e-8.  Only for terms that are summed and never stored, such as the
// denominator of log-softmax, where that error is far below the result's own rounding.
__device__ __forceinline__ float exp_quick(float x)
{
  return __builtin_amdgcn_exp2f(x * 1.44269502162933349609375f);
}

__device__ __forceinline__ float exp_keep_denormals(float x)
{
  // below exp(-87.3) the result is denormal: evaluate 2^64 times larger, scale back
  const bool tiny = x < -87.0f;
  const float e = exp_fast(tiny ? x + 44.3614196f : x);       // 64*ln2
  return tiny ? e * 5.42101086e-20f : e;                      // 2^-64
}

// log(s) for the sum of a max-shifted softmax row, which always lies in [1, n] (the row
// maximum contributes exp(0) = 1): one v_log_f32 and a multiply, about 1 ulp there.
__device__ __forceinline__ float log_of_sum(float s)
{
  return __builtin_amdgcn_logf(s) * 0.693147182464599609375f;
}

// 1/sqrt(v) for v > 0 from v_rsq_f32 and one Newton step (about 1 ulp), 5 operations
// instead of the ~35 of a correctly rounded square root followed by a division.
__device__ __forceinline__ float rsqrt_refined(float v)
{
  const float y = __builtin_amdgcn_rsqf(v);
  const float h = 0.5f * v;
  return __builtin_fmaf(y, __builtin_fmaf(-h * y, y, 0.5f), y);
}

// ---------------------------------------------------------------------------
// Wave64 reductions on the DPP data path (no LDS traffic): four cross-lane steps fold
// every row of 16 lanes (quad swap, quad-pair swap, half-row mirror, row mirror), two
// row broadcasts (lane 15 of a row into the next row, lane 31 into the upper half) then
// chain the four rows, which leaves the result of the whole wave in lane 63.
template <int CTRL, int ROW_MASK = 0xF>
__device__ __forceinline__ float dpp_move(float v, float old = 0.f)
{
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, old),
                                                               __builtin_bit_cast(int, v), CTRL,
                                                               ROW_MASK, 0xF, false));
}
__device__ __forceinline__ float read_lane(float v, int lane)
{
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}
constexpr int kDppQuadSwap1 = 0xB1;     // quad_perm:[1,0,3,2]
constexpr int kDppQuadSwap2 = 0x4E;     // quad_perm:[2,3,0,1]
constexpr int kDppHalfMirror = 0x141;   // row_half_mirror
constexpr int kDppRowMirror = 0x140;    // row_mirror
constexpr int kDppRowBcast15 = 0x142;   // lane 15 of each row to the next row
constexpr int kDppRowBcast31 = 0x143;   // lane 31 to rows 2 and 3

// Sum over the wave, valid in lane 63 only.
__device__ __forceinline__ float wave_sum_in_last(float v)
{
  v += dpp_move<kDppQuadSwap1>(v);
  v += dpp_move<kDppQuadSwap2>(v);
  v += dpp_move<kDppHalfMirror>(v);
  v += dpp_move<kDppRowMirror>(v);
  v += dpp_move<kDppRowBcast15, 0xA>(v);  // rows 1 and 3 add rows 0 and 2; the others add 0
  v += dpp_move<kDppRowBcast31, 0xC>(v);  // row 3 adds rows 0+1
  return v;
}
__device__ __forceinline__ float wave_max_in_last(float v)
{
  v = fmaxf(v, dpp_move<kDppQuadSwap1>(v));
  v = fmaxf(v, dpp_move<kDppQuadSwap2>(v));
  v = fmaxf(v, dpp_move<kDppHalfMirror>(v));
  v = fmaxf(v, dpp_move<kDppRowMirror>(v));
  v = fmaxf(v, dpp_move<kDppRowBcast15, 0xA>(v, v));  // disabled rows keep their own value
  v = fmaxf(v, dpp_move<kDppRowBcast31, 0xC>(v, v));
  return v;
}
// Sum / maximum over each group of 16 consecutive lanes (a DPP row); every lane of the
// group gets the result.  Lanes of other groups are never read, so whole groups may be
// inactive.
__device__ __forceinline__ float row16_sum(float v)
{
  v += dpp_move<kDppQuadSwap1>(v);
  v += dpp_move<kDppQuadSwap2>(v);
  v += dpp_move<kDppHalfMirror>(v);
  v += dpp_move<kDppRowMirror>(v);
  return v;
}
__device__ __forceinline__ float row16_max(float v)
{
  v = fmaxf(v, dpp_move<kDppQuadSwap1>(v, v));
  v = fmaxf(v, dpp_move<kDppQuadSwap2>(v, v));
  v = fmaxf(v, dpp_move<kDppHalfMirror>(v, v));
  v = fmaxf(v, dpp_move<kDppRowMirror>(v, v));
  return v;
}
// Every lane gets the result.
__device__ __forceinline__ float wave_sum(float v) { return read_lane(wave_sum_in_last(v), kWave - 1); }
__device__ __forceinline__ float wave_max(float v) { return read_lane(wave_max_in_last(v), kWave - 1); }

// Reductions over a team of NW waves (NW*64 consecutive threads of the block).
// `slot` must point to NW floats (2*NW for the pair version) of LDS that no other
// reduction touches before the next block-wide barrier; every thread of the block
// must make the call when NW > 1.  The summation order is fixed, so results are
// bitwise reproducible run to run.
template <int NW>
__device__ __forceinline__ float team_sum(float v, float* slot, int wave_in_team, int lane)
{
  if constexpr (NW == 1) return wave_sum(v);
  v = wave_sum_in_last(v);
  if (lane == kWave - 1) slot[wave_in_team] = v;
  __syncthreads();
  float r = slot[0];
#pragma unroll
  for (int i = 1; i < NW; ++i) r += slot[i];
  return r;
}

template <int NW>
__device__ __forceinline__ float team_max(float v, float* slot, int wave_in_team, int lane)
{
  if constexpr (NW == 1) return wave_max(v);
  v = wave_max_in_last(v);
  if (lane == kWave - 1) slot[wave_in_team] = v;
  __syncthreads();
  float r = slot[0];
#pragma unroll
  for (int i = 1; i < NW; ++i) r = fmaxf(r, slot[i]);
  return r;
}

// Workgroups are handed to the eight accelerator dies (each with an L2 of its own) in turn: block b
// runs on die b % 8.  Where neighbouring work items share cache lines (channels whose segments
// are not whole lines), this gives die x the items [start(x), start(x + 1)) in the order in which
// its blocks start, so that neighbours meet in one L2 instead of being fetched into two.  A
// bijection of [0, blocks) for any number of blocks.
constexpr unsigned kDies = 8;
__device__ __forceinline__ unsigned item_of_block_by_die(unsigned b, unsigned blocks)
{
  const unsigned die = b % kDies, turn = b / kDies;
  const unsigned q = blocks / kDies, r = blocks % kDies;
  return die * q + (die < r ? die : r) + turn;
}

template <int NW>
__device__ __forceinline__ void team_sum2(float& a, float& b, float* slot, int wave_in_team,
                                          int lane)
{
  if constexpr (NW == 1) {
    a = wave_sum(a);
    b = wave_sum(b);
    return;
  }
  a = wave_sum_in_last(a);
  b = wave_sum_in_last(b);
  if (lane == kWave - 1) {
    slot[2 * wave_in_team] = a;
    slot[2 * wave_in_team + 1] = b;
  }
  __syncthreads();
  float ra = slot[0], rb = slot[1];
#pragma unroll
  for (int i = 1; i < NW; ++i) {
    ra += slot[2 * i];
    rb += slot[2 * i + 1];
  }
  a = ra;
  b = rb;
}

// Thread-block shape used by the register-resident row kernels: a row is owned by a
// team of TPR threads (64, 256 or 1024) and a block holds TEAMS teams.  By default
// blocks have at least 256 threads, so a block covers 4 rows when one wave owns a
// row.  Reductions of multi-wave teams use block-wide barriers, so all teams of a
// block must make the same sequence of reduction calls.
template <int TPR, int TEAMS = (TPR < 256 ? 256 / TPR : 1)>
struct RowBlock {
  static constexpr int kTeams = TEAMS;
  static constexpr int kThreads = TPR * TEAMS;
  static constexpr int kWavesPerTeam = TPR / kWave;
  static_assert(kThreads <= 1024, "block too large");
};

}  // namespace lbn
