// Softmax, log-softmax and channelwise softmax, forward and backward, for gfx950.
//
// All three layers reduce over independent contiguous rows (a matrix column, or a
// channel window of a column).  Three kernel families cover every shape:
//
//  * register-resident row kernels: TPR threads (one wave, 256 or 1024 threads)
//    load a whole row with 128-bit coalesced loads, keep it in registers, reduce
//    on the wave64 DPP path (+ one LDS hop across waves), and store the result.
//    Each tensor is read once and written once.  Used when rows are 16-byte
//    aligned, a multiple of 4 long and at most 32768 entries; rows that are only
//    4-byte aligned (odd lengths) run the same kernels with one float per access up
//    to 8192 entries.
//  * register-resident clusters: rows too long for one workgroup whose tensors
//    exceed the caches are shared by a cluster of workgroups that exchange one
//    (max, sum) pair through memory.
//  * split ("chunked") kernels for the remaining long or unaligned rows: a row is cut
//    into S chunks, one workgroup each; chunks that start off a 16-byte boundary are
//    walked as leading scalars, aligned vectors and trailing scalars.  Kernel 1 leaves one partial reduction per chunk
//    in the workspace (for softmax an online (max, sum) pair), kernel 2 merges the
//    S partials and writes its chunk.  Kernel 1 reads everything before kernel 2
//    writes anything, so in-place operation stays safe with many workgroups per row.
//
// The kernels live in softmax_rows.hpp, softmax_cluster.hpp and softmax_split.hpp; this file
// holds the host side (which kernel a shape takes) and the entry points.
//
// Numerics follow the reference CPU code: max-subtraction, exp at <= 2 ulp (exp_fast),
// reciprocal-then-multiply, and softmax (only) writes 0 for results that are not
// normal floats (include/lbann/utils/dnn_lib/openmp/softmax.hpp:107-116).
#include "cluster_sync.hpp"
#include "device_utils.hpp"
#include "host_utils.hpp"
#include "reference_order.hpp"
#include "softmax_cluster.hpp"
#include "softmax_rows.hpp"
#include "softmax_split.hpp"

#include <mutex>
#include <type_traits>

namespace lbn {

// ==================================================================== host side
struct ChunkPlan {
  int S;
  int64_t chunk;
};

// Chunks per row for the split kernels: enough workgroups to occupy the device
// (about 4 per compute unit) without cutting rows into pieces shorter than 2048
// entries; chunk lengths are multiples of 4 so vector access stays aligned.
static ChunkPlan plan_chunks(int64_t n, int64_t rows)
{
  int64_t S = ceil_div(1024, rows);
  const int64_t by_len = ceil_div(n, 2048);
  if (S > by_len) S = by_len;
  if (S > kMaxChunks) S = kMaxChunks;
  if (S < 1) S = 1;
  int64_t chunk = ceil_div(ceil_div(n, S), 4) * 4;
  S = ceil_div(n, chunk);
  return {static_cast<int>(S), chunk};
}

constexpr int64_t kMaxScalarRow = 8192;   // the same in floats for rows accessed one float at a time
constexpr int64_t kMaxScalarLongRow = 32768;  // with 16 or 32 floats per thread: still one kernel, one read

// Rows of at most 64 access units, when there are many of them, go to teams of 16 lanes
// (four rows per wave) instead of leaving most of a wave idle: attention rows of 64
// entries (16 x 64 x 64 x 256) went from 124 to 54 us per step, 10-class rows from 78 to 21.
// scalar: the units are single entries (rows off the 16-byte grid).  Eight of those per lane
// cost eight registers, so rows of 257 to 512 entries stay with one wave (no barrier, four
// rows per workgroup) instead of four waves with two entries each: 257 x 65536 forward 69 us
// with four waves.
static RowConfig pick_sm_row_config(int64_t units, int64_t rows, bool scalar = false)
{
  // (the same up to 1024 entries with sixteen per lane: 513 x 32768 forward 46 us with four waves)
  if (units <= 64 && rows >= 4096) return {16, units <= 16 ? 1 : units <= 32 ? 2 : 4};
  if (scalar && units > 256 && units <= 512 && rows >= 2048) return {64, 8};
  if (scalar && units > 512 && units <= 1024 && rows >= 2048) return {64, 16};
  if (scalar && units > 1024 && units <= 2048 && rows >= 1024) return {256, 8};  // not sixteen waves of two entries
  return pick_row_config(units, rows);
}

static size_t sm_workspace_bytes(int64_t n, int64_t rows)
{
  if (n <= 0 || rows <= 0) return 0;
  const size_t chunked = kWorkspaceHeaderBytes + static_cast<size_t>(rows) * plan_chunks(n, rows).S * sizeof(float2);
  const size_t cluster = (n > kMaxScalarLongRow) ? cluster_workspace_bytes(rows) : 0;
  return chunked > cluster ? chunked : cluster;
}

// The register-resident cluster kernels read every element once but pay a rendezvous
// (a few microseconds) and a slot-reset launch; the two-kernel split path reads the
// input twice.  While the tensor fits the last-level caches the second read costs no
// HBM traffic, so the cluster path is used only for larger footprints.
constexpr int64_t kClusterMinBytes = int64_t(48) << 20;

// Streaming (non-temporal) loads keep a tensor that is read exactly once from pushing out
// lines that someone will read again.  Whether that pays depends on where the tensor is:
// measured on 32768 x 512 (64 MiB per tensor), us per step with the same buffers every step
// ("resident") / with every step's tensors rotated out of the caches ("cold"):
//   nothing streamed 52.8 / 62.7    backward streams y 52.3 / 60.9    y and dy 55.3 / 56.4
//   forward streams x 55.2 / 61.6   x and y 55.9 / 56.7               all three 54.5 / 58.4
// In a training step the forward input and the upstream gradient have just been written by
// the neighbouring layers and sit in the 256 MB Infinity Cache, while y was written a whole
// forward and backward sweep ago: y is streamed once a call moves more than a third of
// that cache, which costs nothing when the others are resident and helps when they are not.
// Calls that move more than the cache holds stream everything (stream_call_inputs).
constexpr int64_t kStreamOldInputMinBytes = int64_t(96) << 20;

static int stream_loads(int64_t rows, int64_t n, int tensors)
{
  return stream_call_inputs(rows * n * 4 * tensors) ? 1 : 0;
}

// A few very long rows whose tensors fit the caches (262144 x 16): one cluster kernel
// (20.6 us per step) against two split kernels per direction (22.7 us), except while a graph
// is recorded, where the cluster kernel needs a second node (24.1 us).
constexpr int64_t kFewRows = 64;

// Backward: bit 0 streams y, bit 1 streams dy (LBN_STREAM_LOADS_BWD overrides, for experiments).
static int stream_loads_bwd(int64_t rows, int64_t n)
{
  static const int forced = std::getenv("LBN_STREAM_LOADS_BWD") ? std::atoi(std::getenv("LBN_STREAM_LOADS_BWD")) : -1;
  if (forced >= 0) return forced & 3;
  if (stream_loads(rows, n, 3)) return 3;
  return rows * n * 4 * 3 >= kStreamOldInputMinBytes ? 1 : 0;
}

static bool cluster_enabled(hipStream_t st, int64_t rows, int64_t n)
{
  static const bool disabled = std::getenv("LBN_NO_CLUSTER") != nullptr;
  static const bool forced = std::getenv("LBN_FORCE_CLUSTER") != nullptr;
  if (disabled) return false;
  if (forced || rows * n * 4 >= kClusterMinBytes) return true;
  return rows <= kFewRows && !stream_is_capturing(st);
}

// Clusters of a launch that could hold `fit` of them at once.  Every cluster walks the same
// number of rows.  When all rows would fit at once (a few very long rows), a cluster still
// takes two rows as long as every compute unit keeps a workgroup: the second row's loads are
// in flight while the first row's partials cross the cluster, and the first row is written
// while the second one's do (262144 x 16: 13.1 against 14.7 us backward).  Four rows per
// cluster, all loaded up front by one workgroup per compute unit, were measured and are
// slower (forward 14.1 against 10.0 us per launch, backward the same 10.6): one wave per
// SIMD cannot overlap the exponentials of one row with the loads of the next.
static int64_t cluster_count(int64_t rows, int64_t fit, int M)
{
  int64_t per = ceil_div(rows, fit);
  if (per == 1 && rows >= 2 && ceil_div(rows, 2) * M >= 256) per = 2;
  return ceil_div(rows, per);
}

// Launch of the cluster kernels for rows of `units` accesses of W floats each.  Returns -1 when
// the plan or the device's capacity does not allow it (the caller goes on to the split
// kernels), otherwise the call's status.
// Framed access needs every tensor of the call to start each row at the same distance from a
// 16-byte boundary: the base pointers agree modulo 16 bytes and, with more than one column,
// so do the leading dimensions modulo 4 entries (the row stride inside a column is shared).
static bool same_frames(const void* a, int64_t lda, const void* b, int64_t ldb, int64_t w)
{
  const uintptr_t pa = reinterpret_cast<uintptr_t>(a), pb = reinterpret_cast<uintptr_t>(b);
  return (pa & 3u) == 0 && ((pa ^ pb) & 15u) == 0 && (w <= 1 || ((lda - ldb) & 3) == 0);
}

// The same for 16-bit entries (eight to a vector).
static bool same_frames16(const void* a, int64_t lda, const void* b, int64_t ldb, int64_t w)
{
  const uintptr_t pa = reinterpret_cast<uintptr_t>(a), pb = reinterpret_cast<uintptr_t>(b);
  return (pa & 1u) == 0 && ((pa ^ pb) & 15u) == 0 && (w <= 1 || ((lda - ldb) & 7) == 0);
}

// Shortest 16-bit row off the 16-byte grid that takes the packed two-pass kernel rather than the
// register kernels with one entry per access (LBN_F16_LONG_MIN overrides, for experiments).
static int64_t packed_long_min16()
{
  static const int64_t v = std::getenv("LBN_F16_LONG_MIN") ? std::atoll(std::getenv("LBN_F16_LONG_MIN")) : 2048;
  return v;
}

static bool framed_access()
{
  static const bool off = std::getenv("LBN_NO_FRAMED_ACCESS") != nullptr;
  return !off;
}

// FR: framed access (rows off the 16-byte grid moved as 16-byte vectors); `units` is then the
// largest frame, (n + 3 + 3) / 4 vectors, and `n` the row length.
template <int KIND, int W, bool FR = false>
static int sm_fwd_cluster_launch(hipStream_t st, ClusterPlan cp, int64_t units, int64_t rows, const float* x,
                                 int64_t ldx, float* y, int64_t ldy, RowMap map, void* ws, size_t ws_bytes,
                                 unsigned n = 0)
{
  if (!cp.M) return -1;
  if (!ws || ws_bytes < cluster_workspace_bytes(rows) || !aligned16(ws)) return LBN_ERR_WORKSPACE;
  const ClusterWorkspace cw = cluster_workspace(ws);
#define X(VV)                                                                                    \
  if (cp.V == VV) {                                                                              \
    const int cap = cluster_capacity(sm_fwd_cluster<VV, KIND, W, FR>, kClusterThreads);          \
    int64_t ncl = cap / cp.M < rows ? cap / cp.M : rows;                                         \
    if (ncl < 1) return -1;                                                                      \
    ncl = cluster_count(rows, ncl, cp.M);                                                        \
    ClusterLaunchGuard guard(st);                                                                \
    if (guard.failed()) return -1;                                                               \
    const SmClusterArgs a{x, nullptr, y, ldx, 0, ldy, map, rows, static_cast<unsigned>(units),   \
                          n, cp.M, cw, cluster_call_tag(st, cw)};                                \
    hipLaunchKernelGGL((sm_fwd_cluster<VV, KIND, W, FR>), dim3(static_cast<unsigned>(ncl * cp.M)), \
                       dim3(kClusterThreads), 0, st, a);                                         \
    return launch_status();                                                                      \
  }
  X(1) X(2) X(3) X(4)
  if constexpr (!FR) { X(5) X(6) X(7) X(8) }
#undef X
  return -1;
}

template <int KIND, int W, bool FR = false>
static int sm_bwd_cluster_launch(hipStream_t st, ClusterPlan cp, int64_t units, int64_t rows, const float* y,
                                 int64_t ldy, const float* dy, int64_t lddy, float* dx, int64_t lddx, RowMap map,
                                 void* ws, size_t ws_bytes, unsigned n = 0)
{
  if (!cp.M) return -1;
  if (!ws || ws_bytes < cluster_workspace_bytes(rows) || !aligned16(ws)) return LBN_ERR_WORKSPACE;
  const ClusterWorkspace cw = cluster_workspace(ws);
#define X(VV)                                                                                    \
  if (cp.V == VV) {                                                                              \
    const int cap = cluster_capacity(sm_bwd_cluster<VV, KIND, W, FR>, kClusterThreads);          \
    int64_t ncl = cap / cp.M < rows ? cap / cp.M : rows;                                         \
    if (ncl < 1) return -1;                                                                      \
    ncl = cluster_count(rows, ncl, cp.M);                                                        \
    ClusterLaunchGuard guard(st);                                                                \
    if (guard.failed()) return -1;                                                               \
    const SmClusterArgs a{y, dy, dx, ldy, lddy, lddx, map, rows, static_cast<unsigned>(units),   \
                          n, cp.M, cw, cluster_call_tag(st, cw)};                                \
    hipLaunchKernelGGL((sm_bwd_cluster<VV, KIND, W, FR>), dim3(static_cast<unsigned>(ncl * cp.M)), \
                       dim3(kClusterThreads), 0, st, a);                                         \
    return launch_status();                                                                      \
  }
  X(1) X(2) X(3) X(4)
  if constexpr (W == 1) { X(5) X(6) X(7) X(8) }
#undef X
  return -1;
}

#define LBN_ROW_CASES(X)                                                                     \
  X(16, 1) X(16, 2) X(16, 4) X(64, 1) X(64, 2) X(64, 4) X(64, 8) X(256, 1) X(256, 2) X(256, 4) X(256, 8) X(1024, 1)      \
  X(1024, 2) X(1024, 4) X(1024, 8)

// Rows off the 16-byte grid that fit a workgroup's registers as a frame of 16-byte vectors
// (fp32 only).  False: not launched, the caller goes on to the one-float-per-access kernels.
// Measured, us per step framed / one float per access: 197 x 151296: 126 / 105; 1001 x 16384:
// 55 / 56; 4099 x 8192: 134 / 132; 8191 x 4096: 121 / 125; 16385 x 4096: 253 / 267;
// 30522 x 2048: 233 / 248.  The two end vectors of a row cost more than the wider accesses
// save until a row has a few thousand entries.
constexpr int64_t kFramedMinRow = 8000;

template <int KIND, typename S>
static bool sm_fwd_framed_rows(hipStream_t st, int64_t n, int64_t w, int64_t rows, const S* x, int64_t ldx, S* y,
                               int64_t ldy, RowMap map)
{
  if constexpr (!std::is_same<S, float>::value) {
    return false;
  }
  else {
    if (!framed_access() || n < kFramedMinRow || !same_frames(x, ldx, y, ldy, w)) return false;
    const RowConfig c = pick_sm_row_config((n + 6) / 4, rows);
    if (!c.tpr) return false;
#define X(TPR, V)                                                                                      \
  if (c.tpr == TPR && c.v == V) {                                                                      \
    using B = RowBlock<TPR>;                                                                           \
    const unsigned grid = static_cast<unsigned>(ceil_div(rows, B::kTeams));                            \
    hipLaunchKernelGGL((sm_fwd_rows<float, TPR, V, KIND, false, 4, true>), dim3(grid), dim3(B::kThreads), 0, st, \
                       x, y, ldx, ldy, map, rows, static_cast<unsigned>(n));                           \
    return true;                                                                                       \
  }
    LBN_ROW_CASES(X)
#undef X
    return false;
  }
}

template <int KIND, typename S>
static bool sm_bwd_framed_rows(hipStream_t st, int64_t n, int64_t w, int64_t rows, const S* y, int64_t ldy,
                               const S* dy, int64_t lddy, S* dx, int64_t lddx, RowMap map)
{
  if constexpr (!std::is_same<S, float>::value) {
    return false;
  }
  else {
    if (!framed_access() || n < kFramedMinRow || !same_frames(y, ldy, dy, lddy, w) ||
        !same_frames(y, ldy, dx, lddx, w))
      return false;
    const RowConfig c = pick_sm_row_config((n + 6) / 4, rows);
    if (!c.tpr) return false;
#define X(TPR, V)                                                                                      \
  if constexpr (!(TPR == 1024 && V > 8)) /* two tensors of more would not fit 128 registers */         \
  if (c.tpr == TPR && c.v == V) {                                                                      \
    using B = RowBlock<TPR>;                                                                           \
    const unsigned grid = static_cast<unsigned>(ceil_div(rows, B::kTeams));                            \
    hipLaunchKernelGGL((sm_bwd_rows<float, TPR, V, KIND, 0, 4, true>), dim3(grid), dim3(B::kThreads), 0, st, \
                       y, dy, dx, ldy, lddy, lddx, map, rows, static_cast<unsigned>(n));               \
    return true;                                                                                       \
  }
    LBN_ROW_CASES(X)
#undef X
    return false;
  }
}

// Rows off the 16-byte grid (odd lengths or leading dimensions, any row stride) that fit a
// workgroup's registers: the row kernels on 16-byte accesses at the alignment of one entry.  False: not
// launched (LBN_NO_UNALIGNED_ROWS=1 keeps the paths that served these rows before, for tests).
// Measured against what served them before (one half per access up to 2047 entries, the packed
// two-pass kernel from there), us forward / backward: 257 x 65536: 32 / 26 -> 20 / 20; 1025 x
// 16384: 34 / 26 -> 19 / 19; 2049 x 8192: 39 / 33 -> 21 / 19; 4097 x 4096: 25 / 21 -> 19 / 19;
// 30522 x 2048 forward: 51 -> 46.  Not taken: rows of up to 64 entries, which single halves
// spread over all 16 lanes of a team (21 x 1048576: 45 / 41 against 76 / 56), and rows that
// leave a thread more than four vectors per tensor (50257 x 1024 backward: 133 against 74).
constexpr int64_t kUnalignedRowMin = 65;
constexpr int64_t kUnalignedRowMaxFwd = 32768;
constexpr int64_t kUnalignedRowMaxBwd = 16384;
static bool unaligned_rows()
{
  static const bool off = std::getenv("LBN_NO_UNALIGNED_ROWS") != nullptr;
  return !off;
}

// fp32 rows: single floats are as fast or faster everywhere (257 to 1025 and 4097 entries: 23-32 us
// forward against 27-32) except from 2049 to 4096 entries, where they fill 1024 threads with
// two to four registers each (2049 x 8192: 44 / 38 us against 27 / 35 with unaligned vectors).
template <typename S>
static bool unaligned_rows_serve(int64_t n, int64_t longest)
{
  if (!unaligned_rows() || n > longest) return false;
  return sizeof(S) == 2 ? n >= kUnalignedRowMin : (n > 2048 && n <= 4096);
}

template <int KIND, typename S>
static bool sm_fwd_unaligned_rows(hipStream_t st, int64_t n, int64_t rows, const S* x, int64_t ldx, S* y, int64_t ldy,
                                  RowMap map)
{
  if constexpr (KIND == kChannelwise) {
    return false;
  }
  else {
    constexpr int W = 16 / sizeof(S);
    if (!unaligned_rows_serve<S>(n, kUnalignedRowMaxFwd)) return false;
    const RowConfig c = pick_sm_row_config(ceil_div(n, W), rows);
    if (!c.tpr) return false;
#define X(TPR, V)                                                                                       \
  if (c.tpr == TPR && c.v == V) {                                                                       \
    using B = RowBlock<TPR>;                                                                            \
    const unsigned grid = static_cast<unsigned>(ceil_div(rows, B::kTeams));                             \
    hipLaunchKernelGGL((sm_fwd_rows<S, TPR, V, KIND, false, W, false, true>), dim3(grid), dim3(B::kThreads), 0, st, \
                       x, y, ldx, ldy, map, rows, static_cast<unsigned>(n));                            \
    return true;                                                                                        \
  }
    LBN_ROW_CASES(X)
#undef X
    return false;
  }
}

template <int KIND, typename S>
static bool sm_bwd_unaligned_rows(hipStream_t st, int64_t n, int64_t rows, const S* y, int64_t ldy, const S* dy,
                                  int64_t lddy, S* dx, int64_t lddx, RowMap map)
{
  if constexpr (KIND == kChannelwise) {
    return false;
  }
  else {
    constexpr int W = 16 / sizeof(S);
    // (softmax backward gains up to the forward limit: 30522 x 2048 fp16 82 -> 72 us; log-softmax,
    // whose exponentials sit between the loads and the stores, loses there: 64 -> 74 us)
    if (!unaligned_rows_serve<S>(n, KIND == kLogSoftmax ? kUnalignedRowMaxBwd : kUnalignedRowMaxFwd)) return false;
    const RowConfig c = pick_sm_row_config(ceil_div(n, W), rows);
    if (!c.tpr) return false;
#define X(TPR, V)                                                                                       \
  if (c.tpr == TPR && c.v == V) {                                                                       \
    using B = RowBlock<TPR>;                                                                            \
    const unsigned grid = static_cast<unsigned>(ceil_div(rows, B::kTeams));                             \
    hipLaunchKernelGGL((sm_bwd_rows<S, TPR, V, KIND, 0, W, false, true>), dim3(grid), dim3(B::kThreads), 0, st, \
                       y, dy, dx, ldy, lddy, lddx, map, rows, static_cast<unsigned>(n));                \
    return true;                                                                                        \
  }
    LBN_ROW_CASES(X)
#undef X
    return false;
  }
}

// The walking forward kernel for 16-bit rows of four vectors per thread, when the rows need
// more than one workgroup per compute unit.
template <int KIND, typename S>
static bool sm_fwd_walk(hipStream_t st, int64_t rows, unsigned nvec, const S* x, S* y, int64_t ldx, int64_t ldy,
                        RowMap map)
{
  static const bool off = std::getenv("LBN_NO_FWD_WALK") != nullptr;
  if (off || KIND == kChannelwise) return false;
  const int cus = compute_units();
  if (cus < 1 || rows <= cus) return false;
  hipLaunchKernelGGL((sm_fwd_rows_walk<S, 4, KIND>), dim3(static_cast<unsigned>(cus)), dim3(1024), 0, st, x, y, ldx,
                     ldy, map, rows, nvec);
  return true;
}

template <int KIND, typename S = float>
static int sm_fwd(hipStream_t st, int64_t groups, int64_t n, int64_t stride, int64_t w,
                  const S* x, int64_t ldx, S* y, int64_t ldy, void* ws, size_t ws_bytes)
{
  constexpr int VE = 16 / sizeof(S);  // entries per 16-byte vector
  if (groups < 0 || n < 0 || w < 0 || stride < 0) return LBN_ERR_INVALID_ARGUMENT;
  if (groups == 0 || n == 0 || w == 0) return LBN_OK;
  if (!x || !y) return LBN_ERR_INVALID_ARGUMENT;
  const int64_t height = (groups - 1) * stride + n;
  if (w > 1 && (ldx < height || ldy < height)) return LBN_ERR_INVALID_ARGUMENT;
  const int64_t rows = groups * w;
  if (rows > (int64_t(1) << 30)) return LBN_ERR_UNSUPPORTED;
  const RowMap map{groups, stride};
  const bool vec = (n % VE == 0) && rows_aligned16(x, stride, ldx, groups, w, sizeof(S)) &&
                   rows_aligned16(y, stride, ldy, groups, w, sizeof(S));
  if (vec) {
    const RowConfig c = pick_sm_row_config(n / VE, rows);
    if (c.tpr) {
      const unsigned nvec = static_cast<unsigned>(n / VE);
#define X(TPR, V)                                                                            \
  if (c.tpr == TPR && c.v == V) {                                                            \
    using B = RowBlock<TPR>;                                                                 \
    const unsigned grid = static_cast<unsigned>(ceil_div(rows, B::kTeams));                  \
    if constexpr (sizeof(S) == 2 && TPR == 1024 && V == 4 && KIND != kChannelwise) {         \
      if (sm_fwd_walk<KIND>(st, rows, nvec, x, y, ldx, ldy, map)) return launch_status();    \
    }                                                                                        \
    if (stream_loads(rows, n * sizeof(S) / 4, 2))                                            \
      hipLaunchKernelGGL((sm_fwd_rows<S, TPR, V, KIND, true>), dim3(grid), dim3(B::kThreads), 0, st, \
                         x, y, ldx, ldy, map, rows, nvec);                                   \
    else                                                                                     \
      hipLaunchKernelGGL((sm_fwd_rows<S, TPR, V, KIND, false>), dim3(grid), dim3(B::kThreads), 0, st, \
                         x, y, ldx, ldy, map, rows, nvec);                                   \
    return launch_status();                                                                  \
  }
      LBN_ROW_CASES(X)
#undef X
    }
  }
  else if (sm_fwd_framed_rows<KIND>(st, n, w, rows, x, ldx, y, ldy, map)) {
    return launch_status();
  }
  else if (sm_fwd_unaligned_rows<KIND>(st, n, rows, x, ldx, y, ldy, map)) {
    return launch_status();
  }
  else if (sizeof(S) == 2 && n >= packed_long_min16() && groups == 1 && same_frames16(x, ldx, y, ldy, w) &&
           framed_access()) {
    // 16-bit rows off the 16-byte grid, long enough for a workgroup each: the packed two-pass
    // kernel below instead of registers filled two bytes at a time
  }
  else if (n <= kMaxScalarRow) {
    // rows that are only 4-byte aligned and short enough for registers: one float per access
    const RowConfig c = pick_sm_row_config(n, rows, true);
    if (c.tpr) {
      const unsigned nvec = static_cast<unsigned>(n);
#define X(TPR, V)                                                                            \
  if (c.tpr == TPR && c.v == V) {                                                            \
    using B = RowBlock<TPR>;                                                                 \
    const unsigned grid = static_cast<unsigned>(ceil_div(rows, B::kTeams));                  \
    hipLaunchKernelGGL((sm_fwd_rows<S, TPR, V, KIND, false, 1>), dim3(grid), dim3(B::kThreads), 0, st, \
                       x, y, ldx, ldy, map, rows, nvec);                                     \
    return launch_status();                                                                  \
  }
      LBN_ROW_CASES(X) X(64, 16)
#undef X
    }
  }
  else if (n <= kMaxScalarLongRow) {
    // the same up to 32768 entries (16385 x 4096: one kernel instead of partials + apply)
    const unsigned nvec = static_cast<unsigned>(n);
    const unsigned grid = static_cast<unsigned>(rows);
    if (n <= 16 * 1024)
      hipLaunchKernelGGL((sm_fwd_rows<S, 1024, 16, KIND, false, 1>), dim3(grid), dim3(1024), 0, st, x, y, ldx, ldy,
                         map, rows, nvec);
    else
      hipLaunchKernelGGL((sm_fwd_rows<S, 1024, 32, KIND, false, 1>), dim3(grid), dim3(1024), 0, st, x, y, ldx, ldy,
                         map, rows, nvec);
    return launch_status();
  }
  if constexpr (!std::is_same<S, float>::value) {
    // fp16 rows beyond the register kernels: one workgroup per row, two passes of 16-byte
    // accesses when the rows are made of whole aligned vectors, else three passes entry by entry
    if (vec && n < (int64_t(1) << 34))
      hipLaunchKernelGGL((sm_fwd_long_packed<S, KIND, false>), dim3(static_cast<unsigned>(rows)), dim3(kLongThreads),
                         0, st, x, y, ldx, ldy, map, n);
    else if (groups == 1 && same_frames16(x, ldx, y, ldy, w) && n < (int64_t(1) << 34) && framed_access())
      hipLaunchKernelGGL((sm_fwd_long_packed<S, KIND, true>), dim3(static_cast<unsigned>(rows)), dim3(kLongThreads),
                         0, st, x, y, ldx, ldy, map, n);
    else
      hipLaunchKernelGGL((sm_fwd_generic<S, KIND>), dim3(static_cast<unsigned>(rows)), dim3(kChunkThreads), 0, st, x,
                         y, ldx, ldy, map, n);
    return launch_status();
  }
  else {
    if (cluster_enabled(st, rows, n)) {
      int r = -1;
      if (vec && n / 4 < (int64_t(1) << 30)) {
        // four vectors per thread keep five workgroups per CU resident; eight only for rows that need it
        ClusterPlan cp = plan_cluster(n / 4, 4);
        if (!cp.M) cp = plan_cluster(n / 4, 8);
        r = sm_fwd_cluster_launch<KIND, 4>(st, cp, n / 4, rows, x, ldx, y, ldy, map, ws, ws_bytes);
      }
      else if (!vec) {
        // rows off the 16-byte grid (a vocabulary of 50257 entries): framed 16-byte access when both
        // tensors sit on the grid alike, else the same kernel with one float per access.  50257 x 1024,
        // us per step framed / one float per access: softmax 210 / 220, log-softmax 209 / 254
        const int64_t frame = (n + 6) / 4;
        if (framed_access() && same_frames(x, ldx, y, ldy, w) && n < (int64_t(1) << 31))
          r = sm_fwd_cluster_launch<KIND, 4, true>(st, plan_cluster(frame, 4), frame, rows, x, ldx, y, ldy, map, ws,
                                                   ws_bytes, static_cast<unsigned>(n));
        if (r < 0)
          r = sm_fwd_cluster_launch<KIND, 1>(st, plan_cluster(n, 8), n, rows, x, ldx, y, ldy, map, ws, ws_bytes);
      }
      if (r >= 0) return r;
    }
    const ChunkPlan p = plan_chunks(n, rows);
    if (rows * p.S > (int64_t(1) << 30)) return LBN_ERR_UNSUPPORTED;
    if (!ws || ws_bytes < kWorkspaceHeaderBytes + static_cast<size_t>(rows) * p.S * sizeof(float2)) return LBN_ERR_WORKSPACE;
    float2* part = static_cast<float2*>(workspace_payload(ws));
    const dim3 grid(static_cast<unsigned>(rows * p.S)), block(kChunkThreads);
    if (vec) {
      hipLaunchKernelGGL((sm_fwd_partial<true>), grid, block, 0, st, x, ldx, map, n, p.chunk, p.S, part);
      hipLaunchKernelGGL((sm_fwd_apply<true, KIND>), grid, block, 0, st, x, y, ldx, ldy, map, n, p.chunk, p.S, part);
    }
    else {
      hipLaunchKernelGGL((sm_fwd_partial<false>), grid, block, 0, st, x, ldx, map, n, p.chunk, p.S, part);
      hipLaunchKernelGGL((sm_fwd_apply<false, KIND>), grid, block, 0, st, x, y, ldx, ldy, map, n, p.chunk, p.S, part);
    }
    return launch_status();
  }
}

// The walking backward kernel when the rows need more than one resident wave of workgroups.
template <int KIND, typename S>
static bool sm_bwd_walk(hipStream_t st, int hint, int64_t rows, unsigned nvec, const S* y, const S* dy,
                        S* dx, int64_t ldy, int64_t lddy, int64_t lddx, RowMap map)
{
  constexpr int V = 32 / (16 / sizeof(S));  // 32 values of each tensor per thread
  static const bool off = std::getenv("LBN_NO_BWD_WALK") != nullptr;
  if (off) return false;
#define W_(H)                                                                                          \
  if (hint == H) {                                                                                     \
    const int cap = resident_blocks(sm_bwd_rows_walk<S, V, KIND, H>, 1024);                            \
    if (cap < 1 || rows <= cap) return false;                                                          \
    hipLaunchKernelGGL((sm_bwd_rows_walk<S, V, KIND, H>), dim3(static_cast<unsigned>(cap)), dim3(1024), 0, st, y, dy, \
                       dx, ldy, lddy, lddx, map, rows, nvec);                                          \
    return true;                                                                                       \
  }
  W_(0) W_(1) W_(2) W_(3)
#undef W_
  return false;
}

// The same for 16-bit rows of four vectors per thread.
template <int KIND, typename S>
static bool sm_bwd_walk_packed(hipStream_t st, int64_t rows, unsigned nvec, const S* y, const S* dy, S* dx,
                               int64_t ldy, int64_t lddy, int64_t lddx, RowMap map)
{
  static const bool off = std::getenv("LBN_NO_BWD_WALK") != nullptr;
  if (off) return false;
  const int cap = resident_blocks(sm_bwd_rows_walk_packed<S, 4, KIND>, 1024);
  if (cap < 1 || rows <= cap) return false;
  hipLaunchKernelGGL((sm_bwd_rows_walk_packed<S, 4, KIND>), dim3(static_cast<unsigned>(cap)), dim3(1024), 0, st, y,
                     dy, dx, ldy, lddy, lddx, map, rows, nvec);
  return true;
}

template <int KIND, typename S = float>
static int sm_bwd(hipStream_t st, int64_t groups, int64_t n, int64_t stride, int64_t w,
                  const S* y, int64_t ldy, const S* dy, int64_t lddy, S* dx,
                  int64_t lddx, void* ws, size_t ws_bytes)
{
  constexpr int VE = 16 / sizeof(S);
  if (groups < 0 || n < 0 || w < 0 || stride < 0) return LBN_ERR_INVALID_ARGUMENT;
  if (groups == 0 || n == 0 || w == 0) return LBN_OK;
  if (!y || !dy || !dx) return LBN_ERR_INVALID_ARGUMENT;
  const int64_t height = (groups - 1) * stride + n;
  if (w > 1 && (ldy < height || lddy < height || lddx < height)) return LBN_ERR_INVALID_ARGUMENT;
  const int64_t rows = groups * w;
  if (rows > (int64_t(1) << 30)) return LBN_ERR_UNSUPPORTED;
  const RowMap map{groups, stride};
  const bool vec = (n % VE == 0) && rows_aligned16(y, stride, ldy, groups, w, sizeof(S)) &&
                   rows_aligned16(dy, stride, lddy, groups, w, sizeof(S)) &&
                   rows_aligned16(dx, stride, lddx, groups, w, sizeof(S));
  if (vec) {
    // two tensors live in registers: cap each at 4 vectors per thread when a row
    // still fits, so 1024-thread blocks keep two blocks per compute unit
    const RowConfig c = pick_sm_row_config(n / VE, rows);
    if (c.tpr) {
      const unsigned nvec = static_cast<unsigned>(n / VE);
#define X(TPR, V)                                                                            \
  if constexpr (!(TPR == 1024 && V * VE > 32)) /* two tensors of more would not fit 128 registers */ \
  if (c.tpr == TPR && c.v == V) {                                                            \
    using B = RowBlock<TPR>;                                                                 \
    const unsigned grid = static_cast<unsigned>(ceil_div(rows, B::kTeams));                  \
    const int hint = stream_loads_bwd(rows, n * sizeof(S) / 4);                              \
    if constexpr (std::is_same<S, float>::value && TPR == 1024 && V == 8) {                  \
      if (sm_bwd_walk<KIND>(st, hint, rows, nvec, y, dy, dx, ldy, lddy, lddx, map)) return launch_status(); \
    }                                                                                        \
    if constexpr (sizeof(S) == 2 && TPR == 1024 && V == 4) {                                 \
      if (sm_bwd_walk_packed<KIND>(st, rows, nvec, y, dy, dx, ldy, lddy, lddx, map)) return launch_status(); \
    }                                                                                        \
    if (hint == 3)                                                                           \
      hipLaunchKernelGGL((sm_bwd_rows<S, TPR, V, KIND, 3>), dim3(grid), dim3(B::kThreads), 0, st, \
                         y, dy, dx, ldy, lddy, lddx, map, rows, nvec);                       \
    else if (hint == 1)                                                                      \
      hipLaunchKernelGGL((sm_bwd_rows<S, TPR, V, KIND, 1>), dim3(grid), dim3(B::kThreads), 0, st, \
                         y, dy, dx, ldy, lddy, lddx, map, rows, nvec);                       \
    else if (hint == 2)                                                                      \
      hipLaunchKernelGGL((sm_bwd_rows<S, TPR, V, KIND, 2>), dim3(grid), dim3(B::kThreads), 0, st, \
                         y, dy, dx, ldy, lddy, lddx, map, rows, nvec);                       \
    else                                                                                     \
      hipLaunchKernelGGL((sm_bwd_rows<S, TPR, V, KIND, 0>), dim3(grid), dim3(B::kThreads), 0, st, \
                         y, dy, dx, ldy, lddy, lddx, map, rows, nvec);                       \
    return launch_status();                                                                  \
  }
      LBN_ROW_CASES(X)
#undef X
    }
  }
  else if (sm_bwd_framed_rows<KIND>(st, n, w, rows, y, ldy, dy, lddy, dx, lddx, map)) {
    return launch_status();
  }
  else if (sm_bwd_unaligned_rows<KIND>(st, n, rows, y, ldy, dy, lddy, dx, lddx, map)) {
    return launch_status();
  }
  else if (sizeof(S) == 2 && n >= packed_long_min16() && groups == 1 && same_frames16(y, ldy, dy, lddy, w) &&
           same_frames16(y, ldy, dx, lddx, w) && framed_access()) {
    // (as in the forward pass: the packed two-pass kernel below)
  }
  else if (n <= kMaxScalarRow) {
    const RowConfig c = pick_sm_row_config(n, rows, true);
    if (c.tpr) {
      const unsigned nvec = static_cast<unsigned>(n);
#define X(TPR, V)                                                                            \
  if (c.tpr == TPR && c.v == V) {                                                            \
    using B = RowBlock<TPR>;                                                                 \
    const unsigned grid = static_cast<unsigned>(ceil_div(rows, B::kTeams));                  \
    hipLaunchKernelGGL((sm_bwd_rows<S, TPR, V, KIND, 0, 1>), dim3(grid), dim3(B::kThreads), 0, st, \
                       y, dy, dx, ldy, lddy, lddx, map, rows, nvec);                         \
    return launch_status();                                                                  \
  }
      LBN_ROW_CASES(X) X(64, 16)
#undef X
    }
  }
  else if (n <= (std::is_same<S, float>::value ? kMaxScalarLongRow : 16 * 1024)) {
    const unsigned nvec = static_cast<unsigned>(n);
    const unsigned grid = static_cast<unsigned>(rows);
    if (n <= 16 * 1024) {
      hipLaunchKernelGGL((sm_bwd_rows<S, 1024, 16, KIND, 0, 1>), dim3(grid), dim3(1024), 0, st, y, dy, dx, ldy,
                         lddy, lddx, map, rows, nvec);
    }
    else if constexpr (std::is_same<S, float>::value) {
      hipLaunchKernelGGL((sm_bwd_rows<S, 1024, 32, KIND, 0, 1>), dim3(grid), dim3(1024), 0, st, y, dy, dx, ldy,
                         lddy, lddx, map, rows, nvec);
    }
    return launch_status();
  }
  if constexpr (!std::is_same<S, float>::value) {
    if (vec && n < (int64_t(1) << 34))
      hipLaunchKernelGGL((sm_bwd_long_packed<S, KIND, false>), dim3(static_cast<unsigned>(rows)), dim3(kLongThreads),
                         0, st, y, dy, dx, ldy, lddy, lddx, map, n);
    else if (groups == 1 && same_frames16(y, ldy, dy, lddy, w) && same_frames16(y, ldy, dx, lddx, w) &&
             n < (int64_t(1) << 34) && framed_access())
      hipLaunchKernelGGL((sm_bwd_long_packed<S, KIND, true>), dim3(static_cast<unsigned>(rows)), dim3(kLongThreads),
                         0, st, y, dy, dx, ldy, lddy, lddx, map, n);
    else
      hipLaunchKernelGGL((sm_bwd_generic<S, KIND>), dim3(static_cast<unsigned>(rows)), dim3(kChunkThreads), 0, st, y,
                         dy, dx, ldy, lddy, lddx, map, n);
    return launch_status();
  }
  else {
    if (cluster_enabled(st, rows, n)) {
      int r = -1;
      if (vec && n / 4 < (int64_t(1) << 30))
        r = sm_bwd_cluster_launch<KIND, 4>(st, plan_cluster(n / 4, 4), n / 4, rows, y, ldy, dy, lddy, dx, lddx, map, ws,
                                           ws_bytes);
      else if (!vec) {
        const int64_t frame = (n + 6) / 4;
        if (framed_access() && same_frames(y, ldy, dy, lddy, w) && same_frames(y, ldy, dx, lddx, w) &&
            n < (int64_t(1) << 31))
          r = sm_bwd_cluster_launch<KIND, 4, true>(st, plan_cluster(frame, 3), frame, rows, y, ldy, dy, lddy, dx, lddx,
                                                   map, ws, ws_bytes, static_cast<unsigned>(n));
        if (r < 0)
          r = sm_bwd_cluster_launch<KIND, 1>(st, plan_cluster(n, 8), n, rows, y, ldy, dy, lddy, dx, lddx, map, ws,
                                             ws_bytes);
      }
      if (r >= 0) return r;
    }
    const ChunkPlan p = plan_chunks(n, rows);
    if (rows * p.S > (int64_t(1) << 30)) return LBN_ERR_UNSUPPORTED;
    if (!ws || ws_bytes < kWorkspaceHeaderBytes + static_cast<size_t>(rows) * p.S * sizeof(float2)) return LBN_ERR_WORKSPACE;
    float* part = static_cast<float*>(workspace_payload(ws));
    const dim3 grid(static_cast<unsigned>(rows * p.S)), block(kChunkThreads);
    if (vec) {
      hipLaunchKernelGGL((sm_bwd_partial<true, KIND>), grid, block, 0, st, y, dy, ldy, lddy, map, n, p.chunk, p.S, part);
      hipLaunchKernelGGL((sm_bwd_apply<true, KIND>), grid, block, 0, st, y, dy, dx, ldy, lddy, lddx, map, n, p.chunk, p.S, part);
    }
    else {
      hipLaunchKernelGGL((sm_bwd_partial<false, KIND>), grid, block, 0, st, y, dy, ldy, lddy, map, n, p.chunk, p.S, part);
      hipLaunchKernelGGL((sm_bwd_apply<false, KIND>), grid, block, 0, st, y, dy, dx, ldy, lddy, lddx, map, n, p.chunk, p.S, part);
    }
    return launch_status();
  }
}

// Softmax forward fused with the cross-entropy forward.  Returns -1 when the shape is not one
// the fused kernel takes (the caller then runs the two layers' kernels one after the other).
static int sm_ce_fwd_fused(hipStream_t st, int64_t n, int64_t w, int labels, const float* x, int64_t ldx,
                           const float* truth, int64_t ldt, float* y, int64_t ldy, float* loss, int64_t ld_loss)
{
  const bool vec = (n % 4 == 0) && rows_aligned16(x, n, ldx, 1, w, 4) && rows_aligned16(y, n, ldy, 1, w, 4) &&
                   (labels || rows_aligned16(truth, n, ldt, 1, w, 4));
  if (!vec) return -1;
  const RowConfig c = pick_sm_row_config(n / 4, w);
  if (!c.tpr) return -1;
  const unsigned nvec = static_cast<unsigned>(n / 4);
#define X(TPR, V)                                                                                      \
  if (c.tpr == TPR && c.v == V) {                                                                      \
    using B = RowBlock<TPR>;                                                                           \
    const unsigned grid = static_cast<unsigned>(ceil_div(w, B::kTeams));                               \
    if (labels)                                                                                        \
      hipLaunchKernelGGL((sm_ce_fwd_rows<TPR, V, true>), dim3(grid), dim3(B::kThreads), 0, st, x, truth, y, loss, \
                         ldx, ldt, ldy, ld_loss, w, nvec);                                             \
    else                                                                                               \
      hipLaunchKernelGGL((sm_ce_fwd_rows<TPR, V, false>), dim3(grid), dim3(B::kThreads), 0, st, x, truth, y, loss, \
                         ldx, ldt, ldy, ld_loss, w, nvec);                                             \
    return launch_status();                                                                            \
  }
  LBN_ROW_CASES(X)
#undef X
  return -1;
}

// Backward of the pair in one kernel; -1 when the shape is not one the fused kernel takes.
static int sm_ce_bwd_fused(hipStream_t st, int64_t n, int64_t w, int labels, const float* y, int64_t ldy,
                           const float* truth, int64_t ldt, const float* dloss, int64_t ld_dloss, float* dx,
                           int64_t lddx, float* dtruth, int64_t lddt)
{
  const bool vec = (n % 4 == 0) && rows_aligned16(y, n, ldy, 1, w, 4) && rows_aligned16(dx, n, lddx, 1, w, 4) &&
                   (labels || rows_aligned16(truth, n, ldt, 1, w, 4)) &&
                   (labels || !dtruth || rows_aligned16(dtruth, n, lddt, 1, w, 4));
  if (!vec) return -1;
  const RowConfig c = pick_sm_row_config(n / 4, w);
  if (!c.tpr) return -1;
  const unsigned nvec = static_cast<unsigned>(n / 4);
#define X(TPR, V)                                                                                      \
  if (c.tpr == TPR && c.v == V) {                                                                      \
    using B = RowBlock<TPR>;                                                                           \
    const unsigned grid = static_cast<unsigned>(ceil_div(w, B::kTeams));                               \
    if (labels)                                                                                        \
      hipLaunchKernelGGL((sm_ce_bwd_rows<TPR, V, true>), dim3(grid), dim3(B::kThreads), 0, st, y, truth, dloss, dx, \
                         nullptr, ldy, ldt, ld_dloss, lddx, 0, w, nvec);                               \
    else                                                                                               \
      hipLaunchKernelGGL((sm_ce_bwd_rows<TPR, V, false>), dim3(grid), dim3(B::kThreads), 0, st, y, truth, dloss, dx, \
                         dtruth, ldy, ldt, ld_dloss, lddx, lddt, w, nvec);                             \
    return launch_status();                                                                            \
  }
  LBN_ROW_CASES(X)
#undef X
  return -1;
}

// ------------------------------------------------------------ library-owned scratch
// Scratch of the entry point that allocates nothing: one array per GPU, part of the code
// object, so it exists from the moment the library is loaded until the process ends.  The
// array's name is only a host-side handle: host code uses the address that
// hipGetSymbolAddress() reports for the current device, looked up once per device.
constexpr size_t kStaticScratchBytes = size_t(1) << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;

size_t static_scratch_bytes() { return kStaticScratchBytes; }

// Device address of `scratch` on the current device; *out stays null on failure.
int static_scratch_address(void** out)
{
  static std::mutex mu;
  static void* address[kMaxDevices] = {};
  *out = nullptr;
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return static_cast<int>(e);
  if (dev < 0 || dev >= kMaxDevices) return LBN_ERR_UNSUPPORTED;
  std::lock_guard<std::mutex> lock(mu);
  if (!address[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return static_cast<int>(e);
    if (!p) return static_cast<int>(hipErrorInvalidSymbol);
    address[dev] = p;
    // set-up, once per device: the event that orders cluster kernels across streams, so that
    // no later call of the entry point that allocates nothing has to create it
    ClusterLaunchGuard::prepare();
  }
  *out = address[dev];
  return LBN_OK;
}

}  // namespace lbn

using namespace lbn;

extern "C" {

size_t lbn_softmax_workspace_bytes(int64_t height, int64_t width)
{
  return sm_workspace_bytes(height, width);
}

size_t lbn_channelwise_softmax_workspace_bytes(int64_t channels, int64_t channel_size, int64_t width)
{
  if (channels <= 0 || width <= 0) return 0;
  return sm_workspace_bytes(channel_size, channels * width);
}

int lbn_softmax_fwd_f32(lbn_stream_t stream, int64_t height, int64_t width, const float* x,
                        int64_t ldx, float* y, int64_t ldy, void* workspace, size_t workspace_bytes)
{
  return sm_fwd<kSoftmax>(as_stream(stream), 1, height, height, width, x, ldx, y, ldy, workspace, workspace_bytes);
}

int lbn_softmax_bwd_f32(lbn_stream_t stream, int64_t height, int64_t width, const float* y,
                        int64_t ldy, const float* dy, int64_t lddy, float* dx, int64_t lddx,
                        void* workspace, size_t workspace_bytes)
{
  return sm_bwd<kSoftmax>(as_stream(stream), 1, height, height, width, y, ldy, dy, lddy, dx, lddx, workspace, workspace_bytes);
}

size_t lbn_softmax_fwd_static_scratch_max_bytes(void) { return kStaticScratchBytes; }

int lbn_softmax_fwd_static_scratch_f32(lbn_stream_t stream, int64_t height, int64_t width, const float* x,
                                       int64_t ldx, float* y, int64_t ldy)
{
  if (height < 0 || width < 0) return LBN_ERR_INVALID_ARGUMENT;
  if (height == 0 || width == 0) return LBN_OK;
  if (sm_workspace_bytes(height, width) > kStaticScratchBytes) return LBN_ERR_UNSUPPORTED;
  void* ptr = nullptr;
  const int status = static_scratch_address(&ptr);
  if (status != LBN_OK) return status;
  return sm_fwd<kSoftmax>(as_stream(stream), 1, height, height, width, x, ldx, y, ldy, ptr, kStaticScratchBytes);
}

// Parity tests only: the reference's order of summation (reference_order.hpp).
int lbn_softmax_fwd_reference_order_f32(lbn_stream_t stream, int64_t height, int64_t width, const float* x,
                                        int64_t ldx, float* y, int64_t ldy)
{
  if (height < 0 || width < 0 || (width > 1 && (ldx < height || ldy < height))) return LBN_ERR_INVALID_ARGUMENT;
  if (height == 0 || width == 0) return LBN_OK;
  if (!x || !y) return LBN_ERR_INVALID_ARGUMENT;
  if (height > kRefOrderMaxEntries / width || width > (int64_t(1) << 30)) return LBN_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(sm_ref_order_fwd, dim3(static_cast<unsigned>(width)), dim3(kWave), 0, as_stream(stream), x, y, ldx,
                     ldy, height);
  return launch_status();
}

int lbn_log_softmax_bwd_reference_order_f32(lbn_stream_t stream, int64_t height, int64_t width, const float* y,
                                            int64_t ldy, const float* dy, int64_t lddy, float* dx, int64_t lddx)
{
  if (height < 0 || width < 0 || (width > 1 && (ldy < height || lddy < height || lddx < height)))
    return LBN_ERR_INVALID_ARGUMENT;
  if (height == 0 || width == 0) return LBN_OK;
  if (!y || !dy || !dx) return LBN_ERR_INVALID_ARGUMENT;
  if (height > kRefOrderMaxEntries / width || width > (int64_t(1) << 30)) return LBN_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(lsm_ref_order_bwd, dim3(static_cast<unsigned>(width)), dim3(kWave), 0, as_stream(stream), y, dy,
                     dx, ldy, lddy, lddx, height);
  return launch_status();
}

int lbn_softmax_fwd_static_scratch_prepare(void)
{
  void* ptr = nullptr;
  return static_scratch_address(&ptr);
}

int lbn_softmax_fwd_static_scratch_timed_out(lbn_stream_t stream, int* timed_out)
{
  if (!timed_out) return LBN_ERR_INVALID_ARGUMENT;
  *timed_out = 0;
  void* ptr = nullptr;
  const int status = static_scratch_address(&ptr);
  if (status != LBN_OK) return status;
  hipStream_t st = as_stream(stream);
  int word = 0;
  hipError_t e = hipMemcpyAsync(&word, ptr, sizeof(int), hipMemcpyDeviceToHost, st);
  if (e == hipSuccess) e = hipStreamSynchronize(st);
  if (e != hipSuccess) return static_cast<int>(e);
  if (word == kClusterTimedOut) {
    *timed_out = 1;
    e = hipMemsetAsync(ptr, 0, sizeof(int), st);  // read and cleared: the next call starts afresh
    if (e == hipSuccess) e = hipStreamSynchronize(st);
    if (e != hipSuccess) return static_cast<int>(e);
  }
  return LBN_OK;
}

int lbn_log_softmax_fwd_f32(lbn_stream_t stream, int64_t height, int64_t width, const float* x,
                            int64_t ldx, float* y, int64_t ldy, void* workspace, size_t workspace_bytes)
{
  return sm_fwd<kLogSoftmax>(as_stream(stream), 1, height, height, width, x, ldx, y, ldy, workspace, workspace_bytes);
}

int lbn_log_softmax_bwd_f32(lbn_stream_t stream, int64_t height, int64_t width, const float* y,
                            int64_t ldy, const float* dy, int64_t lddy, float* dx, int64_t lddx,
                            void* workspace, size_t workspace_bytes)
{
  return sm_bwd<kLogSoftmax>(as_stream(stream), 1, height, height, width, y, ldy, dy, lddy, dx, lddx, workspace, workspace_bytes);
}

size_t lbn_softmax_cross_entropy_fwd_workspace_bytes(int64_t height, int64_t width)
{
  // the cross-entropy partial sums sit past the header that the softmax kernels keep their wait status in
  const size_t a = lbn_softmax_workspace_bytes(height, width);
  const size_t b = lbn_cross_entropy_fwd_workspace_bytes(height, width);
  return a > b + kWorkspaceHeaderBytes ? a : (b ? b + kWorkspaceHeaderBytes : a);
}

int lbn_softmax_cross_entropy_fwd_f32(lbn_stream_t stream, int64_t height, int64_t width, int use_labels,
                                      int64_t spatial_size, const float* x, int64_t ldx, const float* ground_truth,
                                      int64_t ld_truth, float* y, int64_t ldy, float* loss, int64_t ld_loss,
                                      void* workspace, size_t workspace_bytes)
{
  hipStream_t st = as_stream(stream);
  if (height < 0 || width < 0 || ld_loss < 0) return LBN_ERR_INVALID_ARGUMENT;
  if (width == 0) return LBN_OK;
  if (height == 0)  // no softmax output; the loss of an empty column is 0
    return lbn_cross_entropy_fwd_f32(stream, height, width, use_labels, spatial_size, y, ldy, ground_truth, ld_truth,
                                     loss, ld_loss, nullptr, 0);
  if (!x || !ground_truth || !y || !loss || ld_loss < 1) return LBN_ERR_INVALID_ARGUMENT;
  if (use_labels && spatial_size < 1) return LBN_ERR_INVALID_ARGUMENT;
  if (width > 1 && (ldx < height || ldy < height || ld_truth < (use_labels ? 1 : height)))
    return LBN_ERR_INVALID_ARGUMENT;
  if (!use_labels || spatial_size == 1) {
    const int r = sm_ce_fwd_fused(st, height, width, use_labels ? 1 : 0, x, ldx, ground_truth, ld_truth, y, ldy,
                                  loss, ld_loss);
    if (r >= 0) return r;
  }
  // shapes the fused kernel does not take: the two layers' kernels one after the other
  const int status = sm_fwd<kSoftmax>(st, 1, height, height, width, x, ldx, y, ldy, workspace, workspace_bytes);
  if (status != LBN_OK) return status;
  const bool room = workspace && workspace_bytes > kWorkspaceHeaderBytes;
  return lbn_cross_entropy_fwd_f32(stream, height, width, use_labels, spatial_size, y, ldy, ground_truth, ld_truth,
                                   loss, ld_loss, room ? workspace_payload(workspace) : nullptr,
                                   room ? workspace_bytes - kWorkspaceHeaderBytes : 0);
}

int lbn_softmax_cross_entropy_bwd_f32(lbn_stream_t stream, int64_t height, int64_t width, int use_labels,
                                      int64_t spatial_size, const float* y, int64_t ldy, const float* ground_truth,
                                      int64_t ld_truth, const float* dloss, int64_t ld_dloss, float* dx, int64_t lddx,
                                      float* dground_truth, int64_t ld_dground_truth, void* workspace,
                                      size_t workspace_bytes)
{
  hipStream_t st = as_stream(stream);
  if (height < 0 || width < 0) return LBN_ERR_INVALID_ARGUMENT;
  if (height == 0 || width == 0) return LBN_OK;
  if (!y || !ground_truth || !dloss || !dx || ld_dloss < 1) return LBN_ERR_INVALID_ARGUMENT;
  if (use_labels && spatial_size < 1) return LBN_ERR_INVALID_ARGUMENT;
  if (width > 1 && (ldy < height || lddx < height || ld_truth < (use_labels ? 1 : height))) return LBN_ERR_INVALID_ARGUMENT;
  if (!use_labels && dground_truth && width > 1 && ld_dground_truth < height) return LBN_ERR_INVALID_ARGUMENT;
  if (!use_labels || spatial_size == 1) {
    const int r = sm_ce_bwd_fused(st, height, width, use_labels ? 1 : 0, y, ldy, ground_truth, ld_truth, dloss,
                                  ld_dloss, dx, lddx, use_labels ? nullptr : dground_truth, ld_dground_truth);
    if (r >= 0) return r;
  }
  // shapes the fused kernel does not take: the cross-entropy backward leaves its gradient in dx,
  // the softmax backward then runs in place on it (dx may alias dy there)
  const int status = lbn_cross_entropy_bwd_f32(stream, height, width, use_labels, spatial_size, y, ldy, ground_truth,
                                               ld_truth, dloss, ld_dloss, dx, lddx,
                                               use_labels ? nullptr : dground_truth, ld_dground_truth);
  if (status != LBN_OK) return status;
  return sm_bwd<kSoftmax>(st, 1, height, height, width, y, ldy, dx, lddx, dx, lddx, workspace, workspace_bytes);
}

// fp16 storage (IEEE binary16 in memory, fp32 arithmetic); the workspace arguments are there for
// symmetry with the fp32 entry points and are not used.
int lbn_softmax_fwd_f16(lbn_stream_t stream, int64_t height, int64_t width, const void* x, int64_t ldx, void* y,
                        int64_t ldy, void* workspace, size_t workspace_bytes)
{
  return sm_fwd<kSoftmax, __half>(as_stream(stream), 1, height, height, width, static_cast<const __half*>(x), ldx,
                                  static_cast<__half*>(y), ldy, workspace, workspace_bytes);
}

int lbn_softmax_bwd_f16(lbn_stream_t stream, int64_t height, int64_t width, const void* y, int64_t ldy,
                        const void* dy, int64_t lddy, void* dx, int64_t lddx, void* workspace,
                        size_t workspace_bytes)
{
  return sm_bwd<kSoftmax, __half>(as_stream(stream), 1, height, height, width, static_cast<const __half*>(y), ldy,
                                  static_cast<const __half*>(dy), lddy, static_cast<__half*>(dx), lddx, workspace,
                                  workspace_bytes);
}

int lbn_log_softmax_fwd_f16(lbn_stream_t stream, int64_t height, int64_t width, const void* x, int64_t ldx,
                            void* y, int64_t ldy, void* workspace, size_t workspace_bytes)
{
  return sm_fwd<kLogSoftmax, __half>(as_stream(stream), 1, height, height, width, static_cast<const __half*>(x), ldx,
                                     static_cast<__half*>(y), ldy, workspace, workspace_bytes);
}

int lbn_log_softmax_bwd_f16(lbn_stream_t stream, int64_t height, int64_t width, const void* y, int64_t ldy,
                            const void* dy, int64_t lddy, void* dx, int64_t lddx, void* workspace,
                            size_t workspace_bytes)
{
  return sm_bwd<kLogSoftmax, __half>(as_stream(stream), 1, height, height, width, static_cast<const __half*>(y), ldy,
                                     static_cast<const __half*>(dy), lddy, static_cast<__half*>(dx), lddx, workspace,
                                     workspace_bytes);
}

int lbn_channelwise_softmax_fwd_f32(lbn_stream_t stream, int64_t channels, int64_t channel_size,
                                    int64_t channel_stride, int64_t width, const float* x,
                                    int64_t ldx, float* y, int64_t ldy, void* workspace,
                                    size_t workspace_bytes)
{
  return sm_fwd<kChannelwise>(as_stream(stream), channels, channel_size, channel_stride, width, x, ldx, y, ldy, workspace, workspace_bytes);
}

int lbn_channelwise_softmax_bwd_f32(lbn_stream_t stream, int64_t channels, int64_t channel_size,
                                    int64_t channel_stride, int64_t width, const float* y,
                                    int64_t ldy, const float* dy, int64_t lddy, float* dx,
                                    int64_t lddx, void* workspace, size_t workspace_bytes)
{
  return sm_bwd<kChannelwise>(as_stream(stream), channels, channel_size, channel_stride, width, y, ldy, dy, lddy, dx, lddx, workspace, workspace_bytes);
}

}  // extern "C"
