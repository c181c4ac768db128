// Host-side helpers shared by the entry points: argument checks, alignment tests,
// launch-shape selection for the register-resident row kernels.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdlib>
#include <atomic>
#include <map>
#include <mutex>
#include <utility>

#include "../../include/lbnorm.h"

namespace lbn {

// Every entry point converts its stream argument first: that is also where an error left
// behind by an earlier, unrelated HIP call of this thread is dropped, so that
// launch_status() below reports this call's launches only (the header of the C ABI tells
// callers that their pending error is cleared).
inline hipStream_t as_stream(lbn_stream_t s)
{
  (void)hipGetLastError();
  return reinterpret_cast<hipStream_t>(s);
}

// Status of the launches issued by this thread since the entry point began: 0 or the hipError_t.
inline int launch_status()
{
  const hipError_t e = hipGetLastError();
  return e == hipSuccess ? LBN_OK : static_cast<int>(e);
}

// True while `st` records into a HIP graph.  A recorded launch is replayed with the
// arguments it was recorded with, so anything that must differ from call to call (the
// rendezvous tag of the cluster kernels) has to come from device memory there.
inline bool stream_is_capturing(hipStream_t st)
{
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(st, &status) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  return status != hipStreamCaptureStatusNone;
}

// Calls that move more than the 256 MB last-level cache holds read their inputs with streaming
// (non-temporal) loads: nothing they read is found there, and lines that are read once then do
// not displace each other.  Smaller calls keep ordinary loads, which find what the neighbouring
// layers have just written.  LBN_STREAM_LOADS=0|1 overrides, for experiments.
constexpr int64_t kStreamLoadMinBytes = int64_t(384) << 20;

inline bool stream_call_inputs(int64_t bytes_moved, int64_t min_bytes = kStreamLoadMinBytes)
{
  static const int forced = std::getenv("LBN_STREAM_LOADS") ? std::atoi(std::getenv("LBN_STREAM_LOADS")) : -1;
  if (forced >= 0) return forced != 0;
  return bytes_moved >= min_bytes;
}

// Device address (current device) and size of the library-owned scratch array of the entry
// point that allocates nothing (defined in softmax.hip); *out stays null on failure.
int static_scratch_address(void** out);
size_t static_scratch_bytes();

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// True when every row start of a matrix walked with (stride, ld) keeps 16-byte
// alignment for elements of `esize` bytes.
inline bool rows_aligned16(const void* base, int64_t stride, int64_t ld, int64_t groups,
                           int64_t width, int esize)
{
  const int64_t per = 16 / esize;
  if (!aligned16(base)) return false;
  if (groups > 1 && stride % per != 0) return false;
  if (width > 1 && ld % per != 0) return false;
  return true;
}

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Shape of a register-resident row kernel: `tpr` threads own a row and each keeps
// `v` 16-byte vectors of it in registers.  tpr == 0: the row does not fit.
struct RowConfig {
  int tpr;
  int v;
};

inline int round_up_pow2_le8(int64_t v)
{
  if (v <= 1) return 1;
  if (v <= 2) return 2;
  if (v <= 4) return 4;
  if (v <= 8) return 8;
  return 0;
}

// nvec: 16-byte vectors per row; rows: number of independent rows.
// Prefers <= 4 vectors per thread with the fewest threads per row, and widens the
// team when the launch would otherwise leave most of the 256 compute units without
// work (small problems are latency bound, so more threads per row helps there).
inline RowConfig pick_row_config(int64_t nvec, int64_t rows, int max_v = 8)
{
  static const int force_tpr = std::getenv("LBN_ROW_TPR") ? std::atoi(std::getenv("LBN_ROW_TPR")) : 0;
  const int tprs[3] = {64, 256, 1024};
  int vs[3];
  for (int i = 0; i < 3; ++i) {
    vs[i] = round_up_pow2_le8(ceil_div(nvec, tprs[i]));
    if (vs[i] > max_v) vs[i] = 0;
  }
  if (force_tpr) {
    for (int i = 0; i < 3; ++i)
      if (tprs[i] == force_tpr && vs[i]) return {tprs[i], vs[i]};
  }
  int pick = -1;
  for (int i = 0; i < 3; ++i) {
    if (vs[i] == 0) continue;
    pick = i;
    if (vs[i] <= 4) break;
  }
  if (pick < 0) return {0, 0};
  const int64_t want_waves = 2048;
  while (pick < 2 && vs[pick] > 1 && rows * (tprs[pick] / 64) < want_waves && vs[pick + 1] != 0)
    ++pick;
  return {tprs[pick], vs[pick]};
}

// Compute units of the current device (0 if the query fails); asked once per device.
inline int compute_units()
{
  constexpr int kMaxDevices = 64;
  static std::atomic<int> cached[kMaxDevices];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 0;
  int cus = cached[dev].load(std::memory_order_relaxed);
  if (cus > 0) return cus;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 1) return 0;
  cached[dev].store(cus, std::memory_order_relaxed);
  return cus;
}

// Workgroups of `threads` threads running `kernel` that the current device holds at
// once.  Queried once per (kernel, device); the cache is the only process-wide
// state of the library besides the call-tag counter and holds hardware facts only.
template <typename K>
inline int resident_blocks(K kernel, int threads)
{
  static std::mutex mu;
  static std::map<std::pair<const void*, int>, int> cache;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  const auto key = std::make_pair(reinterpret_cast<const void*>(kernel), dev);
  std::lock_guard<std::mutex> lock(mu);
  auto it = cache.find(key);
  if (it != cache.end()) return it->second;
  int cus = 0, per_cu = 0;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, threads, 0) != hipSuccess) return 0;
  cache[key] = cus * per_cu;
  return cus * per_cu;
}

}  // namespace lbn
