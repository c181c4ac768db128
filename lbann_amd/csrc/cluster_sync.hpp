// Rendezvous of a cluster of M workgroups through device memory, used by the
// register-resident split reductions (batch norm channels, very wide softmax rows).
//
// Each workgroup of a cluster keeps its share of the data in registers, publishes
// one partial pair, waits until all M partials of the cluster are there, and then
// finishes from its registers: every tensor is read from memory exactly once.
//
// Protocol (no fences, no cache write-back or invalidation): every slot is one
// 64-bit word holding two floats.  A small kernel fills the slots of the call with
// an "empty" pattern; a workgroup publishes with ONE relaxed device-scope atomic
// 64-bit store, and one wave of each workgroup polls the M slots of its item in
// parallel (lane j reads slot j) with relaxed device-scope atomic loads until none
// is empty.  The pair is the only data that crosses workgroups, so no ordering with
// other memory traffic is needed.  Published NaNs are canonicalised so that a
// payload can never look like the empty pattern.
//
// Forward progress: the launch never exceeds the number of workgroups the device
// can hold at once (cluster_capacity(), from the occupancy query), so all members
// of a cluster are resident together and the wait always ends.  As a second line of
// defence the wait gives up after kClusterMaxPolls polls and raises the error word
// in the workspace instead of spinning forever; results are then undefined but
// every wave still exits.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <map>
#include <mutex>
#include <utility>

namespace lbn {

constexpr int kClusterThreads = 256;  // workgroup size of the row-cluster (softmax) kernels
constexpr int kClusterMaxM = 64;  // one wave polls and merges the partials of an item
constexpr int kClusterMaxPolls = 1 << 21;
constexpr unsigned long long kSlotEmpty = ~0ull;

__device__ __forceinline__ unsigned long long cluster_pack(float a, float b)
{
  if (a != a) a = __builtin_nanf("");
  if (b != b) b = __builtin_nanf("");
  return (static_cast<unsigned long long>(__float_as_uint(b)) << 32) | __float_as_uint(a);
}

// Publishes the pair (a, b) of workgroup k; called by one lane.
__device__ __forceinline__ void cluster_publish(float a, float b, unsigned long long* slots, int k)
{
  __hip_atomic_store(slots + k, cluster_pack(a, b), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Called by all 64 lanes of ONE wave per workgroup (convergent).  Waits until the M
// slots of an item are published.  On return lane j < M holds the pair published by
// workgroup j in (ra, rb); lanes >= M hold (na, nb).
__device__ __forceinline__ void cluster_collect(unsigned long long* slots, int M, int* error_word,
                                                float na, float nb, float& ra, float& rb)
{
  const int lane = threadIdx.x & 63;
  unsigned long long raw = 0;
  int polls = 0;
  for (;;) {
    raw = lane < M ? __hip_atomic_load(slots + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0ull;
    if (__all(raw != kSlotEmpty)) break;
    if (++polls > kClusterMaxPolls) {
      if (lane == 0) __hip_atomic_store(error_word, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      break;
    }
    __builtin_amdgcn_s_sleep(1);
  }
  const bool have = lane < M && raw != kSlotEmpty;
  ra = have ? __uint_as_float(static_cast<unsigned>(raw)) : na;
  rb = have ? __uint_as_float(static_cast<unsigned>(raw >> 32)) : nb;
}

// Publish and collect in one go.
__device__ __forceinline__ void cluster_exchange(float a, float b, unsigned long long* slots, int k,
                                                 int M, int* error_word, float na, float nb,
                                                 float& ra, float& rb)
{
  if ((threadIdx.x & 63) == 0) cluster_publish(a, b, slots, k);
  cluster_collect(slots, M, error_word, na, nb, ra, rb);
}

// Marks `n` slots empty and clears the error word.
static __global__ void __launch_bounds__(256)
cluster_reset(unsigned long long* slots, int64_t n, int* error_word)
{
  const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i < n) slots[i] = kSlotEmpty;
  if (i == 0) *error_word = 0;
}

// Layout of the cluster part of a workspace: int error[16], then 64-bit slots.
struct ClusterWorkspace {
  int* error;
  unsigned long long* slots;
};

inline size_t cluster_workspace_bytes(int64_t items)
{
  return 64 + static_cast<size_t>(items) * kClusterMaxM * sizeof(unsigned long long);
}

inline ClusterWorkspace cluster_workspace(void* ws)
{
  char* base = static_cast<char*>(ws);
  return {reinterpret_cast<int*>(base), reinterpret_cast<unsigned long long*>(base + 64)};
}

inline void launch_cluster_reset(hipStream_t st, const ClusterWorkspace& cw, int64_t nslots)
{
  hipLaunchKernelGGL(cluster_reset, dim3(static_cast<unsigned>((nslots + 255) / 256)), dim3(256), 0, st,
                     cw.slots, nslots, cw.error);
}

// Cluster shape for an item of E 16-byte vectors: V vectors per thread (<= max_v), M
// workgroups of kClusterThreads per item (<= kClusterMaxM); M == 0: does not fit.
struct ClusterPlan {
  int V, M;
};

inline ClusterPlan plan_cluster(int64_t E, int max_v, int threads = kClusterThreads)
{
  const int64_t per_v = threads;
  const int64_t M = (E + per_v * max_v - 1) / (per_v * max_v);
  if (M > kClusterMaxM || M < 1) return {0, 0};
  const int64_t V = (E + per_v * M - 1) / (per_v * M);
  return {static_cast<int>(V), static_cast<int>(M)};
}

// Workgroups of `threads` threads running `kernel` that the current device holds at
// once.  Queried once per (kernel, device); the cache is the only process-wide
// state of the library and holds hardware facts only.
template <typename K>
inline int cluster_capacity(K kernel, int threads)
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
