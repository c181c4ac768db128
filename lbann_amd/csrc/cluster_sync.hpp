// Rendezvous of a cluster of M workgroups through device memory, used by the
// register-resident split reductions (batch norm channels, very wide softmax rows).
//
// Each workgroup of a cluster keeps its share of the data in registers, publishes
// one partial pair, waits until all M partials of the cluster are there, and then
// finishes from its registers: every tensor is read from memory exactly once.
//
// Protocol (no fences, no cache write-back or invalidation, no clearing pass): a slot
// is two 64-bit words, each holding one float of the pair and one half of a 64-bit
// call tag.  The tag is drawn per call from a process-wide counter (and, for a call that a
// HIP graph replays, advanced per replay through a counter word in the workspace), so
// whatever an earlier call (or anything else) left in the workspace can never look
// published: a slot counts only when both of its words carry the two halves of this
// call's tag.
// A workgroup publishes with two relaxed device-scope atomic 64-bit stores, and one
// wave of each workgroup polls the M slots of its item in parallel (lane j reads slot
// j) with relaxed device-scope atomic loads.  The pair is the only data that crosses
// workgroups, so no ordering with other memory traffic is needed.
//
// Forward progress: the launch never exceeds the number of workgroups the device
// can hold at once (cluster_capacity(), from the occupancy query), so all members
// of a cluster are resident together and the wait always ends.  As a second line of
// defence the wait gives up after kClusterMaxPolls polls and raises the (sticky)
// error word in the workspace (lbn_workspace_timed_out() reads it) instead of spinning
// forever; results are then undefined
// but every wave still exits.
#pragma once

#include <hip/hip_runtime.h>

#include <atomic>
#include <chrono>
#include <cstdint>
#include <mutex>
#include <thread>

#include "device_utils.hpp"
#include "host_utils.hpp"

namespace lbn {

constexpr int kClusterThreads = 256;  // workgroup size of the row-cluster (softmax) kernels
constexpr int kClusterMaxM = 64;  // one wave polls and merges the partials of an item
constexpr int kClusterMaxPolls = 1 << 21;
// Value of the workspace's first word after a wait ran out of polls (anything else,
// including whatever the memory held before, means that none did).
constexpr int kClusterTimedOut = 0x7E57FA11;

struct ClusterTag {
  unsigned lo, hi;
  // Null for an ordinary call.  A call recorded into a HIP graph repeats its arguments on
  // every replay, so there the tag also takes in a counter word in the workspace that a
  // one-thread kernel node in front of the cluster kernel advances (cluster_call_tag()).
  const unsigned long long* replay_word;
};

// A fresh tag per call.  The counter starts from the clock so that slots written by
// an earlier process into recycled device memory do not match either.
inline ClusterTag next_cluster_tag()
{
  static std::atomic<uint64_t> counter{
    static_cast<uint64_t>(std::chrono::steady_clock::now().time_since_epoch().count()) * 0x9E3779B97F4A7C15ull};
  const uint64_t v = counter.fetch_add(0x9E3779B97F4A7C15ull, std::memory_order_relaxed);
  return {static_cast<unsigned>(v), static_cast<unsigned>(v >> 32), nullptr};
}

// First thing a cluster kernel does with its tag: fold in the replay counter, if any.  All
// workgroups read the same value: the node that advances the word precedes the kernel.
__device__ __forceinline__ void cluster_resolve_tag(ClusterTag& tag)
{
  if (tag.replay_word) {
    const unsigned long long v = __hip_atomic_load(tag.replay_word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    tag.lo ^= static_cast<unsigned>(v);
    tag.hi ^= static_cast<unsigned>(v >> 32);
  }
}

// Whatever the word held before (the workspace is never cleared), successive replays see
// successive values; xor-ed with the recorded call's own tag they stay distinct from the
// tags of every other call that used this memory.
static __global__ void __launch_bounds__(64)
cluster_advance_replay_word(unsigned long long* word)
{
  if (threadIdx.x == 0) *word += 0x9E3779B97F4A7C15ull;
}

__device__ __forceinline__ unsigned long long cluster_word(float value, unsigned tag)
{
  return (static_cast<unsigned long long>(tag) << 32) | __float_as_uint(value);
}

// Publishes the pair (a, b) of workgroup k; called by one lane.
__device__ __forceinline__ void cluster_publish(float a, float b, unsigned long long* slots, int k,
                                                ClusterTag tag)
{
  __hip_atomic_store(slots + 2 * k, cluster_word(a, tag.lo), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __hip_atomic_store(slots + 2 * k + 1, cluster_word(b, tag.hi), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Called by all 64 lanes of ONE wave per workgroup (convergent).  Waits until the M
// slots of an item are published.  One poll at a time: keeping two or four polls in flight,
// to notice a publication sooner, was measured on the softmax clusters and is slower the
// deeper it goes (262144 x 16: 19.9 / 21.3 / 24.0 us per step at depths 1 / 2 / 4), like
// every other change that adds device-scope loads.  On return lane j < M holds the pair published by
// workgroup j in (ra, rb); lanes >= M hold (na, nb).
__device__ __forceinline__ void cluster_collect(unsigned long long* slots, int M, ClusterTag tag,
                                                int* error_word, float na, float nb, float& ra,
                                                float& rb, int max_polls = kClusterMaxPolls)
{
  const int lane = threadIdx.x & 63;
  unsigned long long wa = 0, wb = 0;
  bool have = false;
  int polls = 0;
  for (;;) {
    if (lane < M) {
      wa = __hip_atomic_load(slots + 2 * lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      wb = __hip_atomic_load(slots + 2 * lane + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      have = static_cast<unsigned>(wa >> 32) == tag.lo && static_cast<unsigned>(wb >> 32) == tag.hi;
    }
    if (__all(have || lane >= M)) break;
    if (++polls > max_polls) {
      if (lane == 0) __hip_atomic_store(error_word, kClusterTimedOut, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      break;
    }
    __builtin_amdgcn_s_sleep(1);
  }
  ra = have ? __uint_as_float(static_cast<unsigned>(wa)) : na;
  rb = have ? __uint_as_float(static_cast<unsigned>(wb)) : nb;
}

// The same for clusters of up to 2 x 64 members whose pairs are simply added: lane j polls
// slots j and j + 64; every lane returns the cluster's totals.  (Four slots per lane were
// measured: the extra registers of the polling wave cost the cluster kernels, which sit at
// the 128-register boundary, a factor of 1.3 to 3.)
constexpr int kClusterSumSlotsPerLane = 2;
constexpr int kClusterMaxSumM = 64 * kClusterSumSlotsPerLane;

// On the DPP path (device_utils.hpp): a butterfly of shuffles here cost layer norm over
// 64 huge rows 8 % of its time, the collecting wave being what every other wave waits for.
__device__ __forceinline__ float cluster_wave_total(float v) { return wave_sum(v); }

// ONE_SLOT_PATH: clusters of up to 64 take the one-slot loop (2.5 % on batch norm's usual
// shapes); kernels whose clusters are mostly larger leave it out and save its registers.
template <bool ONE_SLOT_PATH = true>
__device__ __forceinline__ void cluster_collect_sums(unsigned long long* slots, int M, ClusterTag tag,
                                                     int* error_word, float& ta, float& tb)
{
  if (ONE_SLOT_PATH && M <= 64) {
    float ra, rb;
    cluster_collect(slots, M, tag, error_word, 0.f, 0.f, ra, rb);
    ta = cluster_wave_total(ra);
    tb = cluster_wave_total(rb);
    return;
  }
  const int lane = threadIdx.x & 63;
  constexpr int H = kClusterSumSlotsPerLane;
  unsigned long long w[H][2];
  bool have[H];
#pragma unroll
  for (int h = 0; h < H; ++h) {
    w[h][0] = w[h][1] = 0;
    have[h] = false;
  }
  int polls = 0;
  for (;;) {
    bool all = true;
#pragma unroll
    for (int h = 0; h < H; ++h) {
      const int j = lane + 64 * h;
      if (j < M && !have[h]) {
        w[h][0] = __hip_atomic_load(slots + 2 * j, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        w[h][1] = __hip_atomic_load(slots + 2 * j + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        have[h] = static_cast<unsigned>(w[h][0] >> 32) == tag.lo && static_cast<unsigned>(w[h][1] >> 32) == tag.hi;
      }
      all = all && (have[h] || j >= M);
    }
    if (__all(all)) break;
    if (++polls > kClusterMaxPolls) {
      if (lane == 0) __hip_atomic_store(error_word, kClusterTimedOut, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      break;
    }
    __builtin_amdgcn_s_sleep(1);
  }
  float a = 0.f, b = 0.f;
#pragma unroll
  for (int h = 0; h < H; ++h) {
    if (have[h]) {
      a += __uint_as_float(static_cast<unsigned>(w[h][0]));
      b += __uint_as_float(static_cast<unsigned>(w[h][1]));
    }
  }
  ta = cluster_wave_total(a);
  tb = cluster_wave_total(b);
}

// ------------------------------------------------- waves that never meet at a barrier
// A variant of the cluster kernels keeps its waves free of workgroup barriers: a wave
// leaves its partial pair in LDS and counts itself in; the wave that arrives last adds the
// workgroup's pairs in wave order (so the result does not depend on which wave that was)
// and publishes them for the cluster; the first wave that needs the cluster's totals takes
// the polling duty and hands them to the others through LDS.  A fast wave is then never
// held back by the slowest wave of its workgroup, only by the data it needs.
//
// `count` and `claim` are never reset: a use of the stage is complete when they reach the
// next multiple of NW; `ready` counts completed hand-overs.  A stage may be reused for
// item i + 2 or later: a wave gets to item i + 2 only after it has seen item i published,
// which the last wave of item i does after it has read the stage.
template <int NW>
struct WaveMerge {
  float part[NW][2];
  unsigned count;
  unsigned claim, ready;
  float total[2];
};

// Zeroes the counters of `n` stages; the caller follows with the kernel's one barrier.
template <int NW>
__device__ __forceinline__ void wave_merge_init(WaveMerge<NW>* stages, int n)
{
  if (static_cast<int>(threadIdx.x) < n) stages[threadIdx.x].count = stages[threadIdx.x].claim = stages[threadIdx.x].ready = 0;
}

// Called by every wave of the workgroup once per item, with its pair valid in lane 63.
// True (in all lanes) in the wave that arrived last.
template <int NW>
__device__ __forceinline__ bool wave_merge_arrive(WaveMerge<NW>& st, float a, float b)
{
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = wave_index();
  unsigned prev = 0;
  if (lane == kWave - 1) {
    st.part[wave][0] = a;
    st.part[wave][1] = b;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");  // LDS only: no wait for global memory
    prev = __hip_atomic_fetch_add(&st.count, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  }
  prev = static_cast<unsigned>(__builtin_amdgcn_readlane(static_cast<int>(prev), kWave - 1));
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
  return prev % NW == NW - 1;
}

// Finish side with one polling wave per workgroup: the first wave to ask takes the duty
// (true), polls the cluster, and hands the totals to the others through LDS; `use` counts
// the earlier uses of the stage.
template <int NW>
__device__ __forceinline__ bool wave_merge_claim(WaveMerge<NW>& st)
{
  unsigned prev = 0;
  if ((threadIdx.x & (kWave - 1)) == kWave - 1)
    prev = __hip_atomic_fetch_add(&st.claim, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  prev = static_cast<unsigned>(__builtin_amdgcn_readlane(static_cast<int>(prev), kWave - 1));
  return prev % NW == 0;
}

template <int NW>
__device__ __forceinline__ void wave_merge_broadcast(WaveMerge<NW>& st, unsigned use, float a, float b)
{
  if ((threadIdx.x & (kWave - 1)) == 0) {
    st.total[0] = a;
    st.total[1] = b;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __hip_atomic_store(&st.ready, use + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  }
}

template <int NW>
__device__ __forceinline__ void wave_merge_wait(WaveMerge<NW>& st, unsigned use, int* error_word, float& a, float& b)
{
  // The polling wave gives up after kClusterMaxPolls rounds and still broadcasts, so this loop
  // ends with it; it also has a bound of its own (the polling wave's budget and as much again,
  // an LDS poll being shorter than a device-scope one) and raises the error word past it.
  int polls = 0;
  while (__hip_atomic_load(&st.ready, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) != use + 1) {
    if (++polls > 2 * kClusterMaxPolls) {
      if ((threadIdx.x & (kWave - 1)) == 0)
        __hip_atomic_store(error_word, kClusterTimedOut, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      break;
    }
    __builtin_amdgcn_s_sleep(1);
  }
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
  a = st.total[0];
  b = st.total[1];
}

// In the last wave: lane j < NW gets the pair of wave j, the other lanes (na, nb).
template <int NW>
__device__ __forceinline__ void wave_merge_read(const WaveMerge<NW>& st, float na, float nb, float& a, float& b)
{
  static_assert(NW <= kWave, "one lane per wave of the workgroup");
  const int lane = threadIdx.x & (kWave - 1);
  a = lane < NW ? st.part[lane][0] : na;
  b = lane < NW ? st.part[lane][1] : nb;
}

// One round of polling loads of a cluster's M slots, H slots per lane (lane j takes slots
// j, j + 64, ...), without waiting for them: issued ahead of other loads, the words are
// back first (a wave's loads return in order).
template <int H>
struct ClusterPoll {
  unsigned long long w[H][2];
};

template <int H>
__device__ __forceinline__ void cluster_poll_issue(ClusterPoll<H>& p, const unsigned long long* slots, int M)
{
  const int lane = threadIdx.x & (kWave - 1);
#pragma unroll
  for (int h = 0; h < H; ++h) {
    const int j = lane + kWave * h;
    p.w[h][0] = p.w[h][1] = 0;
    if (j < M) {
      p.w[h][0] = __hip_atomic_load(slots + 2 * j, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      p.w[h][1] = __hip_atomic_load(slots + 2 * j + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

// Completes a poll begun with cluster_poll_issue(): polls again until all M slots carry the
// call's tag (bounded as in cluster_collect()).  On return have[h] tells whether lane j's
// slot j + 64 h holds a published pair, in the low halves of p.w[h].
template <int H>
__device__ __forceinline__ void cluster_poll_complete(ClusterPoll<H>& p, const unsigned long long* slots, int M,
                                                      ClusterTag tag, int* error_word, bool (&have)[H])
{
  const int lane = threadIdx.x & (kWave - 1);
  int polls = 0;
  for (;;) {
    bool all = true;
#pragma unroll
    for (int h = 0; h < H; ++h) {
      have[h] = static_cast<unsigned>(p.w[h][0] >> 32) == tag.lo && static_cast<unsigned>(p.w[h][1] >> 32) == tag.hi;
      all = all && (have[h] || lane + kWave * h >= M);
    }
    if (__all(all)) break;
    if (++polls > kClusterMaxPolls) {
      if (lane == 0) __hip_atomic_store(error_word, kClusterTimedOut, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      break;
    }
    __builtin_amdgcn_s_sleep(1);
#pragma unroll
    for (int h = 0; h < H; ++h) {
      const int j = lane + kWave * h;
      if (j < M && !have[h]) {
        p.w[h][0] = __hip_atomic_load(slots + 2 * j, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        p.w[h][1] = __hip_atomic_load(slots + 2 * j + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
  }
}

// Completes a one-slot-per-lane poll: lane j < M returns the pair workgroup j published, the
// other lanes (na, nb), like cluster_collect().
__device__ __forceinline__ void cluster_poll_pairs(ClusterPoll<1>& p, const unsigned long long* slots, int M,
                                                   ClusterTag tag, int* error_word, float na, float nb, float& ra,
                                                   float& rb)
{
  bool have[1];
  cluster_poll_complete<1>(p, slots, M, tag, error_word, have);
  ra = have[0] ? __uint_as_float(static_cast<unsigned>(p.w[0][0])) : na;
  rb = have[0] ? __uint_as_float(static_cast<unsigned>(p.w[0][1])) : nb;
}

// The cluster's totals of pairs that are simply added; every lane returns them.
template <int H>
__device__ __forceinline__ void cluster_poll_sums(ClusterPoll<H>& p, const unsigned long long* slots, int M,
                                                  ClusterTag tag, int* error_word, float& ta, float& tb)
{
  bool have[H];
  cluster_poll_complete<H>(p, slots, M, tag, error_word, have);
  float a = 0.f, b = 0.f;
#pragma unroll
  for (int h = 0; h < H; ++h) {
    if (have[h]) {
      a += __uint_as_float(static_cast<unsigned>(p.w[h][0]));
      b += __uint_as_float(static_cast<unsigned>(p.w[h][1]));
    }
  }
  ta = cluster_wave_total(a);
  tb = cluster_wave_total(b);
}

// Clusters of up to 2 x 64 members: two one-slot-per-lane polls, the second only when
// M > 64.  (One loop over two slots per lane costs the compiler's register coalescer
// several seconds per kernel; two plain loops cost nothing.)
struct ClusterPollWide {
  ClusterPoll<1> lo, hi;
};

__device__ __forceinline__ void cluster_poll_issue(ClusterPollWide& p, const unsigned long long* slots, int M)
{
  cluster_poll_issue(p.lo, slots, M < kWave ? M : kWave);
  if (M > kWave) cluster_poll_issue(p.hi, slots + 2 * kWave, M - kWave);
}

__device__ __forceinline__ void cluster_poll_sums(ClusterPollWide& p, const unsigned long long* slots, int M,
                                                  ClusterTag tag, int* error_word, float& ta, float& tb)
{
  cluster_poll_sums(p.lo, slots, M < kWave ? M : kWave, tag, error_word, ta, tb);
  if (M > kWave) {
    float ha, hb;
    cluster_poll_sums(p.hi, slots + 2 * kWave, M - kWave, tag, error_word, ha, hb);
    ta += ha;
    tb += hb;
  }
}

// Publish and collect in one go.
__device__ __forceinline__ void cluster_exchange(float a, float b, unsigned long long* slots, int k,
                                                 int M, ClusterTag tag, int* error_word, float na,
                                                 float nb, float& ra, float& rb)
{
  if ((threadIdx.x & 63) == 0) cluster_publish(a, b, slots, k, tag);
  cluster_collect(slots, M, tag, error_word, na, nb, ra, rb);
}

// Layout of a workspace: 64 bytes of header (error word at byte 0, replay counter at byte 8)
// that only the cluster kernels write, then the call's scratch: two 64-bit words per slot for
// a cluster kernel, partial sums for the multi-kernel paths (workspace_payload()).  Keeping
// the partial sums out of the header means that a call which takes a multi-kernel path can
// neither clear a raised error word nor raise one by accident.
constexpr size_t kWorkspaceHeaderBytes = 64;

inline void* workspace_payload(void* ws) { return static_cast<char*>(ws) + kWorkspaceHeaderBytes; }
struct ClusterWorkspace {
  int* error;
  unsigned long long* replay_word;
  unsigned long long* slots;
};

inline size_t cluster_workspace_bytes(int64_t items, int max_m = kClusterMaxM)
{
  return 64 + static_cast<size_t>(items) * max_m * 2 * sizeof(unsigned long long);
}

inline ClusterWorkspace cluster_workspace(void* ws)
{
  char* base = static_cast<char*>(ws);
  return {reinterpret_cast<int*>(base), reinterpret_cast<unsigned long long*>(base + 8),
          reinterpret_cast<unsigned long long*>(base + 64)};
}

// The tag of one cluster call on stream `st`.  On a stream that is being recorded into a graph
// this also records the node that advances the workspace's replay counter.
inline ClusterTag cluster_call_tag(hipStream_t st, const ClusterWorkspace& cw)
{
  ClusterTag tag = next_cluster_tag();
  if (stream_is_capturing(st)) {
    hipLaunchKernelGGL(cluster_advance_replay_word, dim3(1), dim3(64), 0, st, cw.replay_word);
    tag.replay_word = cw.replay_word;
  }
  return tag;
}

// Keeps the cluster kernels of a device from running side by side.  A cluster kernel sizes its
// grid to what the device holds at once and its workgroups wait for each other: two of them
// started from different streams could each get part of the device and wait for workgroups that
// cannot be scheduled (the bounded waits would then give up and raise the error word).  One
// guard lives around every cluster launch: when the previous cluster launch of the device went
// to another stream, the new one is made to wait for it with an event; the guard also holds a
// mutex, so that launches from several host threads queue up one at a time.
//
// A process that only ever uses one stream for these calls pays nothing: events are recorded
// only from the moment a second stream shows up.  That launch records the event behind the
// earlier launch on the earlier launch's stream (which the guard remembers) and waits for it;
// nothing waits for the device.  The one exception: when the earlier stream was another host
// thread's hipStreamPerThread, which this thread cannot name, the launch waits for the device
// once.  Recording an event after every launch from the start was measured: about 3 us per kernel
// (262144 x 16 softmax 26.6 against 20.9 us per step).  Streams that are being recorded into a
// HIP graph are left alone: keeping graphs that contain cluster kernels from replaying side by
// side is up to the caller.
//
// failed(): the order could not be established (the event calls and the device-wide wait all
// returned errors, e.g. while another thread records a graph in global capture mode).  The
// caller then does not launch its cluster kernel and takes its multi-kernel path instead.
class ClusterLaunchGuard {
 public:
  explicit ClusterLaunchGuard(hipStream_t st) : st_(st), capturing_(stream_is_capturing(st))
  {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) dev = 0;
    state_ = &states()[dev];
    state_->mu.lock();
    if (capturing_ || !state_->have_last || same_stream_as_last()) return;
    if (!state_->several) {
      state_->several = true;
      make_event(*state_);
      // the earlier launch left no event: put one behind it now, on its own stream
      const bool nameable = state_->last != hipStreamPerThread || state_->last_thread == std::this_thread::get_id();
      if (state_->done && nameable && hipEventRecord(state_->done, state_->last) == hipSuccess &&
          hipStreamWaitEvent(st, state_->done, 0) == hipSuccess)
        return;
      wait_for_device();
    }
    else if (!state_->done || hipStreamWaitEvent(st, state_->done, 0) != hipSuccess) {
      wait_for_device();  // no event: order the launches the slow way
    }
  }
  ~ClusterLaunchGuard()
  {
    if (!capturing_ && !failed_) {
      if (state_->several && state_->done && hipEventRecord(state_->done, st_) != hipSuccess) {
        // the next launch from another stream must not trust a stale event
        (void)hipGetLastError();
        (void)hipEventDestroy(state_->done);
        state_->done = nullptr;
      }
      state_->last = st_;
      state_->have_last = true;
      if (st_ == hipStreamPerThread) state_->last_thread = std::this_thread::get_id();
    }
    state_->mu.unlock();
  }
  bool failed() const { return failed_; }
  ClusterLaunchGuard(const ClusterLaunchGuard&) = delete;
  ClusterLaunchGuard& operator=(const ClusterLaunchGuard&) = delete;

  // Creates the current device's event ahead of time, for callers that must not create
  // anything later (the entry point that allocates nothing does this in its set-up).
  static void prepare()
  {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) dev = 0;
    State& s = states()[dev];
    std::lock_guard<std::mutex> lock(s.mu);
    make_event(s);
  }

 private:
  static constexpr int kMaxDevices = 64;
  struct State {
    std::mutex mu;
    hipStream_t last = nullptr;
    std::thread::id last_thread;  // whose hipStreamPerThread `last` is, when it is that handle
    bool have_last = false;
    bool several = false;      // cluster launches have come from more than one stream
    hipEvent_t done = nullptr;  // recorded after every cluster launch once `several` is set
  };
  // hipStreamPerThread is one handle for a different stream in every host thread.
  bool same_stream_as_last() const
  {
    if (state_->last != st_) return false;
    return st_ != hipStreamPerThread || state_->last_thread == std::this_thread::get_id();
  }
  static State* states()
  {
    static State s[kMaxDevices];
    return s;
  }
  void wait_for_device()
  {
    (void)hipGetLastError();  // whatever the event calls left behind
    if (hipDeviceSynchronize() != hipSuccess) {
      (void)hipGetLastError();
      failed_ = true;
    }
  }
  static void make_event(State& s)
  {
    if (!s.done && hipEventCreateWithFlags(&s.done, hipEventDisableTiming) != hipSuccess) {
      (void)hipGetLastError();
      s.done = nullptr;
    }
  }
  hipStream_t st_;
  bool capturing_;
  bool failed_ = false;
  State* state_;
};

// Cluster shape for an item of E 16-byte vectors: V vectors per thread (<= max_v), M
// workgroups of kClusterThreads per item (<= kClusterMaxM); M == 0: does not fit.
struct ClusterPlan {
  int V, M;
};

inline ClusterPlan plan_cluster(int64_t E, int max_v, int threads = kClusterThreads, int max_m = kClusterMaxM)
{
  const int64_t per_v = threads;
  const int64_t M = (E + per_v * max_v - 1) / (per_v * max_v);
  if (M > max_m || M < 1) return {0, 0};
  const int64_t V = (E + per_v * M - 1) / (per_v * M);
  return {static_cast<int>(V), static_cast<int>(M)};
}

// Workgroups of `threads` threads running `kernel` that the current device holds at once.
template <typename K>
inline int cluster_capacity(K kernel, int threads)
{
  return resident_blocks(kernel, threads);
}

}  // namespace lbn
