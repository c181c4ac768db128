// Softmax family: rows shared by a cluster of workgroups that keep them in registers and
// exchange one partial pair through memory (cluster_sync.hpp).  Included by softmax.hip.
#pragma once

#include "cluster_sync.hpp"
#include "softmax_split.hpp"  // block_merge_max_sum

namespace lbn {

// ================================================ register-resident row clusters
// Rows too long for one workgroup's registers: a cluster of M workgroups shares a
// row, workgroup k keeps vectors [k*256*V, (k+1)*256*V) in registers, the cluster
// exchanges one (max, sum) pair per workgroup and every workgroup finishes from its
// registers.  One read and one write per element, and safe in place: a workgroup
// has read its whole share before it writes any of it, and shares are disjoint.
//
// The grid is persistent (cluster cl handles rows cl, cl + nclusters, ...) and rotates
// three register tiles so that nothing waits on something issued in the same step: in
// step s a workgroup (1) reduces tile s+1, whose loads were issued a step earlier, and
// publishes its partial pair, (2) issues the loads of tile s+2, (3) collects the
// cluster's partials of tile s, published a step earlier, and finishes tile s.
struct SmClusterArgs {
  const float* a;  // forward: x; backward: y
  const float* g;  // backward: dy
  float* out;
  int64_t lda, ldg, ldo;
  RowMap map;
  int64_t rows;
  unsigned nvec;
  unsigned n;  // framed access: entries per row (nvec is then the largest frame)
  int M;
  ClusterWorkspace cw;
  ClusterTag tag;
  __device__ __forceinline__ unsigned long long* slots(int64_t row) const { return cw.slots + row * M * 2; }
  // vectors of row `row` (every tensor has the same frames)
  template <bool FR>
  __device__ __forceinline__ unsigned row_nvec(int64_t row) const
  {
    return FR ? row_frame(a + map.offset(row, lda), n).nvec : nvec;
  }
};

template <int V, int W = 4>
struct SmFwdTile {
  float v[V][W];
  float m;  // the thread's own maximum: v holds exp(x - m) (or x - m for log-softmax)
};

template <int V, int W, bool FR = false>
__device__ __forceinline__ void sm_cl_load(float (&t)[V][W], const float* rowp, unsigned base,
                                           unsigned nvec, float fill, unsigned n = 0)
{
  static_assert(!FR || W == 4, "frames are made of 16-byte vectors");
  RowFrame fr{0, 0};
  if constexpr (FR) {
    fr = row_frame(rowp, n);
    rowp -= fr.shift;
    nvec = fr.nvec;
  }
#pragma unroll
  for (int i = 0; i < V; ++i) {
    const unsigned idx = base + i * kClusterThreads;
    if (idx < nvec) {
      if constexpr (FR) frame_load(rowp, idx, fr, n, fill, t[i]);
      else RowIO<float, W>::template load<false>(rowp + W * static_cast<int64_t>(idx), t[i]);
    }
    else {
#pragma unroll
      for (int j = 0; j < W; ++j) t[i][j] = fill;
    }
  }
}

// The entries are exponentiated here, in front of the publication, and only rescaled after the
// exchange.  Summing a two-operation exponential here and exponentiating against the row's
// maximum afterwards (less work before the partials can leave) was measured: no gain on
// 262144 x 16 or 262144 x 256, and rows read one float at a time lose a third (50257 x 1024
// forward 137 against 87 us).
// (1) of a step: thread-local online softmax, one merge of the (max, sum) pairs of the
// workgroup, published for the cluster.
template <int V, int KIND, int W = 4, bool FR = false>
__device__ __forceinline__ void sm_cl_fwd_reduce(const SmClusterArgs& a, int64_t row, int k, unsigned base,
                                                 SmFwdTile<V, W>& t, float (*red)[2])
{
  const unsigned nvec = a.row_nvec<FR>(row);
  float m = -FLT_MAX;
#pragma unroll
  for (int i = 0; i < V; ++i)
#pragma unroll
    for (int j = 0; j < W; ++j) m = fmaxf(m, t.v[i][j]);
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < V; ++i) {
    const bool ok = base + i * kClusterThreads < nvec;
#pragma unroll
    for (int j = 0; j < W; ++j) {
      const float d = t.v[i][j] - m;
      // (the entries of a frame's end vectors that lie outside the row hold -FLT_MAX: exp gives 0)
      const float e = ok ? (KIND == kChannelwise ? exp_keep_denormals(d) : exp_fast(d)) : 0.f;
      s += e;
      t.v[i][j] = (KIND == kLogSoftmax) ? d : e;
    }
  }
  t.m = m;
  block_merge_max_sum(m, s, red);
  if (threadIdx.x == 0) cluster_publish(m, s, a.slots(row), k, a.tag);
}

// (3) of a step.
// `poll` holds the polling loads for `row`, issued before the previous finish's stores (a wave's
// memory operations complete in order: a poll issued after stores waits for their acknowledgement);
// the loads for `next_row` (< 0: none) go out here, ahead of this row's stores.
template <int V, int KIND, int W = 4, bool FR = false>
__device__ __forceinline__ void sm_cl_fwd_finish(const SmClusterArgs& a, int64_t row, unsigned base,
                                                 SmFwdTile<V, W>& t, float* bc, ClusterPoll<1>& poll, int64_t next_row)
{
  if (threadIdx.x < kWave) {
    float pm, ps;
    cluster_poll_pairs(poll, a.slots(row), a.M, a.tag, a.cw.error, -FLT_MAX, 0.f, pm, ps);
    const float gmax = wave_max(pm);
    const float gsum = wave_sum(ps * exp_fast(pm - gmax));
    if (threadIdx.x == 0) {
      bc[0] = gmax;
      bc[1] = gsum;
    }
  }
  __syncthreads();
  const float gm = bc[0];
  const float gs = bc[1];
  if (next_row >= 0 && threadIdx.x < kWave) cluster_poll_issue(poll, a.slots(next_row), a.M);
  asm volatile("" ::: "memory");
  float* yr = a.out + a.map.offset(row, a.ldo);
  RowFrame fr{0, a.nvec};
  if constexpr (FR) {
    fr = row_frame(yr, a.n);
    yr -= fr.shift;
  }
  const float shift = t.m - gm;                     // <= 0: this thread's maximum against the row's
  const float f = exp_fast(shift) * (1.0f / gs);    // rescales exp(x - m) to exp(x - gm) / sum
  const float lse = (KIND == kLogSoftmax) ? log_of_sum(gs) : 0.f;
#pragma unroll
  for (int i = 0; i < V; ++i) {
    const unsigned idx = base + i * kClusterThreads;
    if (idx < fr.nvec) {
#pragma unroll
      for (int j = 0; j < W; ++j) {
        if (KIND == kSoftmax) {
          const float r = f * t.v[i][j];
          t.v[i][j] = __builtin_isnormal(r) ? r : 0.f;
        }
        else if (KIND == kLogSoftmax) {
          t.v[i][j] = (t.v[i][j] + shift) - lse;
        }
        else {
          t.v[i][j] *= f;
        }
      }
      if constexpr (FR) frame_store(yr, idx, fr, a.n, t.v[i]);
      else RowIO<float, W>::store(yr + W * static_cast<int64_t>(idx), t.v[i]);
    }
  }
}

template <int V, int KIND, int W = 4, bool FR = false>
__device__ __forceinline__ void sm_cl_fwd_step(const SmClusterArgs& a, int64_t row, int64_t nc, int k,
                                               unsigned base, SmFwdTile<V, W>& F, SmFwdTile<V, W>& R,
                                               SmFwdTile<V, W>& L, float (*red)[2], float* bc,
                                               ClusterPoll<1>& poll)
{
  if (row + nc < a.rows) sm_cl_fwd_reduce<V, KIND, W, FR>(a, row + nc, k, base, R, red);
  if (row + 2 * nc < a.rows)
    sm_cl_load<V, W, FR>(L.v, a.a + a.map.offset(row + 2 * nc, a.lda), base, a.nvec, -FLT_MAX, a.n);
  asm volatile("" ::: "memory");  // keep the loads above the wait below
  sm_cl_fwd_finish<V, KIND, W, FR>(a, row, base, F, bc, poll, row + nc < a.rows ? row + nc : -1);
}

template <int V, int KIND, int W = 4, bool FR = false>
__global__ void __launch_bounds__(kClusterThreads)
sm_fwd_cluster(SmClusterArgs a)
{
  __shared__ float red[kClusterThreads / kWave][2];
  __shared__ float bc[3][2];
  const int64_t nc = gridDim.x / a.M;
  const int64_t cl = blockIdx.x / a.M;
  const int k = blockIdx.x - static_cast<int>(cl) * a.M;
  const unsigned base = static_cast<unsigned>(k) * (kClusterThreads * V) + threadIdx.x;
  if (cl >= a.rows) return;
  cluster_resolve_tag(a.tag);
  SmFwdTile<V, W> t0, t1, t2;
  sm_cl_load<V, W, FR>(t0.v, a.a + a.map.offset(cl, a.lda), base, a.nvec, -FLT_MAX, a.n);
  if (cl + nc < a.rows) sm_cl_load<V, W, FR>(t1.v, a.a + a.map.offset(cl + nc, a.lda), base, a.nvec, -FLT_MAX, a.n);
  sm_cl_fwd_reduce<V, KIND, W, FR>(a, cl, k, base, t0, red);
  __syncthreads();  // the first step reduces again at once: every wave must have read `red` by then
  ClusterPoll<1> poll;
  if (threadIdx.x < kWave) cluster_poll_issue(poll, a.slots(cl), a.M);
  // Each position of the rotation has its own broadcast slot: a step without a reduction has
  // no barrier between the reads of one finish and the write of the next.
  for (int64_t row = cl; row < a.rows; row += 3 * nc) {
    sm_cl_fwd_step<V, KIND, W, FR>(a, row, nc, k, base, t0, t1, t2, red, bc[0], poll);
    if (row + nc < a.rows) sm_cl_fwd_step<V, KIND, W, FR>(a, row + nc, nc, k, base, t1, t2, t0, red, bc[1], poll);
    if (row + 2 * nc < a.rows)
      sm_cl_fwd_step<V, KIND, W, FR>(a, row + 2 * nc, nc, k, base, t2, t0, t1, red, bc[2], poll);
  }
}

template <int V, int W = 4>
struct SmBwdTile {
  float a[V][W];
  float g[V][W];
};

template <int V, int KIND, int W = 4>
__device__ __forceinline__ void sm_cl_bwd_reduce(const SmClusterArgs& a, int64_t row, int k,
                                                 const SmBwdTile<V, W>& t, float* red)
{
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < V; ++i)
#pragma unroll
    for (int j = 0; j < W; ++j) s += (KIND == kLogSoftmax) ? t.g[i][j] : t.a[i][j] * t.g[i][j];
  s = team_sum<kClusterThreads / kWave>(s, red, threadIdx.x / kWave, threadIdx.x & (kWave - 1));
  if (threadIdx.x == 0) cluster_publish(s, 0.f, a.slots(row), k, a.tag);
}

template <int V, int KIND, int W = 4, bool FR = false>
__device__ __forceinline__ void sm_cl_bwd_finish(const SmClusterArgs& a, int64_t row, unsigned base,
                                                 SmBwdTile<V, W>& t, float* bc, ClusterPoll<1>& poll, int64_t next_row)
{
  if (threadIdx.x < kWave) {
    float pt, unused;
    cluster_poll_pairs(poll, a.slots(row), a.M, a.tag, a.cw.error, 0.f, 0.f, pt, unused);
    pt = wave_sum(pt);
    if (threadIdx.x == 0) bc[0] = pt;
  }
  __syncthreads();
  const float tot = bc[0];
  if (next_row >= 0 && threadIdx.x < kWave) cluster_poll_issue(poll, a.slots(next_row), a.M);
  asm volatile("" ::: "memory");
  float* dr = a.out + a.map.offset(row, a.ldo);
  RowFrame fr{0, a.nvec};
  if constexpr (FR) {
    fr = row_frame(dr, a.n);
    dr -= fr.shift;
  }
#pragma unroll
  for (int i = 0; i < V; ++i) {
    const unsigned idx = base + i * kClusterThreads;
    if (idx < fr.nvec) {
#pragma unroll
      for (int j = 0; j < W; ++j) {
        if (KIND == kLogSoftmax) t.g[i][j] = t.g[i][j] - exp_fast(t.a[i][j]) * tot;
        else t.g[i][j] = t.a[i][j] * (t.g[i][j] - tot);
      }
      if constexpr (FR) frame_store(dr, idx, fr, a.n, t.g[i]);
      else RowIO<float, W>::store(dr + W * static_cast<int64_t>(idx), t.g[i]);
    }
  }
}

template <int V, int W, bool FR = false>
__device__ __forceinline__ void sm_cl_bwd_load(const SmClusterArgs& a, int64_t row, unsigned base,
                                               SmBwdTile<V, W>& t)
{
  sm_cl_load<V, W, FR>(t.a, a.a + a.map.offset(row, a.lda), base, a.nvec, 0.f, a.n);
  sm_cl_load<V, W, FR>(t.g, a.g + a.map.offset(row, a.ldg), base, a.nvec, 0.f, a.n);
}

template <int V, int KIND, int W = 4, bool FR = false>
__device__ __forceinline__ void sm_cl_bwd_step(const SmClusterArgs& a, int64_t row, int64_t nc, int k,
                                               unsigned base, SmBwdTile<V, W>& F, SmBwdTile<V, W>& R,
                                               SmBwdTile<V, W>& L, float* red, float* bc, ClusterPoll<1>& poll)
{
  if (row + nc < a.rows) sm_cl_bwd_reduce<V, KIND, W>(a, row + nc, k, R, red);
  if (row + 2 * nc < a.rows) sm_cl_bwd_load<V, W, FR>(a, row + 2 * nc, base, L);
  asm volatile("" ::: "memory");
  sm_cl_bwd_finish<V, KIND, W, FR>(a, row, base, F, bc, poll, row + nc < a.rows ? row + nc : -1);
}

template <int V, int KIND, int W = 4, bool FR = false>
__global__ void __launch_bounds__(kClusterThreads)
sm_bwd_cluster(SmClusterArgs a)
{
  __shared__ float red[kClusterThreads / kWave];
  __shared__ float bc[3][1];
  const int64_t nc = gridDim.x / a.M;
  const int64_t cl = blockIdx.x / a.M;
  const int k = blockIdx.x - static_cast<int>(cl) * a.M;
  const unsigned base = static_cast<unsigned>(k) * (kClusterThreads * V) + threadIdx.x;
  if (cl >= a.rows) return;
  cluster_resolve_tag(a.tag);
  SmBwdTile<V, W> t0, t1, t2;
  sm_cl_bwd_load<V, W, FR>(a, cl, base, t0);
  if (cl + nc < a.rows) sm_cl_bwd_load<V, W, FR>(a, cl + nc, base, t1);
  sm_cl_bwd_reduce<V, KIND, W>(a, cl, k, t0, red);
  __syncthreads();  // the first step reduces again at once: every wave must have read `red` by then
  ClusterPoll<1> poll;
  if (threadIdx.x < kWave) cluster_poll_issue(poll, a.slots(cl), a.M);
  // Each position of the rotation has its own broadcast slot: a step without a reduction has
  // no barrier between the reads of one finish and the write of the next.
  for (int64_t row = cl; row < a.rows; row += 3 * nc) {
    sm_cl_bwd_step<V, KIND, W, FR>(a, row, nc, k, base, t0, t1, t2, red, bc[0], poll);
    if (row + nc < a.rows) sm_cl_bwd_step<V, KIND, W, FR>(a, row + nc, nc, k, base, t1, t2, t0, red, bc[1], poll);
    if (row + 2 * nc < a.rows)
      sm_cl_bwd_step<V, KIND, W, FR>(a, row + 2 * nc, nc, k, base, t2, t0, t1, red, bc[2], poll);
  }
}

}  // namespace lbn
