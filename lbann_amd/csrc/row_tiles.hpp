// Tiling shared by the kernels whose lanes run along consecutive matrix ROWS (entry-wise
// scale/bias, batch norm over channels that are not a multiple of 4 entries): a 256-thread
// workgroup owns 256/GW rows; consecutive lanes take consecutive row quads (16 bytes of one
// column), the 4*GW column groups of the workgroup each walk every (4*GW)-th column of the
// workgroup's column slab, and per-row partial pairs of the groups are merged by lane
// exchange and one LDS hop in a fixed order.  Short matrices are cut into column slabs
// (grid.y) so that the launch still fills the device.
#pragma once

#include "device_utils.hpp"
#include "host_utils.hpp"

namespace lbn {

constexpr int kRowTileThreads = 256;
constexpr int kRowTileWaves = kRowTileThreads / kWave;
constexpr int kRowTileMaxSlabs = 64;

// Thread (row quad q, column group g) of a workgroup; GW column groups share a wave.
template <int GW>
struct RowTilePos {
  static constexpr int kQuads = kWave / GW;
  static constexpr int kRows = 4 * kQuads;
  static constexpr int kGroups = kRowTileWaves * GW;
  int q, g;
  __device__ __forceinline__ RowTilePos()
  {
    const int lane = threadIdx.x & (kWave - 1);
    q = lane & (kQuads - 1);
    g = lane / kQuads + GW * (threadIdx.x / kWave);
  }
};

// Adds the column groups' partial pairs (a, b) of each of the workgroup's rows.  Every
// thread of the workgroup must call; the totals of a thread's 4 rows are valid on return
// in the threads of column group 0 (p.g == 0) only.
template <int GW>
__device__ __forceinline__ void row_tile_merge(float (&a)[4], float (&b)[4],
                                               float (*lds)[RowTilePos<GW>::kRows][2],
                                               const RowTilePos<GW>& p)
{
  using P = RowTilePos<GW>;
  if (GW == 4) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      a[r] += __shfl_xor(a[r], 16);
      b[r] += __shfl_xor(b[r], 16);
      a[r] += __shfl_xor(a[r], 32);
      b[r] += __shfl_xor(b[r], 32);
    }
  }
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  if (lane < P::kQuads) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      lds[wave][4 * p.q + r][0] = a[r];
      lds[wave][4 * p.q + r][1] = b[r];
    }
  }
  __syncthreads();
  if (p.g != 0) return;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    float sa = 0.f, sb = 0.f;
#pragma unroll
    for (int k = 0; k < kRowTileWaves; ++k) {
      sa += lds[k][4 * p.q + r][0];
      sb += lds[k][4 * p.q + r][1];
    }
    a[r] = sa;
    b[r] = sb;
  }
}

// Launch shape.  Sixteen column groups over 64 rows (GW = 4) measured 4-8 % faster than
// four groups over 256 rows on 1048576 x 64 and 802816 x 64 matrices; mini-batches
// narrower than 16 columns would leave most of those groups idle and take GW = 1.
// Slabs: enough to give the device about four workgroups per compute unit, each slab at
// least one column per group wide.
struct RowTilePlan {
  int gw;
  int64_t tiles;
  int slabs;
  int64_t slab_width;
};

// 16-bit storage (a row quad is 8 bytes): with GW = 4 a wave's access touches four columns, 128
// bytes in each; tall matrices take GW = 1 there, 512 contiguous bytes of one column (batch norm
// on 64 x 111 x 111, w = 32: 65 / 68 -> 47 / 57 us; 96 x 55 x 55, w = 64: 37 / 49 -> 34 / 41), while
// 16384 rows x 512 columns have too few tiles of 256 rows for that (24 / 24 -> 33 / 37 us).
constexpr int64_t kRowTileTallRows = 65536;

inline RowTilePlan row_tile_plan(int64_t h, int64_t w, int elem_bytes = 4)
{
  RowTilePlan p;
  p.gw = (w >= 16 && !(elem_bytes == 2 && h >= kRowTileTallRows)) ? 4 : 1;
  p.tiles = ceil_div(h, p.gw == 1 ? RowTilePos<1>::kRows : RowTilePos<4>::kRows);
  const int64_t min_width = 4 * kRowTileWaves * p.gw;
  const int64_t want = ceil_div(1024, p.tiles);
  const int64_t most = w / min_width > 1 ? w / min_width : 1;
  int64_t s = want < most ? want : most;
  if (s > kRowTileMaxSlabs) s = kRowTileMaxSlabs;
  if (s < 1) s = 1;
  p.slab_width = ceil_div(w, s);
  p.slabs = static_cast<int>(ceil_div(w, p.slab_width));
  return p;
}

// Row quads (16 bytes of fp32, 8 bytes of fp16) need h % 4 == 0 and every column start aligned.
inline bool row_quads_ok(int64_t h, int64_t w, const void* p, int64_t ld, int elem_bytes = 4)
{
  return h % 4 == 0 && reinterpret_cast<uintptr_t>(p) % (4 * elem_bytes) == 0 && (w <= 1 || ld % 4 == 0);
}

}  // namespace lbn
