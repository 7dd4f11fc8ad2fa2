// Reduction kernels used by more than one translation unit.
#pragma once
#include "ahl_device.h"

namespace ahl {

// ------------------------------------------------------------------------------------------
// out[t, r] = max_{c in tile t} |x[r, c]|. One wave per (row, tile), consecutive waves on
// consecutive tiles of a row; grid = ceil(rows * n_tiles / 4) blocks of 4 waves.
template <class D, bool VEC>
__global__ __launch_bounds__(256) void k_sliced_absmax(const void* __restrict__ x, int64_t rows,
                                                       int64_t ld, Tiling tl,
                                                       void* __restrict__ out) {
  const int lane = threadIdx.x & 63;
  const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int64_t r = wave / tl.n_tiles;
  const int32_t t = (int32_t)(wave % tl.n_tiles);
  if (r >= rows) return;
  const typename D::elem* row = (const typename D::elem*)x + r * ld;
  float m = 0.0f;
  wave_row_foreach<D, VEC>(row, tl.start(t), tl.start(t + 1), lane,
                           [&](float v) { m = fmaxf(m, fabsf(v)); });
  m = wave_max(m);
  if (lane == 0) D::store(out, (int64_t)t * rows + r, m);
}

// tile_max[t] = max_r v[t, r], tile_min[t] = min_r v[t, r]; one block per tile. The loads of a
// thread do not depend on each other: eight are in flight at a time (the kernel is a handful of
// blocks, so its duration is the latency of a thread's chain of loads).
template <class D>
__global__ __launch_bounds__(256) void k_tile_minmax(const void* __restrict__ v, int64_t rows,
                                                     float* __restrict__ tile_max,
                                                     float* __restrict__ tile_min) {
  __shared__ float smax[4], smin[4];
  const int t = blockIdx.x;
  float mx = 0.0f, mn = __builtin_inff();
  for (int64_t r0 = threadIdx.x; r0 < rows; r0 += 256 * 8) {
    float a[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int64_t r = r0 + 256 * u;
      a[u] = D::load(v, (int64_t)t * rows + (r < rows ? r : r0));  // r0 again: no effect on max / min
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      mx = fmaxf(mx, a[u]);
      mn = fminf(mn, a[u]);
    }
  }
  mx = wave_max(mx);
  mn = wave_min(mn);
  if ((threadIdx.x & 63) == 0) { smax[threadIdx.x >> 6] = mx; smin[threadIdx.x >> 6] = mn; }
  __syncthreads();
  if (threadIdx.x == 0) {
    tile_max[t] = fmaxf(fmaxf(smax[0], smax[1]), fmaxf(smax[2], smax[3]));
    tile_min[t] = fminf(fminf(smin[0], smin[1]), fminf(smin[2], smin[3]));
  }
}

// p[0..n) = v (a fill kernel instead of a memset node, so callers may capture it in a graph)
__attribute__((unused)) static __global__ void k_fill_u32(uint32_t* p, uint32_t v, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = v;
}

// kept[r] = 1 unless every element of row r is zero (-0.0 counts as zero, NaN does not);
// *n_kept += number of kept rows (n_kept may be null: flags only). One wave per row, one atomic
// per block (atomics on one address are served one after the other: a per-row atomic cost more
// than reading the rows).
template <class D, bool VEC>
__global__ __launch_bounds__(256) void k_row_nonzero(const void* __restrict__ x, int64_t rows,
                                                     int64_t cols, int64_t ld,
                                                     uint8_t* __restrict__ kept,
                                                     uint32_t* __restrict__ n_kept) {
  __shared__ uint32_t wave_kept[4];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t r = (int64_t)blockIdx.x * 4 + wave;
  bool keep = false;
  if (r < rows) {
    const typename D::elem* row = (const typename D::elem*)x + r * ld;
    bool any = false;
    wave_row_foreach_n<D, VEC, 4>(row, 0, (int32_t)cols, lane, [&](float v) { any |= (v != 0.0f); });
    keep = __builtin_amdgcn_ballot_w64(any) != 0ull;
    if (lane == 0) kept[r] = keep ? 1 : 0;
  }
  if (lane == 0) wave_kept[wave] = keep ? 1u : 0u;
  __syncthreads();
  if (threadIdx.x == 0) {
    const uint32_t n = wave_kept[0] + wave_kept[1] + wave_kept[2] + wave_kept[3];
    if (n && n_kept != nullptr) atomicAdd(n_kept, n);
  }
}

}  // namespace ahl
