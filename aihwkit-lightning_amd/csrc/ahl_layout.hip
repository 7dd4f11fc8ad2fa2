// Padded tile layout: copies between a dense [rows, K] matrix and the layout in which every
// K-tile starts on a multiple of `stride` columns (a multiple of 256) and is zero-filled up to the
// next tile. The MFMA kernels of the bf16 path need tile starts on their block boundaries; with
// this layout they serve every split the reference's rule produces, not only the aligned ones.
//
// Both copies are HBM-bound. Tile starts of a dense row are in general only element-aligned, so
// both sides are accessed one element per lane with consecutive lanes on consecutive elements:
// every wave instruction still covers one contiguous 128- or 256-byte span, and eight
// independent accesses per thread keep enough of them in flight.
#include "ahl_host.h"

namespace ahl {

static constexpr int kCopyUnroll = 8;
static constexpr int kCopySpan = 256 * kCopyUnroll;  // columns per block

// one block: 2048 consecutive padded columns of one row
template <class E>
__global__ __launch_bounds__(256) void k_pad_tiles(const E* __restrict__ src, int64_t ld_src,
                                                   E* __restrict__ dst, int64_t ld_dst,
                                                   Tiling tl, int32_t stride, int32_t spans) {
  const int64_t row = blockIdx.x / spans;
  const int32_t p0 = (int32_t)(blockIdx.x % spans) * kCopySpan + threadIdx.x;
  const int32_t padded = tl.n_tiles * stride;
  const E* s = src + row * ld_src;
  E* d = dst + row * ld_dst;
  E v[kCopyUnroll];
#pragma unroll
  for (int u = 0; u < kCopyUnroll; ++u) {
    const int32_t p = p0 + u * 256;
    v[u] = (E)0;
    if (p < padded) {
      const int32_t t = p / stride, j = p - t * stride;
      if (j < tl.size(t)) v[u] = s[tl.start(t) + j];
    }
  }
#pragma unroll
  for (int u = 0; u < kCopyUnroll; ++u) {
    const int32_t p = p0 + u * 256;
    if (p < padded) d[p] = v[u];
  }
}

// one block: 2048 consecutive dense columns of one row
template <class E>
__global__ __launch_bounds__(256) void k_unpad_tiles(const E* __restrict__ src, int64_t ld_src,
                                                     E* __restrict__ dst, int64_t ld_dst,
                                                     Tiling tl, int32_t stride, int32_t K,
                                                     int32_t spans) {
  const int64_t row = blockIdx.x / spans;
  const int32_t c0 = (int32_t)(blockIdx.x % spans) * kCopySpan + threadIdx.x;
  const E* s = src + row * ld_src;
  E* d = dst + row * ld_dst;
  E v[kCopyUnroll];
#pragma unroll
  for (int u = 0; u < kCopyUnroll; ++u) {
    const int32_t c = c0 + u * 256;
    v[u] = (E)0;
    if (c < K) {
      const int32_t t = tl.tile_of(c);
      v[u] = s[(int64_t)t * stride + (c - tl.start(t))];
    }
  }
#pragma unroll
  for (int u = 0; u < kCopyUnroll; ++u) {
    const int32_t c = c0 + u * 256;
    if (c < K) d[c] = v[u];
  }
}

int64_t padded_stride(int64_t K, int32_t n_tiles) {
  const int64_t widest = (K + n_tiles - 1) / n_tiles;
  return (widest + 255) / 256 * 256;
}

// Launchers shared with the backward entry points, which pad x and un-pad dx / dw internally.
int launch_pad_tiles(const void* src, int64_t ld_src, int32_t dtype, int64_t rows, const Tiling& tl,
                     int64_t stride, void* dst, int64_t ld_dst, hipStream_t s) {
  const int64_t padded = (int64_t)tl.n_tiles * stride;
  const int64_t spans = cdiv(padded, kCopySpan);
  if (padded > 0x7fffffff || rows * spans > 0x7fffffff) return AHL_ERR_UNSUPPORTED;
  const dim3 grid((unsigned)(rows * spans));
  if (dtype == AHL_F16) dtype = AHL_BF16;   // copies of 2-byte elements
  if (dtype == AHL_F32)
    hipLaunchKernelGGL((k_pad_tiles<uint32_t>), grid, dim3(256), 0, s, (const uint32_t*)src, ld_src,
                       (uint32_t*)dst, ld_dst, tl, (int32_t)stride, (int32_t)spans);
  else if (dtype == AHL_BF16)
    hipLaunchKernelGGL((k_pad_tiles<uint16_t>), grid, dim3(256), 0, s, (const uint16_t*)src, ld_src,
                       (uint16_t*)dst, ld_dst, tl, (int32_t)stride, (int32_t)spans);
  else
    return AHL_ERR_ARG;
  return check_launch("k_pad_tiles");
}

int launch_unpad_tiles(const void* src, int64_t ld_src, int32_t dtype, int64_t rows, int64_t K,
                       const Tiling& tl, int64_t stride, void* dst, int64_t ld_dst, hipStream_t s) {
  const int64_t spans = cdiv(K, kCopySpan);
  if ((int64_t)tl.n_tiles * stride > 0x7fffffff || rows * spans > 0x7fffffff)
    return AHL_ERR_UNSUPPORTED;
  const dim3 grid((unsigned)(rows * spans));
  if (dtype == AHL_F16) dtype = AHL_BF16;   // copies of 2-byte elements
  if (dtype == AHL_F32)
    hipLaunchKernelGGL((k_unpad_tiles<uint32_t>), grid, dim3(256), 0, s, (const uint32_t*)src,
                       ld_src, (uint32_t*)dst, ld_dst, tl, (int32_t)stride, (int32_t)K,
                       (int32_t)spans);
  else if (dtype == AHL_BF16)
    hipLaunchKernelGGL((k_unpad_tiles<uint16_t>), grid, dim3(256), 0, s, (const uint16_t*)src,
                       ld_src, (uint16_t*)dst, ld_dst, tl, (int32_t)stride, (int32_t)K,
                       (int32_t)spans);
  else
    return AHL_ERR_ARG;
  return check_launch("k_unpad_tiles");
}

}  // namespace ahl

using namespace ahl;

extern "C" int64_t ahl_tile_stride(int64_t K, int32_t n_tiles, int32_t dtype) {
  if (K <= 0 || n_tiles <= 0 || n_tiles > K || (dtype != AHL_BF16 && dtype != AHL_F16)) return 0;
  if (K % n_tiles == 0 && (K / n_tiles) % 256 == 0) return 0;  // dense tiles are aligned already
  return padded_stride(K, n_tiles);
}

static int check_layout_args(const void* src, const void* dst, int64_t rows, int64_t K,
                             const int32_t* ends, int32_t n_tiles, int64_t stride, Tiling* tl) {
  if (!src || !dst || rows <= 0 || K <= 0) return AHL_ERR_ARG;
  if (!make_tiling(ends, n_tiles, K, tl)) return AHL_ERR_TILING;
  if (stride <= 0 || stride % 256 != 0 || stride < widest_tile(*tl)) return AHL_ERR_ARG;
  return AHL_OK;
}

extern "C" int ahl_pad_tiles(const void* src, int64_t ld_src, int32_t dtype, int64_t rows,
                             int64_t K, const int32_t* tile_ends_host, int32_t n_tiles,
                             int64_t tile_stride, void* dst, int64_t ld_dst, void* stream) {
  Tiling tl;
  const int rc = check_layout_args(src, dst, rows, K, tile_ends_host, n_tiles, tile_stride, &tl);
  if (rc != AHL_OK) return rc;
  if (ld_src < K || ld_dst < (int64_t)n_tiles * tile_stride) return AHL_ERR_ARG;
  return launch_pad_tiles(src, ld_src, dtype, rows, tl, tile_stride, dst, ld_dst,
                          (hipStream_t)stream);
}

extern "C" int ahl_unpad_tiles(const void* src, int64_t ld_src, int32_t dtype, int64_t rows,
                               int64_t K, const int32_t* tile_ends_host, int32_t n_tiles,
                               int64_t tile_stride, void* dst, int64_t ld_dst, void* stream) {
  Tiling tl;
  const int rc = check_layout_args(src, dst, rows, K, tile_ends_host, n_tiles, tile_stride, &tl);
  if (rc != AHL_OK) return rc;
  if (ld_dst < K || ld_src < (int64_t)n_tiles * tile_stride) return AHL_ERR_ARG;
  return launch_unpad_tiles(src, ld_src, dtype, rows, K, tl, tile_stride, dst, ld_dst,
                            (hipStream_t)stream);
}
