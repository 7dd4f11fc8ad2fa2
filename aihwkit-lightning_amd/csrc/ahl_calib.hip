// Statistics of the post-training input-range calibration that need more than a reduction
// (reference inference/calibration/calibration.py:57-152): the q-quantile of every K-tile of a
// batch over the rows that are not all zero, and the moving-average update of the ranges.
//
// The quantile is exact: torch.quantile's linear interpolation between the two neighbouring
// order statistics, which are found by a most-significant-digit radix selection on the
// order-preserving integer image of the fp32 values -- four histogram passes of 8 bits over the
// data (integer atomics only: deterministic). The successor of the selected value, which the
// interpolation needs, comes out of the last pass: it is the next non-empty bin of that pass's
// histogram, or else the smallest key whose upper 24 bits exceed the selected prefix, a minimum
// the last pass takes on the way.
// Seven launches: the row filter, the set-up, the four histogram passes, the interpolation;
// "which bin holds the rank" is worked out from the previous pass's histogram by every wave of
// the next pass for itself (a 256-bin prefix sum) rather than by a launch between.
// No sort, no copy of the data; everything stays on the device, so a calibration run never
// synchronises with the host.
#include "ahl_host.h"
#include "ahl_reduce_kernels.h"
#include <math.h>

namespace ahl {

// order-preserving map fp32 -> uint32 (negative values reversed below the positive ones)
AHL_DEV uint32_t f32_key(float v) {
  const uint32_t u = __float_as_uint(v);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
AHL_DEV float key_f32(uint32_t k) {
  return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}

// per-tile selection state; st[p][t] is the state in front of histogram pass p (after p digits)
struct SelState {
  uint32_t prefix;    // digits of the selected key found so far (right-aligned)
  uint32_t k_rem;     // rank of the wanted element among the elements that match the prefix
  uint32_t lo;        // rank of the lower order statistic
  uint32_t need_hi;   // the interpolation needs the next order statistic too
  float weight;       // interpolation weight of the upper order statistic
  uint32_t n_le;      // elements <= the selected value (set with the last digit)
  uint32_t n;         // elements of the tile over the kept rows
  uint32_t pad;
};
static_assert(sizeof(SelState) == 32, "layout");

// Set-up, one block per tile: the number of kept rows (a sum over the row flags), from it n,
// rank and weight -- rank = q * (n - 1) evaluated in fp32 as torch.quantile does for an fp32
// input (aten/src/ATen/native/Sorting.cpp quantile_compute) --, cleared histograms of all four
// passes, "no successor yet" and "no NaN seen".
__global__ __launch_bounds__(256) void k_select_init(SelState* st, uint32_t* hist, uint32_t* next_key,
                                                     uint32_t* has_nan, const uint8_t* __restrict__ kept,
                                                     int64_t rows, Tiling tl, float q) {
  __shared__ uint32_t part[4];
  const int t = blockIdx.x, i = threadIdx.x;
  const int32_t n_tiles = gridDim.x;
  for (int p = 0; p < 4; ++p) hist[((int64_t)p * n_tiles + t) * 256 + i] = 0u;
  uint32_t cnt = 0u;
  for (int64_t r = i; r < rows; r += 256) cnt += kept[r];
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) cnt += (uint32_t)__shfl_xor((int)cnt, off, 64);
  if ((i & 63) == 0) part[i >> 6] = cnt;
  __syncthreads();
  if (i != 0) return;
  next_key[t] = 0xffffffffu;
  has_nan[t] = 0u;
  const uint64_t n64 = (uint64_t)(part[0] + part[1] + part[2] + part[3]) * (uint64_t)tl.size(t);
  SelState s;
  s.n = (uint32_t)n64;
  s.prefix = 0u; s.n_le = 0u; s.pad = 0u;
  if (n64 == 0) { s.k_rem = 0u; s.lo = 0u; s.need_hi = 0u; s.weight = 0.0f; st[t] = s; return; }
  const float rank = q * (float)(n64 - 1);
  const float below = floorf(rank);
  s.lo = (uint32_t)below;
  s.k_rem = s.lo;
  s.weight = rank - below;
  s.need_hi = ceilf(rank) > below ? 1u : 0u;
  st[t] = s;
}

// The state after digit `pass`, from the state in front of it and the finished histogram of
// that pass, computed by one wave (every lane gets the result): the bin that holds rank k_rem
// -- the first of bins 0..254 whose running count exceeds the rank, bin 255 otherwise -- extends
// the prefix and rebases the rank. Lane l owns bins 4 l .. 4 l + 3.
AHL_DEV SelState wave_pick(const SelState& s0, const uint32_t* __restrict__ h, int pass, int lane) {
  if (s0.n == 0) return s0;
  uint32_t c[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) c[j] = h[4 * lane + j];
  const uint32_t mine = c[0] + c[1] + c[2] + c[3];
  uint32_t incl = mine;   // inclusive sum over lanes
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const uint32_t o = (uint32_t)__shfl_up((int)incl, off, 64);
    if (lane >= off) incl += o;
  }
  uint32_t excl = incl - mine, bin_excl = 0u, bin_c = 0u;
  int bin = -1;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int b = 4 * lane + j;
    if (bin < 0 && b < 255 && excl <= s0.k_rem && excl + c[j] > s0.k_rem) { bin = b; bin_excl = excl; bin_c = c[j]; }
    if (b == 255 && bin < 0) { bin_excl = excl; bin_c = c[j]; }   // lane 63 keeps bin 255 at hand
    excl += c[j];
  }
  const uint64_t found = __builtin_amdgcn_ballot_w64(bin >= 0);
  const int src = found ? __builtin_ctzll(found) : 63;
  const int pick = found ? __shfl(bin, src, 64) : 255;
  const uint32_t p_excl = (uint32_t)__shfl((int)bin_excl, src, 64);
  const uint32_t p_c = (uint32_t)__shfl((int)bin_c, src, 64);
  SelState s = s0;
  s.prefix = (s.prefix << 8) | (uint32_t)pick;
  s.k_rem -= p_excl;
  if (pass == 3) s.n_le = (s.lo - s.k_rem) + p_c;  // below + equal
  return s;
}

// Histogram of digit `pass` (0 = most significant byte) over the kept elements of every tile
// whose higher digits equal the tile's prefix. One wave per (group of rows, tile); per-wave
// histogram in LDS, then one integer atomic per non-empty bin.
template <class D, bool VEC>
__global__ __launch_bounds__(256) void k_select_hist(const void* __restrict__ x, int64_t rows,
                                                     int64_t ld, const uint8_t* __restrict__ kept,
                                                     Tiling tl, int rpw, int pass,
                                                     SelState* __restrict__ st,
                                                     uint32_t* __restrict__ hist,
                                                     uint32_t* __restrict__ has_nan,
                                                     uint32_t* __restrict__ next_key) {
  // eight copies of the wave's histogram, one per lane residue: the leading digits of real data
  // fall into a handful of bins, and a single copy would serialise the LDS atomics of a wave
  __shared__ uint32_t lh[4][8][256];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  for (int i = lane; i < 2048; i += 64) (&lh[w][0][0])[i] = 0u;
  uint32_t* mine = lh[w][lane & 7];
  const int64_t wave = (int64_t)blockIdx.x * 4 + w;
  const int64_t grp = wave / tl.n_tiles;
  const int32_t t = (int32_t)(wave % tl.n_tiles);
  const int64_t r0 = grp * rpw;
  if (r0 < rows) {  // no early return: nothing below synchronises across waves, but keep it simple
    SelState s = st[(int64_t)(pass > 0 ? pass - 1 : 0) * tl.n_tiles + t];
    if (pass > 0) {
      s = wave_pick(s, hist + ((int64_t)(pass - 1) * tl.n_tiles + t) * 256, pass - 1, lane);
      if (grp == 0 && lane == 0) st[(int64_t)pass * tl.n_tiles + t] = s;   // for the next launch
    }
    const uint32_t prefix = s.prefix;
    uint32_t* ht = hist + ((int64_t)pass * tl.n_tiles + t) * 256;
    const int shift = 24 - 8 * pass;
    bool nan = false;
    uint32_t above = 0xffffffffu;   // last pass: smallest key whose upper 24 bits exceed the prefix
    for (int i = 0; i < rpw; ++i) {
      const int64_t r = r0 + i;
      if (r >= rows) break;
      if (!kept[r]) continue;
      const typename D::elem* row = (const typename D::elem*)x + r * ld;
      wave_row_foreach<D, VEC>(row, tl.start(t), tl.start(t + 1), lane, [&](float v) {
        nan |= (v != v);
        const uint32_t key = f32_key(v);
        // digits above this pass must match the prefix found so far
        if (pass == 0 || (key >> (shift + 8)) == prefix) atomicAdd(&mine[(key >> shift) & 255u], 1u);
        if (pass == 3 && (key >> 8) > prefix && key < above) above = key;
      });
    }
    if (pass == 0 && __builtin_amdgcn_ballot_w64(nan) != 0ull && lane == 0) atomicOr(&has_nan[t], 1u);
    if (pass == 3) {
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) {
        const uint32_t o = (uint32_t)__shfl_xor((int)above, off, 64);
        above = o < above ? o : above;
      }
      if (lane == 0 && above < __hip_atomic_load(&next_key[t], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))
        atomicMin(&next_key[t], above);
    }
    for (int i = lane; i < 256; i += 64) {
      uint32_t c = 0u;
#pragma unroll
      for (int j = 0; j < 8; ++j) c += lh[w][j][i];
      if (c) atomicAdd(&ht[i], c);
    }
  }
}

// One wave per tile: the last digit, the successor of the selected key -- the next non-empty bin
// of the last histogram, else the smallest key beyond the prefix that the last pass left in
// next_key -- and out[t] = lerp(x_(lo), x_(lo+1), weight) with torch's two-sided lerp formula.
__global__ __launch_bounds__(64) void k_select_final(const SelState* st, const uint32_t* hist,
                                                     const uint32_t* next_key, const uint32_t* has_nan,
                                                     float* out) {
  const int t = blockIdx.x, lane = threadIdx.x;
  const int32_t n_tiles = gridDim.x;
  const uint32_t* h = hist + ((int64_t)3 * n_tiles + t) * 256;
  const SelState s = wave_pick(st[(int64_t)3 * n_tiles + t], h, 3, lane);
  if (s.n == 0 || has_nan[t]) {
    if (lane == 0) out[t] = __builtin_nanf("");
    return;
  }
  const int digit = (int)(s.prefix & 255u);
  int nb = 256;   // first non-empty bin above the selected digit among this lane's four
#pragma unroll
  for (int j = 3; j >= 0; --j)
    if (4 * lane + j > digit && h[4 * lane + j] != 0u) nb = 4 * lane + j;
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const int o = __shfl_xor(nb, off, 64);
    nb = o < nb ? o : nb;
  }
  const uint32_t succ = nb < 256 ? ((s.prefix & ~255u) | (uint32_t)nb) : next_key[t];
  if (lane != 0) return;
  const float lo = key_f32(s.prefix);
  float hi = lo;
  if (s.need_hi && s.n_le < s.lo + 2u && succ != 0xffffffffu) hi = key_f32(succ);
  const float w = s.weight, diff = hi - lo;
  out[t] = w < 0.5f ? lo + w * diff : hi - diff * (1.0f - w);
}

// input_range[t] <- (input_range[t] * idx[t] + val[t]) / (idx[t] + 1), idx[t] += 1: the moving
// average of calibration.py:126-147. The reference evaluates it on a 0-dim fp32 tensor (Python
// float times an int32 tensor element), then casts to the range's dtype.
template <class D>
__global__ void k_ir_moving_update(void* ir, int32_t* idx, const float* __restrict__ val,
                                   int32_t n_tiles, double alpha, int32_t val_in_dtype) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= n_tiles) return;
  const float old = D::load(ir, t);
  const int32_t i = idx[t];
  // the statistic as the Python float the reference holds: alpha * std (std in the tensor dtype)
  // or the fp32 quantile
  const float stat = val_in_dtype ? D::rd(val[t]) : val[t];
  // No statistic (NaN: no row of the batch was kept, e.g. the all-zero hidden state of a
  // recurrent layer's first step): the batch is passed over. The reference would average the
  // NaN in and lose the range for good.
  if (stat != stat) return;
  const float v = (float)(alpha * (double)stat);
  const float num = old * (float)i + v;
  D::store(ir, t, __fdiv_rn(num, (float)(i + 1)));
  idx[t] = i + 1;
}

// Rows per wave of the selection passes: every wave ends with one atomic per non-empty bin of
// its tile's histogram, and atomics on one address are served one after the other, so a few
// hundred waves per tile is the budget (the leading digit of real data fills a handful of bins).
static int select_rpw(int64_t rows) {
  const int64_t r = rows / 256;
  return (int)(r < 1 ? 1 : (r > 32 ? 32 : r));
}

}  // namespace ahl

using namespace ahl;

extern "C" {

// workspace: [SelState[4][T] | hist[4][T][256] | next_key[T] | has_nan[T] | kept flags, one byte per row]
static int64_t select_head_bytes(int32_t n_tiles) {
  return ((int64_t)n_tiles * (int64_t)(4 * sizeof(SelState) + 4 * 1024 + 8) + 255) / 256 * 256;
}

int64_t ahl_sliced_quantile_ws_bytes(int64_t rows, int32_t n_tiles) {
  if (rows <= 0 || n_tiles <= 0) return 0;
  return select_head_bytes(n_tiles) + rows;
}

int ahl_sliced_quantile(const void* x, int32_t dtype, int64_t rows, int64_t cols, int64_t ld,
                        const int32_t* tile_ends_host, int32_t n_tiles, float q, float* out,
                        void* ws, void* stream) {
  if (!x || !out || !ws || rows <= 0 || cols <= 0 || ld < cols) return AHL_ERR_ARG;
  if (!(q >= 0.0f && q <= 1.0f)) return AHL_ERR_ARG;
  Tiling tl;
  if (!make_tiling(tile_ends_host, n_tiles, cols, &tl)) return AHL_ERR_TILING;
  if (rows * (int64_t)widest_tile(tl) > 0xffffffffll) return AHL_ERR_UNSUPPORTED;
  hipStream_t s = (hipStream_t)stream;
  SelState* st = (SelState*)ws;
  uint32_t* hist = (uint32_t*)(st + 4 * (int64_t)n_tiles);
  uint32_t* next_key = hist + 4 * (int64_t)n_tiles * 256;
  uint32_t* has_nan = next_key + n_tiles;
  uint8_t* kept = (uint8_t*)ws + select_head_bytes(n_tiles);
  const int rpw = select_rpw(rows);
  const int64_t nb = cdiv(cdiv(rows, rpw) * n_tiles, 4);
  if (nb > 0x7fffffff || cdiv(rows, 4) > 0x7fffffff) return AHL_ERR_ARG;
  uint32_t* no_count = nullptr;   // the set-up kernel counts the kept rows from the flags
  AHL_DISPATCH_DTYPE(dtype, {
    const bool vec = aligned16(x) && (ld % D::EPV == 0);
    if (vec) hipLaunchKernelGGL((k_row_nonzero<D, true>), dim3((unsigned)cdiv(rows, 4)), dim3(256), 0, s, x, rows, cols, ld, kept, no_count);
    else hipLaunchKernelGGL((k_row_nonzero<D, false>), dim3((unsigned)cdiv(rows, 4)), dim3(256), 0, s, x, rows, cols, ld, kept, no_count);
    hipLaunchKernelGGL(k_select_init, dim3(n_tiles), dim3(256), 0, s, st, hist, next_key, has_nan, (const uint8_t*)kept, rows, tl, q);
    for (int pass = 0; pass < 4; ++pass) {
      if (vec) hipLaunchKernelGGL((k_select_hist<D, true>), dim3((unsigned)nb), dim3(256), 0, s, x, rows, ld, (const uint8_t*)kept, tl, rpw, pass, st, hist, has_nan, next_key);
      else hipLaunchKernelGGL((k_select_hist<D, false>), dim3((unsigned)nb), dim3(256), 0, s, x, rows, ld, (const uint8_t*)kept, tl, rpw, pass, st, hist, has_nan, next_key);
    }
  });
  hipLaunchKernelGGL(k_select_final, dim3((unsigned)n_tiles), dim3(64), 0, s, (const SelState*)st,
                     (const uint32_t*)hist, (const uint32_t*)next_key, (const uint32_t*)has_nan, out);
  return check_launch("ahl_sliced_quantile");
}

int ahl_row_nonzero(const void* x, int32_t dtype, int64_t rows, int64_t cols, int64_t ld,
                    uint8_t* kept, uint32_t* n_kept, void* stream) {
  if (!x || !kept || !n_kept || rows <= 0 || cols <= 0 || ld < cols) return AHL_ERR_ARG;
  if (cols > 0x7fffffff || cdiv(rows, 4) > 0x7fffffff) return AHL_ERR_UNSUPPORTED;
  hipStream_t s = (hipStream_t)stream;
  hipLaunchKernelGGL(k_fill_u32, dim3(1), dim3(64), 0, s, n_kept, 0u, 1);
  AHL_DISPATCH_DTYPE(dtype, {
    const bool vec = aligned16(x) && (ld % D::EPV == 0);
    if (vec) hipLaunchKernelGGL((k_row_nonzero<D, true>), dim3((unsigned)cdiv(rows, 4)), dim3(256), 0, s, x, rows, cols, ld, kept, n_kept);
    else hipLaunchKernelGGL((k_row_nonzero<D, false>), dim3((unsigned)cdiv(rows, 4)), dim3(256), 0, s, x, rows, cols, ld, kept, n_kept);
  });
  return check_launch("ahl_row_nonzero");
}

int ahl_ir_moving_update(void* ir, int32_t* idx, const float* val, int32_t dtype, int32_t n_tiles,
                         double alpha, int32_t val_in_dtype, void* stream) {
  if (!ir || !idx || !val || n_tiles <= 0) return AHL_ERR_ARG;
  AHL_DISPATCH_DTYPE(dtype, {
    hipLaunchKernelGGL((k_ir_moving_update<D>), dim3((unsigned)cdiv(n_tiles, 64)), dim3(64), 0,
                       (hipStream_t)stream, ir, idx, val, n_tiles, alpha, val_in_dtype);
  });
  return check_launch("ahl_ir_moving_update");
}

}  // extern "C"
