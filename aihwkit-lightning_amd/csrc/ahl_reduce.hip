// Memory-bound kernels of the AnalogLinear path: per-tile abs-max and std reductions, running
// abs-max (calibration), input-range initialisation, weight clipping, column sums, transposes.
// All are wave64 shuffle reductions over coalesced 16-byte row reads; none uses LDS for data
// except the transposes. Reductions are two-stage and deterministic (no float atomics).
#include "ahl_host.h"
#include "ahl_reduce_kernels.h"

namespace ahl {

__global__ void k_seed_advance(uint64_t* state, uint64_t delta) { state[1] += delta; }

static thread_local char g_err[256] = {0};
int record_hip_error(hipError_t e, const char* where) {
  snprintf(g_err, sizeof(g_err), "%s: %s", where, hipGetErrorString(e));
  return AHL_ERR_LAUNCH;
}

// ------------------------------------------------------------------------------------------
// Per-tile sum and sum of squares, in double. Every wave owns `rpw` consecutive rows and writes
// its own partial sums: no block-level synchronisation, and the grid has thousands of waves
// even for a few thousand rows. The summation order is fixed by (rows, rpw), so results are
// reproducible run to run.
static constexpr int kStdRows = 16;  // rows per block of the whole-matrix clip kernels below

// rows per wave: aim at >= 1024 groups of rows (times the number of tiles: waves), at most 16 rows
// each. Few fat waves with several rows' loads in flight finish a pass over a few tens of MB sooner
// than many thin ones (k_running_absmax_rows).
static int rows_per_wave(int64_t rows) {
  const int64_t r = rows / 1024;
  return (int)(r < 1 ? 1 : (r > 16 ? 16 : r));
}

template <class D, bool VEC>
__global__ __launch_bounds__(256) void k_sliced_sums(const void* __restrict__ x, int64_t rows,
                                                     int64_t ld, Tiling tl, int rpw,
                                                     double* __restrict__ partial) {
  const int lane = threadIdx.x & 63;
  // one wave per (group of rpw rows, tile): consecutive waves read consecutive tiles of a row
  const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int64_t grp = wave / tl.n_tiles;
  const int32_t t = (int32_t)(wave % tl.n_tiles);
  const int64_t r0 = grp * rpw;
  if (r0 >= rows) return;
  double s = 0.0, s2 = 0.0;
  for (int i = 0; i < rpw; ++i) {
    const int64_t r = r0 + i;
    if (r >= rows) break;
    const typename D::elem* row = (const typename D::elem*)x + r * ld;
    wave_row_foreach<D, VEC>(row, tl.start(t), tl.start(t + 1), lane, [&](float v) {
      s += (double)v;
      s2 += (double)v * (double)v;
    });
  }
  s = wave_sum(s);
  s2 = wave_sum(s2);
  if (lane == 0) {
    double* p = partial + wave * 2;  // == (grp * n_tiles + t) * 2
    p[0] = s;
    p[1] = s2;
  }
}

// The same partial sums for 16-byte aligned rows whose tiles are NV x 64 vectors wide, with all of a
// wave's RPW x NV loads issued before the first value is used (see k_running_absmax_rows). A lane
// adds its values in the same order as k_sliced_sums does (row by row, ascending columns), so the
// partial sums are the same to the bit.
template <class D, int RPW, int NV>
__global__ __launch_bounds__(256) void k_sliced_sums_rows(const void* __restrict__ x, int64_t rows,
                                                          int64_t ld, Tiling tl,
                                                          double* __restrict__ partial) {
  constexpr int E = D::EPV;
  const int lane = threadIdx.x & 63;
  const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int64_t grp = wave / tl.n_tiles;
  const int32_t t = (int32_t)(wave % tl.n_tiles);
  const int64_t r0 = grp * RPW;
  if (r0 >= rows) return;
  const typename D::elem* base = (const typename D::elem*)x + (int64_t)tl.base * t + lane * E;
  u32x4 v[RPW][NV];
#pragma unroll
  for (int i = 0; i < RPW; ++i) {
    const int64_t r = r0 + i < rows ? r0 + i : rows - 1;
#pragma unroll
    for (int j = 0; j < NV; ++j) v[i][j] = ld16_stream(base + r * ld + j * 64 * E);
  }
  double s = 0.0, s2 = 0.0;
#pragma unroll
  for (int i = 0; i < RPW; ++i) {
    if (r0 + i >= rows) break;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      float e[E];
      D::unpack(v[i][j], e);
#pragma unroll
      for (int q = 0; q < E; ++q) {
        s += (double)e[q];
        s2 += (double)e[q] * (double)e[q];
      }
    }
  }
  s = wave_sum(s);
  s2 = wave_sum(s2);
  if (lane == 0) {
    double* p = partial + wave * 2;
    p[0] = s;
    p[1] = s2;
  }
}

template <class D>
static void launch_sums_rows(int nv, int rpw, dim3 grid, hipStream_t s, const void* x, int64_t rows, int64_t ld,
                             const Tiling& tl, double* partial) {
#define AHL_SUMS(R, V) hipLaunchKernelGGL((k_sliced_sums_rows<D, R, V>), grid, dim3(256), 0, s, x, rows, ld, tl, partial)
  if (nv == 1) { if (rpw == 1) AHL_SUMS(1, 1); else if (rpw == 2) AHL_SUMS(2, 1); else AHL_SUMS(4, 1); }
  else { if (rpw == 1) AHL_SUMS(1, 2); else if (rpw == 2) AHL_SUMS(2, 2); else AHL_SUMS(4, 2); }
#undef AHL_SUMS
}

// out[t] = sqrt((S2 - S^2/n) / (n - 1)); one wave per tile, fixed summation order.
__global__ __launch_bounds__(256) void k_std_finalize(const double* __restrict__ partial,
                                                      int64_t n_blocks, int64_t rows, Tiling tl,
                                                      float* __restrict__ out,
                                                      const uint32_t* __restrict__ rows_kept) {
  __shared__ double sh[4][2];
  const int t = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  double s = 0.0, s2 = 0.0;
  const int64_t stride = (int64_t)tl.n_tiles * 2;
  const double* p = partial + (int64_t)t * 2;
  int64_t b = tid;
  for (; b + 768 < n_blocks; b += 1024) {  // four independent loads in flight per thread
    const double a0 = p[b * stride], a1 = p[(b + 256) * stride];
    const double a2 = p[(b + 512) * stride], a3 = p[(b + 768) * stride];
    const double q0 = p[b * stride + 1], q1 = p[(b + 256) * stride + 1];
    const double q2 = p[(b + 512) * stride + 1], q3 = p[(b + 768) * stride + 1];
    s += (a0 + a1) + (a2 + a3);
    s2 += (q0 + q1) + (q2 + q3);
  }
  for (; b < n_blocks; b += 256) {
    s += p[b * stride];
    s2 += p[b * stride + 1];
  }
  s = wave_sum(s);
  s2 = wave_sum(s2);
  if (lane == 0) { sh[wave][0] = s; sh[wave][1] = s2; }
  __syncthreads();
  if (tid == 0) {
    s = (sh[0][0] + sh[1][0]) + (sh[2][0] + sh[3][0]);
    s2 = (sh[0][1] + sh[1][1]) + (sh[2][1] + sh[3][1]);
    // all-zero rows add nothing to either sum: leaving them out only changes the count
    const double n = (double)(rows_kept ? (int64_t)*rows_kept : rows) * (double)tl.size(t);
    double var = (s2 - s * s / n) / (n - 1.0);  // n == 1 gives 0/0 = nan like torch
    if (var < 0.0) var = 0.0;
    out[t] = (float)sqrt(var);
  }
}

// ------------------------------------------------------------------------------------------
// Input-range initialisation from data (reference torch_utils/torch_linear.py:338-352).
template <class D>
__global__ void k_ir_init_update(void* ir, void* idx, const float* __restrict__ stdv, int32_t T,
                                 float init_from_data, float alpha) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= T) return;
  const float i = D::load(idx, t);
  if (!(i < init_from_data)) return;
  float r = D::load(ir, t);
  const float s = D::rd(stdv[t]);  // std() is returned in the tensor dtype
  if (s > 0.0f) {
    // float(ir) * idx + alpha * float(std), divided by (idx + 1) evaluated in the tensor dtype
    const float num = r * i + alpha * s;
    r = D::rd(__fdiv_rn(num, D::rd(i + 1.0f)));
    D::store(idx, t, D::rd(i + 1.0f));
  }
  D::store(ir, t, fabsf(r));
}

// ------------------------------------------------------------------------------------------
// cache[t] = max(cache[t], max over the block's rows and the tile's columns of |x|).
// Non-negative floats order like their int32 bit patterns, and -inf (the initial value) is a
// negative int, so a signed integer atomicMax implements the float max exactly.
template <class D, bool VEC>
__global__ __launch_bounds__(256) void k_running_absmax(const void* __restrict__ x, int64_t rows,
                                                        int64_t ld, Tiling tl, int rpw, float* cache) {
  const int lane = threadIdx.x & 63;
  const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int64_t grp = wave / tl.n_tiles;
  const int32_t t = (int32_t)(wave % tl.n_tiles);
  const int64_t r0 = grp * rpw;
  if (r0 >= rows) return;
  float m = 0.0f;
  for (int i = 0; i < rpw; ++i) {
    const int64_t r = r0 + i;
    if (r >= rows) break;
    const typename D::elem* row = (const typename D::elem*)x + r * ld;
    wave_row_foreach<D, VEC>(row, tl.start(t), tl.start(t + 1), lane,
                             [&](float v) { m = fmaxf(m, fabsf(v)); });
  }
  m = wave_max(m);
  // most waves find the cached maximum already above theirs and skip the atomic
  if (lane == 0 && __float_as_int(m) > __hip_atomic_load((int*)cache + t, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))
    atomicMax((int*)cache + t, __float_as_int(m));
}

// The same for 16-byte aligned rows whose tiles are NV x 64 vectors wide: a wave takes RPW rows of
// one tile and issues all its RPW x NV 16-byte loads before it uses the first value (a wave that
// walks its rows one after the other has one row's loads in flight, and a pass over a few tens of
// MB is over before such waves have covered the latency). Rows beyond the matrix re-read the last
// row: the maximum does not change. Measured at 2048 x 3072 fp32 (25 MB, launches replayed from a
// graph): 7.2 us with one row per wave, 5.7 / 5.9 / 6.1 us with RPW = 2 / 4 / 8.
template <class D, int RPW, int NV>
__global__ __launch_bounds__(256) void k_running_absmax_rows(const void* __restrict__ x, int64_t rows,
                                                             int64_t ld, Tiling tl, float* cache) {
  constexpr int E = D::EPV;
  const int lane = threadIdx.x & 63;
  const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int64_t grp = wave / tl.n_tiles;
  const int32_t t = (int32_t)(wave % tl.n_tiles);
  const int64_t r0 = grp * RPW;
  if (r0 >= rows) return;
  const typename D::elem* base = (const typename D::elem*)x + (int64_t)tl.base * t + lane * E;
  u32x4 v[RPW][NV];
#pragma unroll
  for (int i = 0; i < RPW; ++i) {
    const int64_t r = r0 + i < rows ? r0 + i : rows - 1;
#pragma unroll
    for (int j = 0; j < NV; ++j) v[i][j] = ld16_stream(base + r * ld + j * 64 * E);
  }
  float m = 0.0f;
#pragma unroll
  for (int i = 0; i < RPW; ++i)
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      float e[E];
      D::unpack(v[i][j], e);
#pragma unroll
      for (int q = 0; q < E; ++q) m = fmaxf(m, fabsf(e[q]));
    }
  m = wave_max(m);
  if (lane == 0 && __float_as_int(m) > __hip_atomic_load((int*)cache + t, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))
    atomicMax((int*)cache + t, __float_as_int(m));
}

// ------------------------------------------------------------------------------------------
// fast_mode input range (reference torch_utils/torch_linear.py:361-419).
// Stage 1: signed min and max of every (row group, tile), one wave each.
template <class D, bool VEC>
__global__ __launch_bounds__(256) void k_sliced_minmax(const void* __restrict__ x, int64_t rows,
                                                       int64_t ld, Tiling tl, int rpw,
                                                       float* __restrict__ partial) {
  const int lane = threadIdx.x & 63;
  const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int64_t grp = wave / tl.n_tiles;
  const int32_t t = (int32_t)(wave % tl.n_tiles);
  const int64_t r0 = grp * rpw;
  if (r0 >= rows) return;
  float mn = __builtin_inff(), mx = -__builtin_inff();
  for (int i = 0; i < rpw; ++i) {
    const int64_t r = r0 + i;
    if (r >= rows) break;
    const typename D::elem* row = (const typename D::elem*)x + r * ld;
    wave_row_foreach<D, VEC>(row, tl.start(t), tl.start(t + 1), lane, [&](float v) {
      mn = fminf(mn, v);
      mx = fmaxf(mx, v);
    });
  }
  mn = wave_min(mn);
  mx = wave_max(mx);
  if (lane == 0) { partial[wave * 2] = mn; partial[wave * 2 + 1] = mx; }
}

// Stage 2, one block per tile: finish the min / max, then the update of x_min, x_max, the step
// counter and the range, every operation rounded to the dtype of the buffers as torch does.
template <class D>
__global__ __launch_bounds__(256) void k_ir_fast_update(const float* __restrict__ partial,
                                                        int64_t n_groups, int32_t n_tiles, void* ir,
                                                        void* idx, void* x_min, void* x_max,
                                                        float init_from_data, float momentum,
                                                        float one_minus_momentum) {
  __shared__ float sh[4][2];
  const int t = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  float mn = __builtin_inff(), mx = -__builtin_inff();
  for (int64_t g = tid; g < n_groups; g += 256) {
    mn = fminf(mn, partial[(g * n_tiles + t) * 2]);
    mx = fmaxf(mx, partial[(g * n_tiles + t) * 2 + 1]);
  }
  mn = wave_min(mn);
  mx = wave_max(mx);
  if (lane == 0) { sh[wave][0] = mn; sh[wave][1] = mx; }
  __syncthreads();
  if (tid != 0) return;
  const float act_min = fminf(fminf(sh[0][0], sh[1][0]), fminf(sh[2][0], sh[3][0]));
  const float act_max = fmaxf(fmaxf(sh[0][1], sh[1][1]), fmaxf(sh[2][1], sh[3][1]));
  const float step = D::load(idx, t);
  if (!(step < init_from_data)) return;
  float lo = D::load(x_min, t), hi = D::load(x_max, t);
  const float thr = D::rd(1.1e-5f);  // the comparison constant takes the dtype of the buffer
  if (lo > -thr && hi < thr) {       // still at the initial +-1e-5: start from the first batch
    lo = D::rd(lo + act_min);
    hi = D::rd(hi + act_max);
  } else if (momentum == -1.0f) {    // plain running extrema
    lo = fminf(lo, act_min);
    hi = fmaxf(hi, act_max);
  } else {
    lo = D::rd(D::rd(lo * momentum) + D::rd(act_min * one_minus_momentum));
    hi = D::rd(D::rd(hi * momentum) + D::rd(act_max * one_minus_momentum));
  }
  D::store(x_min, t, lo);
  D::store(x_max, t, hi);
  D::store(idx, t, D::rd(step + 1.0f));
  D::store(ir, t, fmaxf(fabsf(lo), fabsf(hi)));
}

// ------------------------------------------------------------------------------------------
// Weight clipping. Per channel: one wave per row computes the unbiased std of the row in
// double, then re-reads the row (L2 resident) and stores only the 16-byte vectors in which
// at least one element changed.
template <class D, bool VEC>
AHL_DEV void clamp_row(void* rowp, int32_t cols, int lane, float bound) {
  typename D::elem* row = (typename D::elem*)rowp;
  if (VEC) {
    constexpr int E = D::EPV;
    const int32_t nv = cols / E;
    for (int32_t v = lane; v < nv; v += 64) {
      float e[E];
      D::unpack(ld16(row + (int64_t)v * E), e);
      bool changed = false;
#pragma unroll
      for (int i = 0; i < E; ++i) {
        const float c = fminf(fmaxf(e[i], -bound), bound);
        changed |= (c != e[i]);
        e[i] = c;
      }
      if (changed) st16(row + (int64_t)v * E, D::pack(e));
    }
    for (int32_t c = nv * E + lane; c < cols; c += 64) {
      const float a = D::load(row, c);
      const float b = fminf(fmaxf(a, -bound), bound);
      if (a != b) D::store(row, c, b);
    }
  } else {
    for (int32_t c = lane; c < cols; c += 64) {
      const float a = D::load(row, c);
      const float b = fminf(fmaxf(a, -bound), bound);
      if (a != b) D::store(row, c, b);
    }
  }
}

template <class D>
AHL_DEV float clip_bound(double s, double s2, double n, float sigma) {
  double var = (s2 - s * s / n) / (n - 1.0);
  if (var < 0.0) var = 0.0;
  const float sd = D::rd((float)sqrt(var));  // std() result in the tensor dtype
  return D::rd(sigma * sd);                 // python float * tensor
}

template <class D, bool VEC>
__global__ __launch_bounds__(256) void k_clip_rows(void* w, int64_t rows, int32_t cols, int64_t ld,
                                                   float sigma) {
  const int lane = threadIdx.x & 63;
  const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= rows) return;
  typename D::elem* row = (typename D::elem*)w + r * ld;
  double s = 0.0, s2 = 0.0;
  wave_row_foreach<D, VEC>(row, 0, cols, lane, [&](float v) {
    s += (double)v;
    s2 += (double)v * (double)v;
  });
  s = wave_sum(s);
  s2 = wave_sum(s2);
  const float bound = clip_bound<D>(s, s2, (double)cols, sigma);
  if (bound != bound) return;  // a one-element row has no unbiased std; leave it untouched
  clamp_row<D, VEC>(row, cols, lane, bound);
}

// Per channel, rows of at most 64 * R 16-byte vectors: the wave keeps its row in registers
// between the sums and the clamp, so the matrix is read once. All R loads are issued before the
// first value is used (vectors beyond the row re-read its first vector and count as zeros); sums
// in the order of k_clip_rows, so both kernels give the same bound bit for bit.
template <class D, int R>
__global__ __launch_bounds__(256) void k_clip_rows_held(void* w, int64_t rows, int32_t cols,
                                                        int64_t ld, float sigma) {
  constexpr int E = D::EPV;
  const int lane = threadIdx.x & 63;
  const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= rows) return;
  typename D::elem* row = (typename D::elem*)w + r * ld;
  const int32_t nv = cols / E;
  u32x4 held[R];
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int32_t v = lane + 64 * i;
    held[i] = ld16_stream(row + (int64_t)(v < nv ? v : 0) * E);
  }
  double s = 0.0, s2 = 0.0;
#pragma unroll
  for (int i = 0; i < R; ++i) {
    if (lane + 64 * i >= nv) {
      const u32x4 zero = {0u, 0u, 0u, 0u};
      held[i] = zero;
    }
    float e[E];
    D::unpack(held[i], e);
#pragma unroll
    for (int j = 0; j < E; ++j) {
      s += (double)e[j];
      s2 += (double)e[j] * (double)e[j];
    }
  }
  s = wave_sum(s);
  s2 = wave_sum(s2);
  const float bound = clip_bound<D>(s, s2, (double)cols, sigma);
  if (bound != bound) return;
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int32_t v = lane + 64 * i;
    float e[E];
    D::unpack(held[i], e);
    bool changed = false;
#pragma unroll
    for (int j = 0; j < E; ++j) {
      const float c = fminf(fmaxf(e[j], -bound), bound);
      changed |= (c != e[j]);
      e[j] = c;
    }
    if (changed && v < nv) st16(row + (int64_t)v * E, D::pack(e));
  }
}

// Whole-matrix variant, stage 1: per-block (sum, sum of squares) over kStdRows rows.
template <class D, bool VEC>
__global__ __launch_bounds__(256) void k_matrix_sums(const void* __restrict__ w, int64_t rows,
                                                     int32_t cols, int64_t ld,
                                                     double* __restrict__ partial) {
  __shared__ double sh[4][2];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t r0 = (int64_t)blockIdx.x * kStdRows;
  double s = 0.0, s2 = 0.0;
  for (int i = wave; i < kStdRows; i += 4) {
    const int64_t r = r0 + i;
    if (r >= rows) break;
    const typename D::elem* row = (const typename D::elem*)w + r * ld;
    wave_row_foreach<D, VEC>(row, 0, cols, lane, [&](float v) {
      s += (double)v;
      s2 += (double)v * (double)v;
    });
  }
  s = wave_sum(s);
  s2 = wave_sum(s2);
  if (lane == 0) { sh[wave][0] = s; sh[wave][1] = s2; }
  __syncthreads();
  if (threadIdx.x == 0) {
    partial[(int64_t)blockIdx.x * 2] = (sh[0][0] + sh[1][0]) + (sh[2][0] + sh[3][0]);
    partial[(int64_t)blockIdx.x * 2 + 1] = (sh[0][1] + sh[1][1]) + (sh[2][1] + sh[3][1]);
  }
}

// Stage 2: every block re-reduces the partials in the same fixed order, then clamps its rows.
template <class D, bool VEC>
__global__ __launch_bounds__(256) void k_clip_matrix(void* w, int64_t rows, int32_t cols,
                                                     int64_t ld, float sigma,
                                                     const double* __restrict__ partial,
                                                     int64_t n_partials) {
  __shared__ double sh[4][2];
  __shared__ float sbound;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  double s = 0.0, s2 = 0.0;
  for (int64_t b = threadIdx.x; b < n_partials; b += 256) {
    s += partial[b * 2];
    s2 += partial[b * 2 + 1];
  }
  s = wave_sum(s);
  s2 = wave_sum(s2);
  if (lane == 0) { sh[wave][0] = s; sh[wave][1] = s2; }
  __syncthreads();
  if (threadIdx.x == 0) {
    const double S = (sh[0][0] + sh[1][0]) + (sh[2][0] + sh[3][0]);
    const double S2 = (sh[0][1] + sh[1][1]) + (sh[2][1] + sh[3][1]);
    sbound = clip_bound<D>(S, S2, (double)rows * (double)cols, sigma);
  }
  __syncthreads();
  const float bound = sbound;
  if (bound != bound) return;
  const int64_t r0 = (int64_t)blockIdx.x * kStdRows;
  for (int i = wave; i < kStdRows; i += 4) {
    const int64_t r = r0 + i;
    if (r >= rows) break;
    clamp_row<D, VEC>((typename D::elem*)w + r * ld, cols, lane, bound);
  }
}

// ------------------------------------------------------------------------------------------
// Column sums, stage 1: partial[s, c] = sum over rows r = s (mod kColSplits) ... of x[r, c].
static constexpr int kColSplits = 64;

template <class D>
__global__ __launch_bounds__(256) void k_col_partial(const void* __restrict__ x, int64_t rows,
                                                     int64_t cols, int64_t ld,
                                                     float* __restrict__ partial) {
  const int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (c >= cols) return;
  const int64_t per = cdiv_dev(rows, kColSplits);
  const int64_t r0 = (int64_t)blockIdx.y * per;
  const int64_t r1 = r0 + per < rows ? r0 + per : rows;
  float s = 0.0f;
  for (int64_t r = r0; r < r1; ++r) s += D::load(x, r * ld + c);
  partial[(int64_t)blockIdx.y * cols + c] = s;
}

template <class D>
__global__ __launch_bounds__(256) void k_col_final(const float* __restrict__ partial, int64_t cols,
                                                   void* __restrict__ out) {
  const int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (c >= cols) return;
  float s = 0.0f;
  for (int i = 0; i < kColSplits; ++i) s += partial[(int64_t)i * cols + c];
  D::store(out, c, D::rd(s));
}

}  // namespace ahl

using namespace ahl;

// ============================================================================================
extern "C" {

int ahl_abi_version(void) { return 16; }

int ahl_seed_advance(uint64_t* state, uint64_t delta, void* stream) {
  if (!state) return AHL_ERR_ARG;
  hipLaunchKernelGGL(k_seed_advance, dim3(1), dim3(1), 0, (hipStream_t)stream, state, delta);
  return check_launch("ahl_seed_advance");
}
const char* ahl_last_hip_error(void) { return ahl::g_err; }

int ahl_sliced_absmax(const void* x, int32_t dtype, int64_t rows, int64_t cols, int64_t ld,
                      const int32_t* tile_ends_host, int32_t n_tiles, void* out, float* tile_max,
                      float* tile_min, void* stream) {
  if (!x || !out || rows <= 0 || cols <= 0 || ld < cols) return AHL_ERR_ARG;
  if ((tile_max == nullptr) != (tile_min == nullptr)) return AHL_ERR_ARG;
  Tiling tl;
  if (!make_tiling(tile_ends_host, n_tiles, cols, &tl)) return AHL_ERR_TILING;
  hipStream_t s = (hipStream_t)stream;
  if (cdiv(rows * n_tiles, 4) > 0x7fffffff) return AHL_ERR_ARG;
  const dim3 grid((unsigned)cdiv(rows * n_tiles, 4));
  AHL_DISPATCH_DTYPE(dtype, {
    const bool vec = aligned16(x) && (ld % D::EPV == 0);
    if (vec) hipLaunchKernelGGL((k_sliced_absmax<D, true>), grid, dim3(256), 0, s, x, rows, ld, tl, out);
    else hipLaunchKernelGGL((k_sliced_absmax<D, false>), grid, dim3(256), 0, s, x, rows, ld, tl, out);
    if (tile_max)
      hipLaunchKernelGGL((k_tile_minmax<D>), dim3(n_tiles), dim3(256), 0, s, out, rows, tile_max, tile_min);
  });
  return check_launch("ahl_sliced_absmax");
}

int64_t ahl_sliced_std_ws_bytes(int64_t rows, int32_t n_tiles) {
  if (rows <= 0 || n_tiles <= 0) return 0;
  return cdiv(rows, rows_per_wave(rows)) * (int64_t)n_tiles * 2 * (int64_t)sizeof(double);
}

int ahl_sliced_std(const void* x, int32_t dtype, int64_t rows, int64_t cols, int64_t ld,
                   const int32_t* tile_ends_host, int32_t n_tiles, float* out, void* ws_partials,
                   void* stream) {
  if (!x || !out || !ws_partials || rows <= 0 || cols <= 0 || ld < cols) return AHL_ERR_ARG;
  Tiling tl;
  if (!make_tiling(tile_ends_host, n_tiles, cols, &tl)) return AHL_ERR_TILING;
  hipStream_t s = (hipStream_t)stream;
  const int rpw = rows_per_wave(rows);
  const int64_t nw = cdiv(rows, rpw), nb = cdiv(nw * n_tiles, 4);
  if (nb > 0x7fffffff) return AHL_ERR_ARG;
  AHL_DISPATCH_DTYPE(dtype, {
    const bool vec = aligned16(x) && (ld % D::EPV == 0);
    // equal tiles of 64 or 128 vectors: the kernel with all of a wave's loads in flight (same
    // grouping of rows into waves, same sums)
    const int nv = (vec && tl.extra == 0 && tl.base % (64 * D::EPV) == 0) ? tl.base / (64 * D::EPV) : 0;
    if ((nv == 1 || nv == 2) && (rpw == 1 || rpw == 2 || rpw == 4)) {
      launch_sums_rows<D>(nv, rpw, dim3((unsigned)nb), s, x, rows, ld, tl, (double*)ws_partials);
    } else if (vec) {
      hipLaunchKernelGGL((k_sliced_sums<D, true>), dim3((unsigned)nb), dim3(256), 0, s, x, rows, ld, tl, rpw, (double*)ws_partials);
    } else {
      hipLaunchKernelGGL((k_sliced_sums<D, false>), dim3((unsigned)nb), dim3(256), 0, s, x, rows, ld, tl, rpw, (double*)ws_partials);
    }
  });
  hipLaunchKernelGGL(k_std_finalize, dim3(n_tiles), dim3(256), 0, s, (const double*)ws_partials, nw, rows, tl, out,
                     (const uint32_t*)nullptr);
  return check_launch("ahl_sliced_std");
}

// workspace: [partial sums of ahl_sliced_std | kept-row counter | kept flags, one byte per row]
int64_t ahl_sliced_std_kept_ws_bytes(int64_t rows, int32_t n_tiles) {
  return (ahl_sliced_std_ws_bytes(rows, n_tiles) + 255) / 256 * 256 + 256 + rows;
}

int ahl_sliced_std_kept(const void* x, int32_t dtype, int64_t rows, int64_t cols, int64_t ld,
                        const int32_t* tile_ends_host, int32_t n_tiles, float* out, void* ws,
                        void* stream) {
  if (!x || !out || !ws || rows <= 0 || cols <= 0 || ld < cols) return AHL_ERR_ARG;
  Tiling tl;
  if (!make_tiling(tile_ends_host, n_tiles, cols, &tl)) return AHL_ERR_TILING;
  hipStream_t s = (hipStream_t)stream;
  const int rpw = rows_per_wave(rows);
  const int64_t nw = cdiv(rows, rpw), nb = cdiv(nw * n_tiles, 4);
  if (nb > 0x7fffffff || cdiv(rows, 4) > 0x7fffffff) return AHL_ERR_ARG;
  double* partial = (double*)ws;
  uint32_t* n_kept = (uint32_t*)((char*)ws + (ahl_sliced_std_ws_bytes(rows, n_tiles) + 255) / 256 * 256);
  uint8_t* kept = (uint8_t*)n_kept + 256;
  hipLaunchKernelGGL(k_fill_u32, dim3(1), dim3(64), 0, s, n_kept, 0u, 1);
  AHL_DISPATCH_DTYPE(dtype, {
    const bool vec = aligned16(x) && (ld % D::EPV == 0);
    if (vec) {
      hipLaunchKernelGGL((k_row_nonzero<D, true>), dim3((unsigned)cdiv(rows, 4)), dim3(256), 0, s, x, rows, cols, ld, kept, n_kept);
      hipLaunchKernelGGL((k_sliced_sums<D, true>), dim3((unsigned)nb), dim3(256), 0, s, x, rows, ld, tl, rpw, partial);
    } else {
      hipLaunchKernelGGL((k_row_nonzero<D, false>), dim3((unsigned)cdiv(rows, 4)), dim3(256), 0, s, x, rows, cols, ld, kept, n_kept);
      hipLaunchKernelGGL((k_sliced_sums<D, false>), dim3((unsigned)nb), dim3(256), 0, s, x, rows, ld, tl, rpw, partial);
    }
  });
  hipLaunchKernelGGL(k_std_finalize, dim3(n_tiles), dim3(256), 0, s, (const double*)partial, nw, rows, tl, out,
                     (const uint32_t*)n_kept);
  return check_launch("ahl_sliced_std_kept");
}

int ahl_ir_init_update(void* ir, void* idx, const float* std, int32_t dtype, int32_t n_tiles,
                       float init_from_data, float init_std_alpha, void* stream) {
  if (!ir || !idx || !std || n_tiles <= 0) return AHL_ERR_ARG;
  hipStream_t s = (hipStream_t)stream;
  AHL_DISPATCH_DTYPE(dtype, {
    hipLaunchKernelGGL((k_ir_init_update<D>), dim3((unsigned)cdiv(n_tiles, 64)), dim3(64), 0, s, ir, idx, std, n_tiles, init_from_data, init_std_alpha);
  });
  return check_launch("ahl_ir_init_update");
}

int ahl_running_absmax(const void* x, int32_t dtype, int64_t rows, int64_t cols, int64_t ld,
                       const int32_t* tile_ends_host, int32_t n_tiles, float* cache, void* stream) {
  if (!x || !cache || rows <= 0 || cols <= 0 || ld < cols) return AHL_ERR_ARG;
  Tiling tl;
  if (!make_tiling(tile_ends_host, n_tiles, cols, &tl)) return AHL_ERR_TILING;
  hipStream_t s = (hipStream_t)stream;
  const int rpw = rows_per_wave(rows);
  const int64_t nb = cdiv(cdiv(rows, rpw) * n_tiles, 4);
  if (nb > 0x7fffffff) return AHL_ERR_ARG;
  AHL_DISPATCH_DTYPE(dtype, {
    const bool vec = aligned16(x) && (ld % D::EPV == 0);
    // equal tiles of 64 or 128 vectors (256 / 512 fp32, 512 / 1024 16-bit columns), many rows
    const int nv = (vec && tl.extra == 0 && tl.base % (64 * D::EPV) == 0) ? tl.base / (64 * D::EPV) : 0;
    if ((nv == 1 || nv == 2) && rows >= 512) {
      const int64_t nbr = cdiv(cdiv(rows, 2) * n_tiles, 4);
      if (nv == 1) hipLaunchKernelGGL((k_running_absmax_rows<D, 2, 1>), dim3((unsigned)nbr), dim3(256), 0, s, x, rows, ld, tl, cache);
      else hipLaunchKernelGGL((k_running_absmax_rows<D, 2, 2>), dim3((unsigned)nbr), dim3(256), 0, s, x, rows, ld, tl, cache);
    } else if (vec) {
      hipLaunchKernelGGL((k_running_absmax<D, true>), dim3((unsigned)nb), dim3(256), 0, s, x, rows, ld, tl, rpw, cache);
    } else {
      hipLaunchKernelGGL((k_running_absmax<D, false>), dim3((unsigned)nb), dim3(256), 0, s, x, rows, ld, tl, rpw, cache);
    }
  });
  return check_launch("ahl_running_absmax");
}

int64_t ahl_ir_fast_update_ws_bytes(int64_t rows, int32_t n_tiles) {
  if (rows <= 0 || n_tiles <= 0) return 0;
  return cdiv(rows, rows_per_wave(rows)) * (int64_t)n_tiles * 2 * (int64_t)sizeof(float);
}

int ahl_ir_fast_update(const void* x, int32_t dtype, int64_t rows, int64_t cols, int64_t ld,
                       const int32_t* tile_ends_host, int32_t n_tiles, void* ir, void* idx,
                       void* x_min, void* x_max, float init_from_data, double momentum, void* ws,
                       void* stream) {
  if (!x || !ir || !idx || !x_min || !x_max || !ws || rows <= 0 || cols <= 0 || ld < cols)
    return AHL_ERR_ARG;
  Tiling tl;
  if (!make_tiling(tile_ends_host, n_tiles, cols, &tl)) return AHL_ERR_TILING;
  hipStream_t s = (hipStream_t)stream;
  const int rpw = rows_per_wave(rows);
  const int64_t ng = cdiv(rows, rpw), nb = cdiv(ng * n_tiles, 4);
  if (nb > 0x7fffffff) return AHL_ERR_ARG;
  AHL_DISPATCH_DTYPE(dtype, {
    const bool vec = aligned16(x) && (ld % D::EPV == 0);
    if (vec) hipLaunchKernelGGL((k_sliced_minmax<D, true>), dim3((unsigned)nb), dim3(256), 0, s, x, rows, ld, tl, rpw, (float*)ws);
    else hipLaunchKernelGGL((k_sliced_minmax<D, false>), dim3((unsigned)nb), dim3(256), 0, s, x, rows, ld, tl, rpw, (float*)ws);
    hipLaunchKernelGGL((k_ir_fast_update<D>), dim3(n_tiles), dim3(256), 0, s, (const float*)ws, ng, n_tiles,
                       ir, idx, x_min, x_max, init_from_data, (float)momentum, (float)(1.0 - momentum));
  });
  return check_launch("ahl_ir_fast_update");
}

int64_t ahl_clip_weights_ws_bytes(int64_t rows) {
  return cdiv(rows, kStdRows) * 2 * (int64_t)sizeof(double);
}

int ahl_clip_weights(void* w, int32_t dtype, int64_t rows, int64_t cols, int64_t ld, float sigma,
                     int32_t clip_kind, void* ws, void* stream) {
  if (!w || rows <= 0 || cols <= 0 || cols > 0x7fffffff || ld < cols) return AHL_ERR_ARG;
  if (clip_kind != AHL_CLIP_LAYER && clip_kind != AHL_CLIP_PER_CHANNEL) return AHL_ERR_ARG;
  if (clip_kind == AHL_CLIP_LAYER && !ws) return AHL_ERR_WORKSPACE;
  hipStream_t s = (hipStream_t)stream;
  AHL_DISPATCH_DTYPE(dtype, {
    const bool vec = aligned16(w) && (ld % D::EPV == 0);
    if (clip_kind == AHL_CLIP_PER_CHANNEL) {
      const dim3 grid((unsigned)cdiv(rows, 4));
      const int64_t per_lane = cols % D::EPV == 0 ? cdiv(cols / D::EPV, 64) : 0;
      if (vec && per_lane >= 1 && per_lane <= 4)
        hipLaunchKernelGGL((k_clip_rows_held<D, 4>), grid, dim3(256), 0, s, w, rows, (int32_t)cols, ld, sigma);
      else if (vec && per_lane > 4 && per_lane <= 8)
        hipLaunchKernelGGL((k_clip_rows_held<D, 8>), grid, dim3(256), 0, s, w, rows, (int32_t)cols, ld, sigma);
      else if (vec && per_lane > 8 && per_lane <= 16)
        hipLaunchKernelGGL((k_clip_rows_held<D, 16>), grid, dim3(256), 0, s, w, rows, (int32_t)cols, ld, sigma);
      else if (vec && per_lane > 16 && per_lane <= 32)
        hipLaunchKernelGGL((k_clip_rows_held<D, 32>), grid, dim3(256), 0, s, w, rows, (int32_t)cols, ld, sigma);
      else if (vec) hipLaunchKernelGGL((k_clip_rows<D, true>), grid, dim3(256), 0, s, w, rows, (int32_t)cols, ld, sigma);
      else hipLaunchKernelGGL((k_clip_rows<D, false>), grid, dim3(256), 0, s, w, rows, (int32_t)cols, ld, sigma);
    } else {
      const int64_t nb = cdiv(rows, kStdRows);
      const dim3 grid((unsigned)nb);
      if (vec) {
        hipLaunchKernelGGL((k_matrix_sums<D, true>), grid, dim3(256), 0, s, w, rows, (int32_t)cols, ld, (double*)ws);
        hipLaunchKernelGGL((k_clip_matrix<D, true>), grid, dim3(256), 0, s, w, rows, (int32_t)cols, ld, sigma, (const double*)ws, nb);
      } else {
        hipLaunchKernelGGL((k_matrix_sums<D, false>), grid, dim3(256), 0, s, w, rows, (int32_t)cols, ld, (double*)ws);
        hipLaunchKernelGGL((k_clip_matrix<D, false>), grid, dim3(256), 0, s, w, rows, (int32_t)cols, ld, sigma, (const double*)ws, nb);
      }
    }
  });
  return check_launch("ahl_clip_weights");
}

int64_t ahl_col_sum_ws_bytes(int64_t cols) { return (int64_t)kColSplits * cols * (int64_t)sizeof(float); }

int ahl_col_sum(const void* x, int32_t dtype, int64_t rows, int64_t cols, int64_t ld, void* out,
                void* ws, void* stream) {
  if (!x || !out || !ws || rows <= 0 || cols <= 0 || ld < cols) return AHL_ERR_ARG;
  hipStream_t s = (hipStream_t)stream;
  AHL_DISPATCH_DTYPE(dtype, {
    hipLaunchKernelGGL((k_col_partial<D>), dim3((unsigned)cdiv(cols, 256), kColSplits), dim3(256), 0, s, x, rows, cols, ld, (float*)ws);
    hipLaunchKernelGGL((k_col_final<D>), dim3((unsigned)cdiv(cols, 256)), dim3(256), 0, s, (const float*)ws, cols, out);
  });
  return check_launch("ahl_col_sum");
}

}  // extern "C"
