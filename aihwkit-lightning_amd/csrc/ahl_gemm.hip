// The analog matrix product on CDNA4 MFMA: forward with fused DAC prologue and per-K-tile
// noise/ADC/clamp epilogue, input gradient with fused input-range gradient, weight gradient.
//
// All three products are "row x row" contractions C[i, j] = sum_k A[i, k] * B[j, k] with both
// operands contiguous along k, staged global -> registers -> LDS in 128-byte-wide row chunks
// and consumed by v_mfma_f32_32x32x16_bf16 (bf16) or v_mfma_f32_32x32x2_f32 (fp32).
//
// Block: 256 threads = 4 waves in a 2x2 grid; block tile 128 x 128; wave tile 64 x 64 =
// 2 x 2 MFMA blocks of 32 x 32 (16 fp32 accumulators per lane per block).
//
// LDS layout: one chunk = 128 rows x 128 data bytes, row stride 144 bytes; with this stride
// the 16 lanes that the LDS services together for a 16-byte read hit 16 distinct 4-bank groups.
//
// MFMA operand convention: lane l supplies, for row/column (l % 32), the 16 bytes at byte
// offset 32 * s + 16 * (l / 32) of the chunk row (s = k-step). A and B use the same rule, so
// the contraction pairs identical k positions whatever the hardware's internal k order is.
// MFMA 32x32 result convention: register v of lane l holds
//   C[8 * (v / 4) + 4 * (l / 32) + (v % 4)][l % 32].
#include "ahl_host.h"
#include <math.h>
#include <mutex>

namespace ahl {

static constexpr int kBM = 128;
static constexpr int kBN = 128;
static constexpr int kRowBytes = 128;
static constexpr int kLdsStride = 144;
static constexpr int kChunkLds = 128 * kLdsStride;  // bytes per operand chunk in LDS

template <class D>
struct ChunkK {  // elements along k per chunk
  static constexpr int value = kRowBytes / (int)sizeof(typename D::elem);
};

// ---- MFMA wrappers ---------------------------------------------------------------------------
template <class D>
struct Mma;
template <>
struct Mma<BF16> {
  static AHL_DEV void run(const u32x4& a, const u32x4& b, f32x16& c) {
    c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
};
template <>
struct Mma<F16> {
  static AHL_DEV void run(const u32x4& a, const u32x4& b, f32x16& c) {
    c = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                               __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
};
template <>
struct Mma<F32> {
  static AHL_DEV void run(const u32x4& a, const u32x4& b, f32x16& c) {
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.x), __uint_as_float(b.x), c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.y), __uint_as_float(b.y), c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.z), __uint_as_float(b.z), c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.w), __uint_as_float(b.w), c, 0, 0, 0);
  }
};

// One chunk of MFMAs for a wave: acc[bi][bj] += A(rows wm*64+bi*32..) x B(rows wn*64+bj*32..)
template <class D>
AHL_DEV void mfma_chunk(const char* ldsA, const char* ldsB, int wm, int wn, int lane,
                        f32x16 (&acc)[2][2]) {
  const int r = lane & 31, h = lane >> 5;
  const char* pa = ldsA + (wm * 64 + r) * kLdsStride + h * 16;
  const char* pb = ldsB + (wn * 64 + r) * kLdsStride + h * 16;
#pragma unroll
  for (int s = 0; s < 4; ++s) {
    u32x4 a0 = *(const u32x4*)(pa + s * 32);
    u32x4 a1 = *(const u32x4*)(pa + 32 * kLdsStride + s * 32);
    u32x4 b0 = *(const u32x4*)(pb + s * 32);
    u32x4 b1 = *(const u32x4*)(pb + 32 * kLdsStride + s * 32);
    Mma<D>::run(a0, b0, acc[0][0]);
    Mma<D>::run(a0, b1, acc[0][1]);
    Mma<D>::run(a1, b0, acc[1][0]);
    Mma<D>::run(a1, b1, acc[1][1]);
  }
}

// ---- chunk staging ---------------------------------------------------------------------------
// A thread owns 4 of the 1024 16-byte vectors of a 128 x 128-byte chunk: vector j lives in
// chunk row (tid / 8 + 32 * j), byte column 16 * (tid % 8).
struct VecPos {
  int row0;  // tid / 8
  int cv;    // tid % 8
};
AHL_DEV VecPos vec_pos(int tid) { return VecPos{tid >> 3, tid & 7}; }

// Loads the raw vectors of one chunk: rows [row_base, row_base+128) of `p` (ld elements),
// columns [kc, kc + chunkK) clipped to k_end; rows >= n_rows and columns >= k_end read as 0.
template <class D, bool VEC>
AHL_DEV void load_chunk(const void* p, int64_t ld, int64_t row_base, int64_t n_rows, int32_t kc,
                        int32_t k_end, const VecPos& vp, u32x4 (&raw)[4]) {
  constexpr int E = D::EPV;
  const typename D::elem* base = (const typename D::elem*)p;
  const int32_t k = kc + vp.cv * E;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int64_t row = row_base + vp.row0 + 32 * j;
    u32x4 v = {0u, 0u, 0u, 0u};
    if (row < n_rows) {
      const typename D::elem* q = base + row * ld + k;
      if (VEC) {
        if (k < k_end) v = ld16(q);
      } else {
        float e[E];
#pragma unroll
        for (int i = 0; i < E; ++i) e[i] = (k + i < k_end) ? D::load(q, i) : 0.0f;
        v = D::pack(e);
      }
    }
    raw[j] = v;
  }
}

AHL_DEV void store_chunk(char* lds, const VecPos& vp, const u32x4 (&v)[4]) {
#pragma unroll
  for (int j = 0; j < 4; ++j)
    *(u32x4*)(lds + (vp.row0 + 32 * j) * kLdsStride + vp.cv * 16) = v[j];
}

// XCD-aware block order: the hardware deals consecutive workgroup ids round-robin to the 8
// XCDs; this maps them back so that each XCD (own L2) works on a contiguous range of tiles.
AHL_DEV int64_t xcd_remap(int64_t bid, int64_t nb) {
  if ((nb & 7) != 0) return bid;
  return (bid & 7) * (nb >> 3) + (bid >> 3);
}

// =============================================================================================
// Forward
// =============================================================================================
struct FwdArgs {
  const void* x; int64_t ldx;
  const void* w; int64_t ldw;
  const void* bias;
  void* y; int64_t ldy;
  uint32_t* keep;
  const void* ir;
  const void* wmax;
  const float* tile_max;
  int64_t M, N;
  Tiling tl;
  float inp_res, out_res, out_bound;
  float noise_scale;  // out_noise / sqrt(n_tiles) as float, 0 when the noise is off
  int32_t noise_per_channel, bound_per_channel, skip_rounding;
  int32_t dac_on, adc_on, bound_on, clamp_on, noise_on;
  uint64_t seed, offset;
  const uint64_t* seed_state;  // null, or device {key, call counter} that replaces seed / offset
};

template <class D, bool VEC, int IRMODE>
__global__ __launch_bounds__(256) void k_linear_fwd(FwdArgs a) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  char* ldsA = lds;
  char* ldsB = lds + kChunkLds;
  float* rowir = (float*)(lds + 2 * kChunkLds);  // [2][128] per-row input range (dynamic mode)

  constexpr int CK = ChunkK<D>::value;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const VecPos vp = vec_pos(tid);

  const int64_t nbn = cdiv_dev(a.N, kBN);
  const int64_t logical = xcd_remap(blockIdx.x, gridDim.x);
  const int64_t m0 = (logical / nbn) * kBM, n0 = (logical % nbn) * kBN;
  const int T = a.tl.n_tiles;

  f32x16 total[2][2], acc[2][2];
  uint32_t cwords[2] = {0u, 0u};  // lane L: clamp-mask word of row wm * 64 + L, per column block
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
#pragma unroll
      for (int v = 0; v < 16; ++v) { total[i][j][v] = 0.0f; acc[i][j][v] = 0.0f; }
    }

  // --- state of the chunk being loaded ---
  int ld_t = 0;
  int32_t ld_kc = a.tl.start(0), ld_kend = a.tl.start(1);
  u32x4 rawA[4], rawB[4];
  load_chunk<D, VEC>(a.x, a.ldx, m0, a.M, ld_kc, ld_kend, vp, rawA);
  load_chunk<D, VEC>(a.w, a.ldw, n0, a.N, ld_kc, ld_kend, vp, rawB);
  bool have = true;

  while (have) {
    const int cur_t = ld_t;
    const bool cur_last = (ld_kc + CK >= ld_kend);  // last chunk of its K-tile
    const bool cur_first = (ld_kc == a.tl.start(cur_t));

    // ---- A prologue: clamp + DAC in registers, then stage to LDS ----
    u32x4 qa[4];
    if (IRMODE == AHL_IR_NONE) {
#pragma unroll
      for (int j = 0; j < 4; ++j) qa[j] = rawA[j];
    } else {
      Dac dac;
      if (IRMODE == AHL_IR_STATIC) dac = make_dac<D>(D::load(a.ir, cur_t), a.inp_res);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (IRMODE == AHL_IR_DYNAMIC) {
          const int64_t m = m0 + vp.row0 + 32 * j;
          const float irm = m < a.M ? D::load(a.ir, (int64_t)cur_t * a.M + m) : 0.0f;
          dac = make_dac<D>(irm, a.inp_res);
        }
        float e[D::EPV];
        D::unpack(rawA[j], e);
        if (a.dac_on) {
#pragma unroll
          for (int i = 0; i < D::EPV; ++i)
            e[i] = dac_apply<D, IRMODE == AHL_IR_STATIC, true>(e[i], dac, a.skip_rounding != 0);
        } else if (IRMODE == AHL_IR_STATIC) {
#pragma unroll
          for (int i = 0; i < D::EPV; ++i)
            e[i] = dac_apply<D, true, false>(e[i], dac, false);
        }
        qa[j] = D::pack(e);
      }
    }
    __syncthreads();
    store_chunk(ldsA, vp, qa);
    store_chunk(ldsB, vp, rawB);
    if (IRMODE == AHL_IR_DYNAMIC && cur_first && tid < 128) {
      const int64_t m = m0 + tid;
      rowir[(cur_t & 1) * 128 + tid] = m < a.M ? D::load(a.ir, (int64_t)cur_t * a.M + m) : 0.0f;
    }
    __syncthreads();

    // ---- issue the next chunk's global loads ----
    ld_kc += CK;
    if (ld_kc >= ld_kend) {
      ld_t += 1;
      if (ld_t < T) { ld_kc = a.tl.start(ld_t); ld_kend = a.tl.start(ld_t + 1); }
    }
    have = ld_t < T;
    if (have) {
      load_chunk<D, VEC>(a.x, a.ldx, m0, a.M, ld_kc, ld_kend, vp, rawA);
      load_chunk<D, VEC>(a.w, a.ldw, n0, a.N, ld_kc, ld_kend, vp, rawB);
    }

    mfma_chunk<D>(ldsA, ldsB, wm, wn, lane, acc);

    // ---- per-K-tile epilogue: noise, ADC, clamp, accumulate in dtype ----
    if (cur_last) {
      const int t = cur_t;
      const float ir_t = IRMODE == AHL_IR_STATIC ? D::load(a.ir, t) : 0.0f;
      const float tmax = (a.noise_on || a.bound_on) ? a.tile_max[t] : 0.0f;
      const int h = lane >> 5;
#pragma unroll
      for (int bj = 0; bj < 2; ++bj) {
        const int64_t n = n0 + wn * 64 + bj * 32 + (lane & 31);
        const bool nvalid = n < a.N;
        float wch = 0.0f;
        if ((a.noise_on || a.bound_on) && nvalid) wch = D::load(a.wmax, (int64_t)t * a.N + n);
        const float wr = a.noise_per_channel ? wch : tmax;
        const float wb = a.bound_per_channel ? wch : tmax;
        // per-column constants of the static mode
        float nscale = 0.0f, B = 0.0f, r = 1.0f, rc = 1.0f, rcp = 1.0f;
        if (IRMODE == AHL_IR_STATIC) {
          if (a.noise_on) nscale = D::rd(wr * D::rd(a.noise_scale * ir_t));
          if (a.bound_on) {
            B = D::rd(D::rd(ir_t * a.out_bound) * wb);
            if (a.adc_on) {
              r = quant_step<D>(B, a.out_res);
              rc = fmaxf(r, D::tiny());
              rcp = __fdiv_rn(1.0f, rc);
            }
          }
        }
#pragma unroll
        for (int bi = 0; bi < 2; ++bi) {
          const int rbase = wm * 64 + bi * 32 + 4 * h;  // block-local row of v = 0
#pragma unroll
          for (int gp = 0; gp < 2; ++gp) {
            float xi[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            if (a.noise_on) {
              // rows m0 + rbase + 16 * gp + {0..3, 8..11}: one Philox call per lane and pair of groups
              const uint32_t mrow = (uint32_t)(m0 + rbase + 16 * gp);
              const NoiseKey nk = noise_key(a.seed, a.offset, a.seed_state);
              normal8(nk.seed, nk.offset, (uint32_t)t, (uint32_t)n, (mrow >> 4) * 2 + ((mrow >> 2) & 1), xi);
            }
#pragma unroll
            for (int gg = 0; gg < 2; ++gg) {
              const int g = 2 * gp + gg;
#pragma unroll
              for (int c = 0; c < 4; ++c) {
                const int v = 4 * g + c;
                const int rl = rbase + 8 * g + c;
                float y = D::rd(acc[bi][bj][v]);
                acc[bi][bj][v] = 0.0f;
                if (IRMODE == AHL_IR_DYNAMIC && (a.noise_on || a.bound_on)) {
                  const float irm = rowir[(t & 1) * 128 + rl];
                  if (a.noise_on) nscale = D::rd(wr * D::rd(a.noise_scale * irm));
                  if (a.bound_on) {
                    B = D::rd(D::rd(irm * a.out_bound) * wb);
                    if (a.adc_on) {
                      r = quant_step<D>(B, a.out_res);
                      rc = fmaxf(r, D::tiny());
                      rcp = __fdiv_rn(1.0f, rc);
                    }
                  }
                }
                if (a.noise_on) y = D::rd(__builtin_fmaf(nscale, xi[4 * gg + c], y));
                if (a.bound_on) {
                  if (a.adc_on) {
                    float q = D::rd(D::div_exact_rcp(y, rc, rcp));
                    if (!a.skip_rounding) q = rintf(q);
                    y = D::rd(q * r);
                  }
                  if (a.clamp_on) {
                    const bool kp = (y >= -B) && (y <= B);
                    if (a.keep != nullptr) clamp_record(!kp && nvalid, 32 * bi + 8 * g + c, cwords[bj]);
                    y = fminf(fmaxf(y, -B), B);
                  }
                }
                total[bi][bj][v] = D::rd(total[bi][bj][v] + y);
              }
            }
          }
        }
        // the clamp-mask words of this tile: 64 consecutive rows of one 32-column block
        if (a.keep != nullptr && a.clamp_on) {
          const int64_t m = m0 + wm * 64 + lane;
          const int64_t nb0 = n0 + wn * 64 + bj * 32;
          if (m < a.M && nb0 < a.N)
            a.keep[(int64_t)t * clamp_plane_words(a.M, a.N) + clamp_word(m, nb0, a.M)] = cwords[bj];
          cwords[bj] = 0u;
        }
      }
    }
  }

  // ---- store: y = total (+ bias) ----
  {
    const int h = lane >> 5;
#pragma unroll
    for (int bj = 0; bj < 2; ++bj) {
      const int64_t n = n0 + wn * 64 + bj * 32 + (lane & 31);
      if (n >= a.N) continue;
      const float b = a.bias ? D::load(a.bias, n) : 0.0f;
#pragma unroll
      for (int bi = 0; bi < 2; ++bi)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int64_t m = m0 + wm * 64 + bi * 32 + 8 * (v >> 2) + 4 * h + (v & 3);
          if (m < a.M) {
            float o = total[bi][bj][v];
            if (a.bias) o = D::rd(o + b);
            D::store(a.y, m * a.ldy + n, o);
          }
        }
    }
  }
}

// =============================================================================================
// Input gradient (+ input-range gradient partials)
// =============================================================================================
struct DxArgs {
  const void* g; int64_t ldg;
  const uint32_t* keep;
  const uint32_t* clamp_flag;
  uint32_t flag_token;
  const void* wt;  // w_eff_t [K, N]
  const void* x; int64_t ldx;
  const void* ir;
  void* dx; int64_t lddx;
  float* partial;  // [m_blocks * k_blocks][4]
  int64_t M, N, K;
  Tiling tl;
  int32_t kb_big, kb_small;  // 128-wide column blocks per tile of size base+1 / base
  int32_t ir_rule;           // AHL_IR_GRAD_*
};

// Decodes a column-block index into (tile, first column, end column).
AHL_DEV void decode_kblock(const Tiling& tl, int32_t kb_big, int32_t kb_small, int32_t idx, int& t,
                           int32_t& c0, int32_t& c1) {
  const int32_t big_total = tl.extra * kb_big;
  int32_t within;
  if (idx < big_total) { t = idx / kb_big; within = idx % kb_big; }
  else { t = tl.extra + (idx - big_total) / kb_small; within = (idx - big_total) % kb_small; }
  c0 = tl.start(t) + within * kBN;
  c1 = tl.start(t + 1);
}

// Applies the clamp mask of tile t to a vector of gradient values g[m, n .. n+E) (ALONG_N) or
// g[m .. m+E, n) (!ALONG_N, the transposed operand of the weight gradient).
template <class D, bool ALONG_N>
AHL_DEV u32x4 mask_vec(const u32x4& raw, const uint32_t* plane, int64_t M, int64_t m, int64_t n,
                       int64_t lim) {
  constexpr int E = D::EPV;
  float e[E];
  D::unpack(raw, e);
#pragma unroll
  for (int i = 0; i < E; ++i) {
    const int64_t mi = ALONG_N ? m : m + i, ni = ALONG_N ? n + i : n;
    if ((ALONG_N ? ni : mi) < lim) {
      const uint32_t w = plane[clamp_word(mi, ni, M)];
      if ((w >> (int)(ni & 31)) & 1u) e[i] = 0.0f;
    }
  }
  return D::pack(e);
}

template <class D, bool VEC, int IRMODE>
__global__ __launch_bounds__(256) void k_linear_bwd_dx(DxArgs a) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  char* ldsA = lds;
  char* ldsB = lds + kChunkLds;
  __shared__ float red[4][3];

  constexpr int CK = ChunkK<D>::value;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const VecPos vp = vec_pos(tid);

  const int32_t nkb = a.tl.extra * a.kb_big + (a.tl.n_tiles - a.tl.extra) * a.kb_small;
  const int64_t logical = xcd_remap(blockIdx.x, gridDim.x);
  const int64_t m0 = (logical / nkb) * kBM;
  int t; int32_t c0, c1;
  decode_kblock(a.tl, a.kb_big, a.kb_small, (int32_t)(logical % nkb), t, c0, c1);
  const bool use_keep = a.keep != nullptr && clamp_flag_says_clamped(a.clamp_flag, a.flag_token);
  const uint32_t* plane =
      use_keep ? a.keep + (int64_t)t * clamp_plane_words(a.M, a.N) : nullptr;

  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  u32x4 rawA[4], rawB[4];
  int32_t kc = 0;
  const int32_t kend = (int32_t)a.N;
  load_chunk<D, VEC>(a.g, a.ldg, m0, a.M, kc, kend, vp, rawA);
  load_chunk<D, VEC>(a.wt, a.N, c0, c1, kc, kend, vp, rawB);
  while (true) {
    u32x4 qa[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
      qa[j] = (plane && m0 + vp.row0 + 32 * j < a.M)
                  ? mask_vec<D, true>(rawA[j], plane, a.M, m0 + vp.row0 + 32 * j,
                                      kc + vp.cv * D::EPV, kend)
                  : rawA[j];
    __syncthreads();
    store_chunk(ldsA, vp, qa);
    store_chunk(ldsB, vp, rawB);
    __syncthreads();
    kc += CK;
    const bool more = kc < kend;
    if (more) {
      load_chunk<D, VEC>(a.g, a.ldg, m0, a.M, kc, kend, vp, rawA);
      load_chunk<D, VEC>(a.wt, a.N, c0, c1, kc, kend, vp, rawB);
    }
    mfma_chunk<D>(ldsA, ldsB, wm, wn, lane, acc);
    if (!more) break;
  }

  // ---- epilogue: round, input-range gradient partial sums, straight-through clamp mask ----
  const float ir_t = IRMODE == AHL_IR_STATIC ? D::load(a.ir, t) : 0.0f;
  float s_up = 0.0f, s_lo = 0.0f, cnt = 0.0f;
  const int h = lane >> 5;
#pragma unroll
  for (int bj = 0; bj < 2; ++bj) {
    const int64_t k = (int64_t)c0 + wn * 64 + bj * 32 + (lane & 31);
    if (k >= c1) continue;
#pragma unroll
    for (int bi = 0; bi < 2; ++bi)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int64_t m = m0 + wm * 64 + bi * 32 + 8 * (v >> 2) + 4 * h + (v & 3);
        if (m >= a.M) continue;
        float d = D::rd(acc[bi][bj][v]);
        if (IRMODE == AHL_IR_STATIC) {
          const float xv = D::load(a.x, m * a.ldx + k);
          if (a.ir_rule == AHL_IR_GRAD_LEARNED) {
            const bool up = xv >= ir_t, lo = xv <= -ir_t;
            if (up) s_up += fminf(d, 0.0f);
            if (lo) s_lo += fmaxf(d, 0.0f);
            if (up || lo) cnt += 1.0f;
          } else {
            if (xv > ir_t) s_up += d;
            if (xv < -ir_t) s_lo += d;
          }
          if (fabsf(xv) > ir_t) d = 0.0f;
        }
        D::store(a.dx, m * a.lddx + k, d);
      }
  }
  if (IRMODE == AHL_IR_STATIC) {
    s_up = wave_sum(s_up); s_lo = wave_sum(s_lo); cnt = wave_sum(cnt);
    if (lane == 0) { red[wave][0] = s_up; red[wave][1] = s_lo; red[wave][2] = cnt; }
    __syncthreads();
    if (tid == 0) {
      float* p = a.partial + logical * 4;
      p[0] = (red[0][0] + red[1][0]) + (red[2][0] + red[3][0]);
      p[1] = (red[0][1] + red[1][1]) + (red[2][1] + red[3][1]);
      p[2] = (red[0][2] + red[1][2]) + (red[2][2] + red[3][2]);
      p[3] = 0.0f;
    }
  }
}

// ir_grad[t] from the per-block partials (reference torch_utils/torch_linear.py:92-106).
template <class D>
__global__ __launch_bounds__(64) void k_ir_grad_finalize(const float* __restrict__ partial,
                                                         int64_t m_blocks, int32_t nkb,
                                                         int32_t kb_big, int32_t kb_small,
                                                         Tiling tl, int64_t M, const void* ir,
                                                         void* ir_grad, float decay, float min_pct,
                                                         int32_t rule) {
  const int t = blockIdx.x, lane = threadIdx.x;
  const int32_t first = t < tl.extra ? t * kb_big : tl.extra * kb_big + (t - tl.extra) * kb_small;
  const int32_t count = t < tl.extra ? kb_big : kb_small;
  double s_up = 0.0, s_lo = 0.0, cnt = 0.0;
  const int64_t total = m_blocks * count;
  for (int64_t i = lane; i < total; i += 64) {
    const int64_t mb = i / count, kb = first + i % count;
    const float* p = partial + (mb * nkb + kb) * 4;
    s_up += (double)p[0]; s_lo += (double)p[1]; cnt += (double)p[2];
  }
  s_up = wave_sum(s_up); s_lo = wave_sum(s_lo); cnt = wave_sum(cnt);
  if (lane == 0) {
    const float irv = D::load(ir, t);
    float gr = D::rd(0.0f + D::rd((float)s_up));
    gr = D::rd(gr - D::rd((float)s_lo));
    if (rule == AHL_IR_GRAD_CLAMP) {  // the two bound gradients, each reduced in dtype, then added
      D::store(ir_grad, t, gr);
      return;
    }
    gr = D::rd(gr * irv);
    if (decay > 0.0f) {
      const float numel = (float)((double)M * (double)tl.size(t));
      const float pct = 1.0f - __fdiv_rn((float)cnt, numel);
      const float add = pct > min_pct ? D::rd(decay * irv) : 0.0f;
      gr = D::rd(gr + add);
    }
    D::store(ir_grad, t, gr);
  }
}

// =============================================================================================
// Weight gradient: dw[n, k] = sum_m gT[n, m] * xqT[k, m], gT zeroed where tile t was clamped
// =============================================================================================
struct DwArgs {
  const void* gt;       // [N, M]
  const uint32_t* keept; // the clamp mask in its native layout, or null
  const uint32_t* clamp_flag;
  uint32_t flag_token;
  const void* xqt;      // [K, M]
  void* dw; int64_t lddw;
  int64_t M, N, K;
  Tiling tl;
  int32_t kb_big, kb_small;
};

template <class D, bool VEC>
__global__ __launch_bounds__(256) void k_linear_bwd_dw(DwArgs a) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  char* ldsA = lds;
  char* ldsB = lds + kChunkLds;
  constexpr int CK = ChunkK<D>::value;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const VecPos vp = vec_pos(tid);

  const int32_t nkb = a.tl.extra * a.kb_big + (a.tl.n_tiles - a.tl.extra) * a.kb_small;
  const int64_t logical = xcd_remap(blockIdx.x, gridDim.x);
  const int64_t n0 = (logical / nkb) * kBM;
  int t; int32_t c0, c1;
  decode_kblock(a.tl, a.kb_big, a.kb_small, (int32_t)(logical % nkb), t, c0, c1);
  const bool use_keep = a.keept != nullptr && clamp_flag_says_clamped(a.clamp_flag, a.flag_token);
  const uint32_t* plane =
      use_keep ? a.keept + (int64_t)t * clamp_plane_words(a.M, a.N) : nullptr;

  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  u32x4 rawA[4], rawB[4];
  int32_t kc = 0;
  const int32_t kend = (int32_t)a.M;
  load_chunk<D, VEC>(a.gt, a.M, n0, a.N, kc, kend, vp, rawA);
  load_chunk<D, VEC>(a.xqt, a.M, c0, c1, kc, kend, vp, rawB);
  while (true) {
    u32x4 qa[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
      qa[j] = (plane && n0 + vp.row0 + 32 * j < a.N)
                  ? mask_vec<D, false>(rawA[j], plane, a.M, kc + vp.cv * D::EPV,
                                       n0 + vp.row0 + 32 * j, kend)
                  : rawA[j];
    __syncthreads();
    store_chunk(ldsA, vp, qa);
    store_chunk(ldsB, vp, rawB);
    __syncthreads();
    kc += CK;
    const bool more = kc < kend;
    if (more) {
      load_chunk<D, VEC>(a.gt, a.M, n0, a.N, kc, kend, vp, rawA);
      load_chunk<D, VEC>(a.xqt, a.M, c0, c1, kc, kend, vp, rawB);
    }
    mfma_chunk<D>(ldsA, ldsB, wm, wn, lane, acc);
    if (!more) break;
  }
  const int h = lane >> 5;
#pragma unroll
  for (int bj = 0; bj < 2; ++bj) {
    const int64_t k = (int64_t)c0 + wn * 64 + bj * 32 + (lane & 31);
    if (k >= c1) continue;
#pragma unroll
    for (int bi = 0; bi < 2; ++bi)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int64_t n = n0 + wm * 64 + bi * 32 + 8 * (v >> 2) + 4 * h + (v & 3);
        if (n < a.N) D::store(a.dw, n * a.lddw + k, D::rd(acc[bi][bj][v]));
      }
  }
}

// =============================================================================================
// Transposes feeding the weight gradient
// =============================================================================================
// out[c, r] = f(in[r, c]); 64 x 64 tiles through LDS; E = element type.
template <class E>
__global__ __launch_bounds__(256) void k_transpose(const E* __restrict__ in, int64_t R, int64_t C,
                                                   int64_t ld_in, E* __restrict__ out,
                                                   int64_t ld_out) {
  __shared__ E tile[64][64 + 4 / sizeof(E) + 1];
  const int64_t r0 = (int64_t)blockIdx.y * 64, c0 = (int64_t)blockIdx.x * 64;
  const E* inp = in + (int64_t)blockIdx.z * R * ld_in;
  E* outp = out + (int64_t)blockIdx.z * C * ld_out;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int i = ty; i < 64; i += 4) {
    const int64_t r = r0 + i, c = c0 + tx;
    if (r < R && c < C) tile[i][tx] = inp[r * ld_in + c];
  }
  __syncthreads();
  for (int i = ty; i < 64; i += 4) {
    const int64_t c = c0 + i, r = r0 + tx;
    if (r < R && c < C) outp[c * ld_out + r] = tile[tx][i];
  }
}

// xqt[k, m] = DAC(clamp(x[m, k])) with the input range of k's tile.
template <class D, int IRMODE>
__global__ __launch_bounds__(256) void k_dac_transpose(const void* __restrict__ x, int64_t M,
                                                       int64_t K, int64_t ldx, const void* ir,
                                                       Tiling tl, float inp_res, int32_t dac_on,
                                                       int32_t skip_rounding,
                                                       void* __restrict__ out) {
  __shared__ typename D::elem tile[64][64 + 4];
  const int64_t r0 = (int64_t)blockIdx.y * 64, c0 = (int64_t)blockIdx.x * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  const int64_t k = c0 + tx;
  const int t = k < K ? tl.tile_of((int32_t)k) : 0;
  Dac dac;
  if (IRMODE == AHL_IR_STATIC) dac = make_dac<D>(D::load(ir, t), inp_res);
  for (int i = ty; i < 64; i += 4) {
    const int64_t m = r0 + i;
    if (m < M && k < K) {
      float v = D::load(x, m * ldx + k);
      if (IRMODE == AHL_IR_DYNAMIC) dac = make_dac<D>(D::load(ir, (int64_t)t * M + m), inp_res);
      if (IRMODE != AHL_IR_NONE) {
        if (dac_on) v = dac_apply<D, IRMODE == AHL_IR_STATIC, true>(v, dac, skip_rounding != 0);
        else if (IRMODE == AHL_IR_STATIC) v = dac_apply<D, true, false>(v, dac, false);
      }
      tile[i][tx] = D::to_elem(v);
    }
  }
  __syncthreads();
  for (int i = ty; i < 64; i += 4) {
    const int64_t kk = c0 + i, m = r0 + tx;
    if (m < M && kk < K) ((typename D::elem*)out)[kk * M + m] = tile[tx][i];
  }
}

}  // namespace ahl

using namespace ahl;

static constexpr int kGemmLds = 2 * kChunkLds + 2 * 128 * (int)sizeof(float);

static bool cfg_ok(const AhlLinearCfg* c) {
  if (!c) return false;
  if (!dtype_known(c->dtype)) return false;
  if (c->ir_mode < 0 || c->ir_mode > 2) return false;
  if (c->ir_grad_rule != AHL_IR_GRAD_LEARNED && c->ir_grad_rule != AHL_IR_GRAD_CLAMP) return false;
  if (c->tile_stride < 0 || c->tile_stride % 256 != 0) return false;
  return true;
}

namespace ahl {
bool fast_fwd_eligible(const AhlLinearCfg* cfg, const void* xq, int64_t ldxq, const void* w,
                       int64_t ldw, int64_t K, const Tiling& tl);
int launch_fast_fwd(const void* xq, int64_t ldxq, const void* w_eff, int64_t ldw, const void* bias,
                    void* y, int64_t ldy, uint32_t* keep, uint32_t* clamp_flag, const void* ir,
                    const void* wmax, const float* tile_max, int64_t M, int64_t K, int64_t N,
                    const Tiling& tl, const AhlLinearCfg* cfg, void* ws, hipStream_t s,
                    const ConvMap* conv = nullptr);
int64_t fast_fwd_ws_bytes(int64_t M, int64_t N, int32_t n_tiles);
__global__ void k_set_u32(uint32_t* p, uint32_t v) { *p = v; }
bool fast_bwd_eligible(int32_t dtype, const Tiling& tl, int64_t M, int64_t K, int64_t N);
int launch_fast_dx(int32_t dtype, const void* g, int64_t ldg, const uint32_t* keep, const uint32_t* clamp_flag,
                   uint32_t flag_token, const void* w_eff, int64_t ldw, const void* x, int64_t ldx, const void* ir,
                   void* dx, int64_t lddx, void* ws, int64_t M, int64_t K, int64_t N,
                   const Tiling& tl, int ir_static, int32_t dense_tile, const Tiling* dense,
                   hipStream_t s);
int64_t fast_dx_ws_bytes(int64_t M, int64_t K, int64_t N);
int64_t fast_dx_row_blocks(int64_t M, int64_t K, int64_t N, bool element_mode);
int launch_fast_dw(int32_t dtype, const void* g, int64_t ldg, const uint32_t* keep, const uint32_t* clamp_flag,
                   uint32_t flag_token, const void* xq, int64_t ldxq, void* dw, int64_t lddw, void* dbias,
                   void* ws, int64_t M, int64_t K, int64_t N, const Tiling& tl,
                   hipStream_t s, const ConvMap* conv = nullptr, int32_t conv_cols = 0, int block_cols = 256);
int64_t fast_dw_ws_bytes(int64_t M, int64_t K, int64_t N, int block_cols = 256);
int launch_pad_tiles(const void* src, int64_t ld_src, int32_t dtype, int64_t rows, const Tiling& tl,
                     int64_t stride, void* dst, int64_t ld_dst, hipStream_t s);
int launch_unpad_tiles(const void* src, int64_t ld_src, int32_t dtype, int64_t rows, int64_t K,
                       const Tiling& tl, int64_t stride, void* dst, int64_t ld_dst, hipStream_t s);
}  // namespace ahl

template <class D>
static bool tiles_vec_ok(const Tiling& tl) {
  return tl.extra == 0 ? (tl.base % D::EPV == 0) : false;
}

template <class D>
static void launch_fwd(const FwdArgs& a, int ir_mode, dim3 grid, hipStream_t s) {
  const bool vec = aligned16(a.x) && aligned16(a.w) && a.ldx % D::EPV == 0 && a.ldw % D::EPV == 0 &&
                   tiles_vec_ok<D>(a.tl);
  const dim3 block(256);
  if (vec) {
    if (ir_mode == AHL_IR_NONE) hipLaunchKernelGGL((k_linear_fwd<D, true, 0>), grid, block, kGemmLds, s, a);
    else if (ir_mode == AHL_IR_STATIC) hipLaunchKernelGGL((k_linear_fwd<D, true, 1>), grid, block, kGemmLds, s, a);
    else hipLaunchKernelGGL((k_linear_fwd<D, true, 2>), grid, block, kGemmLds, s, a);
  } else {
    if (ir_mode == AHL_IR_NONE) hipLaunchKernelGGL((k_linear_fwd<D, false, 0>), grid, block, kGemmLds, s, a);
    else if (ir_mode == AHL_IR_STATIC) hipLaunchKernelGGL((k_linear_fwd<D, false, 1>), grid, block, kGemmLds, s, a);
    else hipLaunchKernelGGL((k_linear_fwd<D, false, 2>), grid, block, kGemmLds, s, a);
  }
}

template <class D>
static void launch_dx(const DxArgs& a, bool is_static, dim3 grid, hipStream_t s) {
  const bool vec = aligned16(a.g) && aligned16(a.wt) && a.ldg % D::EPV == 0 && a.N % D::EPV == 0 &&
                   (!a.keep || (((uintptr_t)a.keep) & 7u) == 0);
  const dim3 block(256);
  if (vec) {
    if (is_static) hipLaunchKernelGGL((k_linear_bwd_dx<D, true, 1>), grid, block, kGemmLds, s, a);
    else hipLaunchKernelGGL((k_linear_bwd_dx<D, true, 0>), grid, block, kGemmLds, s, a);
  } else {
    if (is_static) hipLaunchKernelGGL((k_linear_bwd_dx<D, false, 1>), grid, block, kGemmLds, s, a);
    else hipLaunchKernelGGL((k_linear_bwd_dx<D, false, 0>), grid, block, kGemmLds, s, a);
  }
}

extern "C" {

int64_t ahl_linear_fwd_ws_bytes(int64_t M, int64_t K, int64_t N, int32_t n_tiles, int32_t dtype) {
  (void)K;
  if ((dtype != AHL_BF16 && dtype != AHL_F16) || M <= 0 || N <= 0 || n_tiles <= 0) return 0;
  return fast_fwd_ws_bytes(M, N, n_tiles);
}

int ahl_linear_fwd(const void* x, int64_t ldx, const void* xq, int64_t ldxq, const void* w_eff,
                   int64_t ldw, const void* bias, void* y, int64_t ldy, uint32_t* keep,
                   uint32_t* clamp_flag, const void* ir, const void* wmax, const float* tile_max,
                   int64_t M, int64_t K, int64_t N, const int32_t* tile_ends_host, int32_t n_tiles,
                   const AhlLinearCfg* cfg, void* ws, void* stream) {
  if (!cfg_ok(cfg) || (!x && !xq) || !w_eff || !y || M <= 0 || K <= 0 || N <= 0) return AHL_ERR_ARG;
  if ((x && ldx < K) || (xq && ldxq < K) || ldw < K || ldy < N) return AHL_ERR_ARG;
  Tiling tl;
  if (!make_tiling(tile_ends_host, n_tiles, K, &tl)) return AHL_ERR_TILING;
  {
    const bool noise_on = cfg->training && cfg->out_noise > 0.0f;
    const bool bound_on = cfg->out_res > 0.0f || cfg->out_bound > 0.0f;
    if (cfg->ir_mode == AHL_IR_NONE && (cfg->inp_res > 0.0f || bound_on || noise_on)) return AHL_ERR_ARG;
    if (cfg->ir_mode != AHL_IR_NONE && !ir) return AHL_ERR_ARG;
    if ((noise_on || bound_on) && (!wmax || !tile_max)) return AHL_ERR_ARG;
  }
  if (fast_fwd_eligible(cfg, xq, ldxq, w_eff, ldw, K, tl) && N % 8 == 0 && ldy % 8 == 0 &&
      aligned16(y) && (!keep || (((uintptr_t)keep) & 3u) == 0))
    return launch_fast_fwd(xq, ldxq, w_eff, ldw, bias, y, ldy, keep, clamp_flag, ir, wmax, tile_max,
                           M, K, N, tl, cfg, ws, (hipStream_t)stream);
  // only the fast path can start from xq alone or read the padded tile layout
  if (!x || cfg->tile_stride > 0) return AHL_ERR_UNSUPPORTED;
  FwdArgs a;
  a.x = x; a.ldx = ldx; a.w = w_eff; a.ldw = ldw; a.bias = bias; a.y = y; a.ldy = ldy;
  a.keep = keep; a.ir = ir; a.wmax = wmax; a.tile_max = tile_max; a.M = M; a.N = N; a.tl = tl;
  a.inp_res = cfg->inp_res; a.out_res = cfg->out_res; a.out_bound = cfg->out_bound;
  a.noise_on = (cfg->training && cfg->out_noise > 0.0f) ? 1 : 0;
  a.noise_scale = a.noise_on ? (float)((double)cfg->out_noise / sqrt((double)n_tiles)) : 0.0f;
  a.noise_per_channel = cfg->out_noise_per_channel; a.bound_per_channel = cfg->bound_per_channel;
  a.skip_rounding = cfg->skip_rounding;
  a.dac_on = cfg->inp_res > 0.0f ? 1 : 0;
  a.adc_on = cfg->out_res > 0.0f ? 1 : 0;
  a.clamp_on = cfg->out_bound > 0.0f ? 1 : 0;
  a.bound_on = (a.adc_on || a.clamp_on) ? 1 : 0;
  a.seed = cfg->seed; a.offset = cfg->offset; a.seed_state = cfg->seed_state;
  if (cfg->ir_mode == AHL_IR_NONE && (a.dac_on || a.bound_on || a.noise_on)) return AHL_ERR_ARG;
  if (cfg->ir_mode != AHL_IR_NONE && !ir) return AHL_ERR_ARG;
  if ((a.noise_on || a.bound_on) && (!wmax || !tile_max)) return AHL_ERR_ARG;
  hipStream_t s = (hipStream_t)stream;
  const int64_t nb = cdiv(M, kBM) * cdiv(N, kBN);
  if (nb > 0x7fffffff) return AHL_ERR_ARG;
  const dim3 grid((unsigned)nb);
  // this kernel does not track clamping: tell the backward to honour the mask
  if (clamp_flag)
    hipLaunchKernelGGL(k_set_u32, dim3(1), dim3(1), 0, s, clamp_flag, cfg->flag_token ? cfg->flag_token : 1u);
  if (cfg->dtype == AHL_F32) launch_fwd<F32>(a, cfg->ir_mode, grid, s);
  else if (cfg->dtype == AHL_F16) launch_fwd<F16>(a, cfg->ir_mode, grid, s);
  else launch_fwd<BF16>(a, cfg->ir_mode, grid, s);
  return check_launch("ahl_linear_fwd");
}

static void kblocks(const Tiling& tl, int32_t* kb_big, int32_t* kb_small) {
  *kb_big = (int32_t)cdiv(tl.base + 1, kBN);
  *kb_small = (int32_t)cdiv(tl.base, kBN);
}

static int64_t align256(int64_t v) { return (v + 255) / 256 * 256; }

static int64_t dx_partial_bytes(int64_t M, int64_t K, int32_t n_tiles) {
  Tiling tl{n_tiles, (int32_t)(K / n_tiles), (int32_t)(K % n_tiles)};
  int32_t kb, ks;
  kblocks(tl, &kb, &ks);
  const int64_t nkb = (int64_t)tl.extra * kb + (int64_t)(n_tiles - tl.extra) * ks;
  return align256(cdiv(M, kBM) * nkb * 4 * (int64_t)sizeof(float));
}

// Workspace of the padded-layout backward: the input-range partial sums
static int64_t dx_padded_partial_bytes(int64_t M, int64_t padded) {
  return align256(cdiv(M, 256) * (padded / 256) * 4 * (int64_t)sizeof(float));
}

int64_t ahl_linear_bwd_dx_ws_bytes(int64_t M, int64_t K, int64_t N, int32_t n_tiles, int32_t dtype,
                                   int64_t tile_stride) {
  if (n_tiles <= 0 || K <= 0 || M <= 0 || N <= 0) return 0;
  const int64_t es = dtype_bytes(dtype);
  if (tile_stride > 0) {  // the MFMA kernel's workspace; x and dx are used in place
    const int64_t padded = (int64_t)n_tiles * tile_stride;
    const int64_t fast = align256(fast_dx_ws_bytes(M, padded, N));
    return fast > dx_padded_partial_bytes(M, padded) ? fast : dx_padded_partial_bytes(M, padded);
  }
  // general kernels: partials + transposed weights; MFMA kernel: its own layout in the same space
  const int64_t generic = dx_partial_bytes(M, K, n_tiles) + align256(K * N * es);
  const int64_t fast = K % 256 == 0 ? align256(fast_dx_ws_bytes(M, K, N)) : 0;
  return generic > fast ? generic : fast;
}

int ahl_linear_bwd_dx(const void* g, int64_t ldg, const uint32_t* keep, const uint32_t* clamp_flag,
                      const void* w_eff, int64_t ldw, const void* x, int64_t ldx, const void* ir,
                      void* dx, int64_t lddx, void* ir_grad, int64_t M, int64_t K, int64_t N,
                      const int32_t* tile_ends_host, int32_t n_tiles, const AhlLinearCfg* cfg,
                      void* ws, void* stream) {
  if (!cfg_ok(cfg) || !g || !w_eff || !dx || !ws || M <= 0 || K <= 0 || N <= 0) return AHL_ERR_ARG;
  if (ldg < N || lddx < K || ldw < K) return AHL_ERR_ARG;
  const bool is_static = cfg->ir_mode == AHL_IR_STATIC;
  if (is_static && (!x || !ir || !ir_grad || ldx < K)) return AHL_ERR_ARG;
  if (!aligned16(ws)) return AHL_ERR_WORKSPACE;
  Tiling tl;
  if (!make_tiling(tile_ends_host, n_tiles, K, &tl)) return AHL_ERR_TILING;
  hipStream_t s = (hipStream_t)stream;
  float* partial = (float*)ws;
  if (cfg->tile_stride > 0) {
    // w_eff is in the padded tile layout: the MFMA kernel runs on aligned tiles of `stride`
    // columns and maps its output columns back onto the dense x / dx in its epilogue
    const int64_t stride = cfg->tile_stride, padded = (int64_t)n_tiles * stride;
    if (stride < widest_tile(tl) || ldw < padded || padded > 0x3fffffff) return AHL_ERR_ARG;
    if ((cfg->dtype != AHL_BF16 && cfg->dtype != AHL_F16) || N % 8 != 0 || N < 8 || !aligned16(g) || !aligned16(w_eff) ||
        ldg % 8 != 0 || ldw % 8 != 0 || (keep && !aligned16(keep)))
      return AHL_ERR_UNSUPPORTED;
    const Tiling ptl{n_tiles, (int32_t)stride, 0};
    const int32_t per_tile = (int32_t)(stride / 256);
    // x and dx stay dense. Equal tiles of a multiple of 8 columns: the kernel's 16-byte vectors
    // of x and dx map one to one onto the dense matrices; any other split: its epilogue works
    // element by element (coalesced 2-byte accesses). No padded copies either way.
    const bool vectors = tl.extra == 0 && tl.base % 8 == 0 && lddx % 8 == 0 && aligned16(dx) &&
                         (!is_static || (ldx % 8 == 0 && aligned16(x)));
    // the element-wise epilogue addresses x and dx with one offset and aligns its vectors on dx
    if (!vectors && (!aligned16(dx) || (is_static && (!aligned16(x) || ldx != lddx))))
      return AHL_ERR_UNSUPPORTED;
    const int rc = launch_fast_dx(cfg->dtype, g, ldg, keep, clamp_flag, cfg->flag_token, w_eff, ldw, x, ldx, ir, dx, lddx, ws,
                                  M, padded, N, ptl, is_static ? 1 + cfg->ir_grad_rule : 0,
                                  vectors ? tl.base : 0, vectors ? nullptr : &tl, s);
    if (rc != AHL_OK) return rc;
    if (is_static) {
      AHL_DISPATCH_DTYPE(cfg->dtype, {
        hipLaunchKernelGGL((k_ir_grad_finalize<D>), dim3(n_tiles), dim3(64), 0, s,
                           (const float*)partial, fast_dx_row_blocks(M, padded, N, !vectors),
                           (int32_t)(padded / 256), per_tile,
                           per_tile, tl, M, ir, ir_grad, cfg->ir_decay, cfg->ir_input_min_percentage,
                           cfg->ir_grad_rule);
      });
    }
    return check_launch("ahl_linear_bwd_dx(fast, padded weights)");
  }
  void* wt = (char*)ws + dx_partial_bytes(M, K, n_tiles);
  const bool fast = fast_bwd_eligible(cfg->dtype, tl, M, K, N) && aligned16(g) && aligned16(w_eff) &&
                    ldg % 8 == 0 && ldw % 8 == 0 && lddx % 8 == 0 && aligned16(dx) &&
                    (!keep || aligned16(keep)) &&
                    (!is_static || (ldx % 8 == 0 && aligned16(x)));
  if (fast) {
    int rc = launch_fast_dx(cfg->dtype, g, ldg, keep, clamp_flag, cfg->flag_token, w_eff, ldw, x, ldx, ir, dx, lddx, ws, M, K,
                            N, tl, is_static ? 1 + cfg->ir_grad_rule : 0, 0, nullptr, s);
    if (rc != AHL_OK) return rc;
    if (is_static) {
      const int32_t per_tile = tl.base / 256;
      AHL_DISPATCH_DTYPE(cfg->dtype, {
        hipLaunchKernelGGL((k_ir_grad_finalize<D>), dim3(n_tiles), dim3(64), 0, s,
                           (const float*)partial, fast_dx_row_blocks(M, K, N, false),
                           (int32_t)(K / 256), per_tile, per_tile,
                           tl, M, ir, ir_grad, cfg->ir_decay, cfg->ir_input_min_percentage,
                           cfg->ir_grad_rule);
      });
    }
    return check_launch("ahl_linear_bwd_dx(fast)");
  }
  DxArgs a;
  a.g = g; a.ldg = ldg; a.keep = keep; a.clamp_flag = clamp_flag; a.flag_token = cfg->flag_token; a.wt = wt; a.x = x; a.ldx = ldx;
  a.ir = ir; a.dx = dx; a.lddx = lddx; a.partial = partial; a.M = M; a.N = N; a.K = K; a.tl = tl;
  a.ir_rule = cfg->ir_grad_rule;
  kblocks(tl, &a.kb_big, &a.kb_small);
  const int64_t nkb = (int64_t)tl.extra * a.kb_big + (int64_t)(n_tiles - tl.extra) * a.kb_small;
  const int64_t mb = cdiv(M, kBM);
  if (mb * nkb > 0x7fffffff) return AHL_ERR_ARG;
  const dim3 tgrid((unsigned)cdiv(K, 64), (unsigned)cdiv(N, 64), 1);
  if (cfg->dtype == AHL_F32)
    hipLaunchKernelGGL((k_transpose<float>), tgrid, dim3(256), 0, s, (const float*)w_eff, N, K, ldw, (float*)wt, N);
  else
    hipLaunchKernelGGL((k_transpose<uint16_t>), tgrid, dim3(256), 0, s, (const uint16_t*)w_eff, N, K, ldw, (uint16_t*)wt, N);
  const dim3 grid((unsigned)(mb * nkb));
  if (cfg->dtype == AHL_F32) launch_dx<F32>(a, is_static, grid, s);
  else if (cfg->dtype == AHL_F16) launch_dx<F16>(a, is_static, grid, s);
  else launch_dx<BF16>(a, is_static, grid, s);
  if (is_static) {
    AHL_DISPATCH_DTYPE(cfg->dtype, {
      hipLaunchKernelGGL((k_ir_grad_finalize<D>), dim3(n_tiles), dim3(64), 0, s, (const float*)partial, mb,
                         (int32_t)nkb, a.kb_big, a.kb_small, tl, M, ir, ir_grad, cfg->ir_decay,
                         cfg->ir_input_min_percentage, cfg->ir_grad_rule);
    });
  }
  return check_launch("ahl_linear_bwd_dx");
}


// ---- allocation-free variant of ahl_linear_bwd_dx -------------------------------------------
// The workspace of the input gradient (input-range partial sums, slice partial results, the
// transposed weights of the general kernels) lives in a file-scope device array instead of a
// caller buffer. Each GPU holds its own copy of the array at its own address; the address is
// looked up once per device and used for every launch (the array's name is only a host-side
// handle, never a device address).
static constexpr int64_t kStaticDxScratchBytes = AHL_STATIC_DX_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticDxScratchBytes];

static constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static void* g_scratch_ptr[kMaxDevices] = {nullptr};

// Device address of `scratch` on the current device (cached per device); null + recorded error
// if the lookup fails.
static void* static_scratch_ptr() {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) { record_hip_error(e, "ahl_linear_bwd_dx_static(hipGetDevice)"); return nullptr; }
  if (dev < 0 || dev >= kMaxDevices) {
    record_hip_error(hipErrorInvalidDevice, "ahl_linear_bwd_dx_static(device index)");
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || ptr == nullptr) {
      record_hip_error(e, "ahl_linear_bwd_dx_static(hipGetSymbolAddress)");
      return nullptr;
    }
    g_scratch_ptr[dev] = ptr;
  }
  return g_scratch_ptr[dev];
}

int ahl_linear_bwd_dx_static(const void* g, int64_t ldg, const uint32_t* keep,
                             const uint32_t* clamp_flag, const void* w_eff, int64_t ldw,
                             const void* x, int64_t ldx, const void* ir, void* dx, int64_t lddx,
                             void* ir_grad, int64_t M, int64_t K, int64_t N,
                             const int32_t* tile_ends_host, int32_t n_tiles,
                             const AhlLinearCfg* cfg, void* stream) {
  if (!cfg_ok(cfg) || M <= 0 || K <= 0 || N <= 0 || n_tiles <= 0) return AHL_ERR_ARG;
  const int64_t need = ahl_linear_bwd_dx_ws_bytes(M, K, N, n_tiles, cfg->dtype, cfg->tile_stride);
  // larger shapes are for ahl_linear_bwd_dx with a caller workspace
  if (need > kStaticDxScratchBytes) return AHL_ERR_WORKSPACE;
  void* ptr = static_scratch_ptr();
  if (ptr == nullptr) return AHL_ERR_LAUNCH;
  // every slot of the workspace is written by this call's kernels before it is read: nothing
  // has to start at zero, whatever the previous call left behind
  return ahl_linear_bwd_dx(g, ldg, keep, clamp_flag, w_eff, ldw, x, ldx, ir, dx, lddx, ir_grad, M,
                           K, N, tile_ends_host, n_tiles, cfg, ptr, stream);
}


int64_t ahl_linear_bwd_dw_ws_bytes(int64_t M, int64_t K, int64_t N, int32_t n_tiles, int32_t dtype,
                                   int32_t has_keep, int64_t tile_stride) {
  const int64_t es = dtype_bytes(dtype);
  (void)has_keep;
  if (tile_stride > 0) {  // [workspace of the MFMA kernel | dw in the padded tile layout]
    const int64_t padded = (int64_t)n_tiles * tile_stride;
    return align256(fast_dw_ws_bytes(M, padded, N)) + align256(N * padded * es);
  }
  const int64_t generic = align256(N * M * es) + align256(K * M * es) + align256(ahl_col_sum_ws_bytes(N));
  const int64_t fast = K % 256 == 0 ? align256(fast_dw_ws_bytes(M, K, N)) : 0;
  return generic > fast ? generic : fast;
}

int ahl_linear_bwd_dw(const void* g, int64_t ldg, const uint32_t* keep, const uint32_t* clamp_flag,
                      const void* x, int64_t ldx, const void* xq, int64_t ldxq, const void* ir,
                      void* dw, int64_t lddw, void* dbias, int64_t M, int64_t K, int64_t N,
                      const int32_t* tile_ends_host, int32_t n_tiles, const AhlLinearCfg* cfg,
                      void* ws, void* stream) {
  if (!cfg_ok(cfg) || !g || (!x && !xq) || !dw || !ws || M <= 0 || K <= 0 || N <= 0) return AHL_ERR_ARG;
  if (ldg < N || (x && ldx < K) || (xq && ldxq < K) || lddw < K) return AHL_ERR_ARG;
  if (!xq && cfg->ir_mode != AHL_IR_NONE && !ir) return AHL_ERR_ARG;
  if (!aligned16(ws)) return AHL_ERR_WORKSPACE;
  Tiling tl;
  if (!make_tiling(tile_ends_host, n_tiles, K, &tl)) return AHL_ERR_TILING;
  hipStream_t s = (hipStream_t)stream;
  if (cfg->tile_stride > 0) {
    // xq is in the padded tile layout: the MFMA kernel writes dw in the same layout into the
    // workspace, then the data columns are copied into the dense dw
    const int64_t stride = cfg->tile_stride, padded = (int64_t)n_tiles * stride;
    if (!xq || stride < widest_tile(tl) || ldxq < padded || padded > 0x3fffffff) return AHL_ERR_ARG;
    if ((cfg->dtype != AHL_BF16 && cfg->dtype != AHL_F16) || N % 8 != 0 || N < 8 || !aligned16(g) || !aligned16(xq) ||
        ldg % 8 != 0 || ldxq % 8 != 0 || (keep && !aligned16(keep)))
      return AHL_ERR_UNSUPPORTED;
    void* dwp = (char*)ws + align256(fast_dw_ws_bytes(M, padded, N));
    const Tiling ptl{n_tiles, (int32_t)stride, 0};
    const int rc = launch_fast_dw(cfg->dtype, g, ldg, keep, clamp_flag, cfg->flag_token, xq, ldxq, dwp, padded, dbias, ws, M,
                                  padded, N, ptl, s);
    if (rc != AHL_OK) return rc;
    return launch_unpad_tiles(dwp, padded, AHL_BF16, N, K, tl, stride, dw, lddw, s);
  }
  if (xq && fast_bwd_eligible(cfg->dtype, tl, M, K, N) && aligned16(g) && aligned16(xq) &&
      ldg % 8 == 0 && ldxq % 8 == 0 && lddw % 8 == 0 && aligned16(dw) && (!keep || aligned16(keep)))
    return launch_fast_dw(cfg->dtype, g, ldg, keep, clamp_flag, cfg->flag_token, xq, ldxq, dw, lddw, dbias, ws, M, K, N, tl, s);
  const int32_t dac_on = cfg->inp_res > 0.0f ? 1 : 0;
  DwArgs a;
  a.M = M; a.N = N; a.K = K; a.tl = tl; a.dw = dw; a.lddw = lddw;
  kblocks(tl, &a.kb_big, &a.kb_small);
  const int64_t nkb = (int64_t)tl.extra * a.kb_big + (int64_t)(n_tiles - tl.extra) * a.kb_small;
  const int64_t nbn = cdiv(N, kBM);
  if (nbn * nkb > 0x7fffffff) return AHL_ERR_ARG;
  const dim3 tgrid_g((unsigned)cdiv(N, 64), (unsigned)cdiv(M, 64), 1);
  const dim3 tgrid_x((unsigned)cdiv(K, 64), (unsigned)cdiv(M, 64), 1);
  AHL_DISPATCH_DTYPE(cfg->dtype, {
    typedef typename D::elem E;
    char* p = (char*)ws;
    E* gt = (E*)p; p += align256(N * M * (int64_t)sizeof(E));
    E* xqt = (E*)p; p += align256(K * M * (int64_t)sizeof(E));
    const uint32_t* keept = keep;
    hipLaunchKernelGGL((k_transpose<E>), tgrid_g, dim3(256), 0, s, (const E*)g, M, N, ldg, gt, M);
    if (xq)
      hipLaunchKernelGGL((k_transpose<E>), tgrid_x, dim3(256), 0, s, (const E*)xq, M, K, ldxq, xqt, M);
    else if (cfg->ir_mode == AHL_IR_NONE)
      hipLaunchKernelGGL((k_dac_transpose<D, 0>), tgrid_x, dim3(256), 0, s, x, M, K, ldx, ir, tl, cfg->inp_res, dac_on, cfg->skip_rounding, (void*)xqt);
    else if (cfg->ir_mode == AHL_IR_STATIC)
      hipLaunchKernelGGL((k_dac_transpose<D, 1>), tgrid_x, dim3(256), 0, s, x, M, K, ldx, ir, tl, cfg->inp_res, dac_on, cfg->skip_rounding, (void*)xqt);
    else
      hipLaunchKernelGGL((k_dac_transpose<D, 2>), tgrid_x, dim3(256), 0, s, x, M, K, ldx, ir, tl, cfg->inp_res, dac_on, cfg->skip_rounding, (void*)xqt);
    a.gt = gt; a.keept = keept; a.xqt = xqt; a.clamp_flag = clamp_flag; a.flag_token = cfg->flag_token;
    const bool vec = M % D::EPV == 0;
    const dim3 grid((unsigned)(nbn * nkb)), block(256);
    if (vec) hipLaunchKernelGGL((k_linear_bwd_dw<D, true>), grid, block, kGemmLds, s, a);
    else hipLaunchKernelGGL((k_linear_bwd_dw<D, false>), grid, block, kGemmLds, s, a);
    if (dbias) {
      const int rc = ahl_col_sum(g, cfg->dtype, M, N, ldg, dbias, p, stream);
      if (rc != AHL_OK) return rc;
    }
  });
  return check_launch("ahl_linear_bwd_dw");
}

}  // extern "C"
