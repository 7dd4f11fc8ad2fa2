// bf16 fast path of the analog forward.
//
// Why the DAC is a separate pass here: quantising an A element costs ~7 VALU instructions
// (clamp, scale, two bf16 roundings, round-to-even, rescale) and a block that owns BN output
// columns repeats that work for every one of the N/BN column blocks. At BN = 128 this is ~1.75x
// the MFMA time of the block, on top of a VALU-heavy per-tile epilogue. One
// memory-bound pass (k_dac_rows: read x once, write xq once, dynamic abs-max fused in) removes
// that redundancy; the GEMM then streams xq through LDS untouched. The fused-prologue kernel
// (ahl_gemm.hip) stays for fp32 and for shapes this path does not take.
//
// k_fwd_fast: block 256 threads = 2x2 waves, block tile 128 x 128, wave tile 64 x 64, chunks of 64
// k; accumulator of the running K-tile in fp32 (64 registers), running total packed as bf16
// pairs (32 registers) -- the total is a bf16 quantity by the semantics of the path -- so two
// blocks fit on a CU and the VALU epilogue of one can overlap the MFMA phase of the other. With
// this wave tile the kernel reads 64 KB of MFMA fragments from LDS and writes 32 KB into it per
// 512 MFMA cycles of a SIMD: LDS bandwidth, not the MFMA pipe, bounds the plain product.
#include "ahl_fwd_common.h"
#include <stdlib.h>

namespace ahl {

static constexpr int kLdsStrideF = 144;            // bytes; 128 data + 16 pad
static constexpr int kChunkLdsF = 128 * kLdsStrideF;

// -------------------------------------------------------------------------------------------
// DAC pre-pass, one wave per row: xq[m, k] = DAC(clamp(x[m, k])) with the input range of k's
// tile. Dynamic mode: the range is the row's abs-max inside the tile and is written to
// ir_out[t, m]. Generic in dtype and alignment.
template <class D, bool VEC, int IRMODE>
__global__ __launch_bounds__(256) void k_dac_rows(const void* __restrict__ x, int64_t ldx,
                                                  void* __restrict__ xq, int64_t ldq,
                                                  const void* __restrict__ ir_in,
                                                  void* __restrict__ ir_out, int64_t M, Tiling tl,
                                                  float inp_res, int32_t dac_on,
                                                  int32_t skip_rounding, int32_t qstride) {
  const int lane = threadIdx.x & 63;
  const int64_t m = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (m >= M) return;
  constexpr int E = D::EPV;
  const typename D::elem* row = (const typename D::elem*)x + m * ldx;
  typename D::elem* qrow = (typename D::elem*)xq + m * ldq;
  for (int32_t t = 0; t < tl.n_tiles; ++t) {
    const int32_t c0 = tl.start(t), c1 = tl.start(t + 1);
    float irv;
    if (IRMODE == AHL_IR_DYNAMIC) {
      float mx = 0.0f;
      wave_row_foreach<D, VEC>(row, c0, c1, lane, [&](float v) { mx = fmaxf(mx, fabsf(v)); });
      irv = wave_max(mx);
      if (lane == 0) D::store(ir_out, (int64_t)t * M + m, irv);
    } else {
      irv = D::load(ir_in, t);
    }
    const Dac dac = make_dac<D>(irv, inp_res);
    auto f = [&](float v) -> float {
      if (dac_on) return dac_apply<D, IRMODE == AHL_IR_STATIC, true>(v, dac, skip_rounding != 0);
      return dac_apply<D, IRMODE == AHL_IR_STATIC, false>(v, dac, false);
    };
    // padded tile layout (qstride > 0): tile t of xq starts at column t * qstride and is
    // zero-filled up to the next tile
    typename D::elem* qt = qstride > 0 ? qrow + ((int64_t)t * qstride - c0) : qrow;
    if (VEC) {  // tile bounds are multiples of E on this path
      for (int32_t v = c0 / E + lane; v < c1 / E; v += 64) {
        float e[E];
        D::unpack(ld16(row + (int64_t)v * E), e);
#pragma unroll
        for (int i = 0; i < E; ++i) e[i] = f(e[i]);
        st16(qt + (int64_t)v * E, D::pack(e));
      }
    } else {
      // element-wise, four independent loads per lane and pass
      int32_t c = c0 + lane;
      for (; c + 192 < c1; c += 256) {
        float e[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) e[i] = D::load(row, c + 64 * i);
#pragma unroll
        for (int i = 0; i < 4; ++i) D::store(qt, c + 64 * i, f(e[i]));
      }
      for (; c < c1; c += 64) D::store(qt, c, f(D::load(row, c)));
    }
    if (qstride > 0)
      for (int32_t c = c1 + lane; c < c0 + qstride; c += 64) D::store(qt, c, 0.0f);
  }
}

// QM, what happens to a tile's outputs after the noise: 0 nothing, 1 clamp at the bound, 2 ADC
// quantisation and clamp, 3 the same without the rounding step (skip_rounding). Compile-time, so
// that the per-group epilogue has no branches apart from the rare "something left the range".
template <class D, int IRMODE, bool NOISE, int QM, int NBJ>
__global__ __launch_bounds__(256, NBJ == 1 ? 3 : 2) void k_fwd_fast(FastFwdArgs a) {
  constexpr bool ADC = QM >= 2, CLAMP = QM >= 1, ROUND = QM != 3;
  constexpr int BN = 64 * NBJ;   // block columns
  constexpr int WN = 32 * NBJ;   // wave columns
  constexpr int NB = 2 * NBJ;    // B vectors per thread and chunk
  extern __shared__ __attribute__((aligned(16))) char lds[];
  char* ldsA = lds;
  char* ldsB = lds + kChunkLdsF;
  float* rowc = (float*)(lds + (128 + BN) * kLdsStrideF);  // dynamic mode: [2][3][128] per-row constants

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int row0 = tid >> 3, cv = tid & 7;
  const int h = lane >> 5;

  const int64_t nbn = cdiv_dev(a.N, BN);
  const bool one_tile = a.part != nullptr;
  const int64_t nb = one_tile ? gridDim.x / a.n_tiles : gridDim.x;   // output blocks
  const int t_first = one_tile ? (int)(blockIdx.x / nb) : 0;
  int64_t bm, bn;
  block_to_tile(blockIdx.x % nb, nb, cdiv_dev(a.M, 128), nbn, 8, bm, bn);
  const int64_t m0 = bm * 128, n0 = bn * BN;
  constexpr bool bound_on = CLAMP;

  const NoiseKey nk = noise_key(a.seed, a.offset, a.seed_state);
  f32x16 acc[2][NBJ];
  uint32_t totp[2][NBJ][8];   // running total, bf16 pairs: [g*2 + (c>>1)] = rows c, c+1 of group g
  uint32_t cwords[NBJ];       // lane L: clamp-mask word of row wm * 64 + L for the current tile
#pragma unroll
  for (int j = 0; j < NBJ; ++j) cwords[j] = 0u;
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < NBJ; ++j) {
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;
#pragma unroll
      for (int v = 0; v < 8; ++v) totp[i][j][v] = 0u;
    }
  uint32_t any_clamp = 0u;

  // Operand loads through buffer descriptors: the per-thread byte offset inside the block's
  // row panel is computed once, the k position advances as the scalar offset, and rows beyond
  // the matrix read as zero (out-of-range check of the descriptor) -- no per-chunk address
  // arithmetic and no predicates.
  // (an image operand reads rows beyond its block's: the descriptor spans the allocation)
  const int64_t rowsA = (a.conv.on ? a.conv.alloc_rows : a.M) - m0, rowsB = a.N - n0;
  const uint64_t bytesA = (uint64_t)rowsA * (uint64_t)a.ldx * 2u, bytesB = (uint64_t)rowsB * (uint64_t)a.ldw * 2u;
  const __amdgpu_buffer_rsrc_t rsA = __builtin_amdgcn_make_buffer_rsrc(
      (void*)((const uint16_t*)a.xq + m0 * a.ldx), 0,
      (int)(bytesA > 0xffffffffull ? 0xffffffffu : (uint32_t)bytesA), 0x00020000);
  const __amdgpu_buffer_rsrc_t rsB = __builtin_amdgcn_make_buffer_rsrc(
      (void*)((const uint16_t*)a.w + n0 * a.ldw), 0,
      (int)(bytesB > 0xffffffffull ? 0xffffffffu : (uint32_t)bytesB), 0x00020000);
  int voA[4], voB[NB];
#pragma unroll
  for (int j = 0; j < 4; ++j) voA[j] = (int)(((int64_t)(row0 + 32 * j) * a.ldx + cv * 8) * 2);
#pragma unroll
  for (int j = 0; j < NB; ++j) voB[j] = (int)(((int64_t)(row0 + 32 * j) * a.ldw + cv * 8) * 2);
  u32x4 rawA[4], rawB[NB];
  // chunk li of tile lt: the weights at column lt * tile_stride + 64 li, the input at the same
  // column or, read off an image, at the chunk's (tap, channels) position
  auto load = [&](int lt, int li) {
    const int32_t kcB = lt * a.tile_stride + li * 64;
    const int32_t kcA = a.conv.on ? conv_chunk_offset(a.conv, lt, li, (int32_t)a.ldx) : kcB;
#pragma unroll
    for (int j = 0; j < 4; ++j)
      rawA[j] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rsA, voA[j], kcA * 2, 0));
#pragma unroll
    for (int j = 0; j < NB; ++j)
      rawB[j] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rsB, voB[j], kcB * 2, 0));
  };
  load(t_first, 0);
  const int cpt = a.tile / 64, nchunks = (one_tile ? 1 : a.n_tiles) * cpt;
  // tile and position inside it of the chunk after the one being loaded
  int lt = t_first, lcin = 1;
  if (lcin == cpt) { lcin = 0; ++lt; }
  int t = t_first, cin = 0;
  // registers -> LDS for the chunk held in rawA/rawB; `tt` is its K-tile, `first` whether it
  // opens that tile (then the dynamic-mode per-row constants of the tile are written too)
  auto stage = [&](int tt, bool first) {
    __syncthreads();
#pragma unroll
    for (int j = 0; j < 4; ++j)
      *(u32x4*)(ldsA + (row0 + 32 * j) * kLdsStrideF + cv * 16) = rawA[j];
#pragma unroll
    for (int j = 0; j < NB; ++j)
      *(u32x4*)(ldsB + (row0 + 32 * j) * kLdsStrideF + cv * 16) = rawB[j];
    if (IRMODE == AHL_IR_DYNAMIC && first && tid < 128) {
      const int64_t m = m0 + tid;
      const float irm = m < a.M ? D::load(a.ir, (int64_t)tt * a.M + m) : 0.0f;
      float* rc = rowc + (tt & 1) * 384;
      // a noise scale that is the same for every channel of the tile (the tile's abs-max) is folded
      // in here, once per row, instead of once per element in the epilogue
      const float nrow = D::rd(a.noise_scale * irm);
      rc[tid] = (!NOISE || a.noise_per_channel) ? nrow : D::rd(a.tile_max[tt] * nrow);
      rc[128 + tid] = D::rd(irm * a.out_bound);
    }
    __syncthreads();
  };
  bool prestaged = false;
  for (int ch = 0; ch < nchunks; ++ch) {
    if (!prestaged) stage(t, cin == 0);
    prestaged = false;
    if (ch + 1 < nchunks) {
      load(lt, lcin);
      if (++lcin == cpt) { lcin = 0; ++lt; }
    }

    {
      const int r = lane & 31;
      const char* pa = ldsA + (wm * 64 + r) * kLdsStrideF + h * 16;
      const char* pb = ldsB + (wn * WN + r) * kLdsStrideF + h * 16;
      // fragments of step s + 1 are read while the MFMAs of step s run
      u32x4 fa[2][2], fb[2][NBJ];
      auto read_frags = [&](int s, int buf) {
        fa[buf][0] = *(const u32x4*)(pa + s * 32);
        fa[buf][1] = *(const u32x4*)(pa + 32 * kLdsStrideF + s * 32);
#pragma unroll
        for (int bj = 0; bj < NBJ; ++bj) fb[buf][bj] = *(const u32x4*)(pb + bj * 32 * kLdsStrideF + s * 32);
      };
      read_frags(0, 0);
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        if (s < 3) read_frags(s + 1, (s + 1) & 1);
        const u32x4 a0 = fa[s & 1][0], a1 = fa[s & 1][1];
        if (s == 0 && cin == 0) {  // first step of a K-tile starts from zero
#pragma unroll
          for (int bj = 0; bj < NBJ; ++bj) {
            Mma16<D>::run_zero(a0, fb[s & 1][bj], acc[0][bj]);
            Mma16<D>::run_zero(a1, fb[s & 1][bj], acc[1][bj]);
          }
        } else {
#pragma unroll
          for (int bj = 0; bj < NBJ; ++bj) {
            Mma16<D>::run(a0, fb[s & 1][bj], acc[0][bj]);
            Mma16<D>::run(a1, fb[s & 1][bj], acc[1][bj]);
          }
        }
      }
    }

    if (++cin < cpt) continue;
    cin = 0;
    // The next chunk (first of the next tile) is staged before the epilogue so that the
    // prefetch registers are dead while the epilogue runs.
    if (ch + 1 < nchunks) { stage(t + 1, true); prestaged = true; }
    // ---------------- per-K-tile epilogue ----------------
    const float ir_t = IRMODE == AHL_IR_STATIC ? D::load(a.ir, t) : 0.0f;
    const float tmax = (NOISE || bound_on) ? a.tile_max[t] : 0.0f;
    const float* rc_t = rowc + (t & 1) * 384;
#pragma unroll
    for (int bj = 0; bj < NBJ; ++bj) {
      const int64_t n = n0 + wn * WN + bj * 32 + (lane & 31);
      const bool nvalid = n < a.N;
      float wch = 0.0f;
      if ((NOISE || bound_on) && nvalid) wch = D::load(a.wmax, (int64_t)t * a.N + n);
      const float wr = a.noise_per_channel ? wch : tmax;
      const float wb = a.bound_per_channel ? wch : tmax;
      float nscale = 0.0f, B = 0.0f, r = 1.0f, rcp = 1.0f;
      if (IRMODE == AHL_IR_STATIC) {
        if (NOISE) nscale = D::rd(wr * D::rd(a.noise_scale * ir_t));
        if (bound_on) {
          B = D::rd(D::rd(ir_t * a.out_bound) * wb);
          if (ADC) {
            r = adc_step<D>(B, a);
            rcp = __fdiv_rn(1.0f, fmaxf(r, D::tiny()));
          }
        }
      }
#pragma unroll
      for (int bi = 0; bi < 2; ++bi) {
        const int rbase = wm * 64 + bi * 32 + 4 * h;
#pragma unroll
        for (int gp = 0; gp < 2; ++gp) {
          float xi[8];
          if (NOISE) {
            const uint32_t mrow = (uint32_t)(m0 + rbase + 16 * gp);
            normal8(nk.seed, nk.offset, (uint32_t)t, (uint32_t)n, (mrow >> 4) * 2 + ((mrow >> 2) & 1), xi);
          }
          // "Did an output leave the range" is decided once per eight elements, from a running
          // maximum kept in a vector register: a compare whose result goes to scalar registers
          // (and the scalar OR that collects it) costs the wave tens of cycles each, which eight
          // times per unit was a quarter of the whole epilogue. The rare case redoes the sums
          // with the clamped values. (A NaN output is no longer treated as clamped; it passes
          // through, as it does through torch.clamp.)
          float y8[8], B8[8];
          uint32_t tpo[4];
          float excess = -1.0f;   // max over the unit of |y| - bound
#pragma unroll
          for (int gg = 0; gg < 2; ++gg) {
            const int g = 2 * gp + gg;
            float y[4];
#pragma unroll
            for (int c = 0; c < 4; ++c) y[c] = acc[bi][bj][4 * g + c];
            round2<D>(y[0], y[1]); round2<D>(y[2], y[3]);
            float ns[4], Bv[4], rv[4], rcpv[4];
#pragma unroll
            for (int c = 0; c < 4; ++c) { ns[c] = nscale; Bv[c] = B; rv[c] = r; rcpv[c] = rcp; }
            if (IRMODE == AHL_IR_DYNAMIC && (NOISE || bound_on)) {
              // the four rows of this group are consecutive: one 16-byte LDS read per constant
              const int rl0 = rbase + 8 * g;
              if (NOISE) {
                const f32x4 nr = *(const f32x4*)(rc_t + rl0);
                if (a.noise_per_channel) {   // uniform over the launch
#pragma unroll
                  for (int c = 0; c < 4; ++c) ns[c] = wr * nr[c];
                  round2<D>(ns[0], ns[1]); round2<D>(ns[2], ns[3]);
                } else {
#pragma unroll
                  for (int c = 0; c < 4; ++c) ns[c] = nr[c];   // the row's scale, tile abs-max included
                }
              }
              if (bound_on) {
                const f32x4 br = *(const f32x4*)(rc_t + 128 + rl0);
#pragma unroll
                for (int c = 0; c < 4; ++c) Bv[c] = br[c] * wb;
              }
              if (bound_on) {
                round2<D>(Bv[0], Bv[1]); round2<D>(Bv[2], Bv[3]);
                if (ADC) {
                  if (__builtin_expect(a.step_by_division != 0, 0)) {
#pragma unroll
                    for (int c = 0; c < 4; ++c) rv[c] = adc_step<D>(Bv[c], a);
                  } else {
                    adc_step4<D>(Bv, rv, a);
                  }
#pragma unroll
                  for (int c = 0; c < 4; ++c) rcpv[c] = __builtin_amdgcn_rcpf(fmaxf(rv[c], D::tiny()));
                }
              }
            }
            if (NOISE) {
              // y + scale * xi with one rounding: xi is an fp32 normal, so there is no bf16
              // product of the reference to reproduce, and the sum is rounded once
#pragma unroll
              for (int c = 0; c < 4; ++c) y[c] = __builtin_fmaf(ns[c], xi[4 * gg + c], y[c]);
              round2<D>(y[0], y[1]); round2<D>(y[2], y[3]);
            }
            if (ADC) {
#pragma unroll
              for (int c = 0; c < 4; ++c)
                y[c] = IRMODE != AHL_IR_STATIC ? D::div(y[c], fmaxf(rv[c], D::tiny()), rcpv[c])
                       : ROUND ? D::div_to_round(y[c], fmaxf(rv[c], D::tiny()), rcpv[c])
                               : D::div_exact_rcp(y[c], fmaxf(rv[c], D::tiny()), rcpv[c]);
              round2<D>(y[0], y[1]); round2<D>(y[2], y[3]);
              if (ROUND) {
#pragma unroll
                for (int c = 0; c < 4; ++c) y[c] = rintf(y[c]);
              }
#pragma unroll
              for (int c = 0; c < 4; ++c) y[c] *= rv[c];
              round2<D>(y[0], y[1]); round2<D>(y[2], y[3]);
            }
            if (CLAMP) {
#pragma unroll
              for (int c = 0; c < 4; ++c) {
                y8[4 * gg + c] = y[c];
                B8[4 * gg + c] = Bv[c];
              }
              if (IRMODE == AHL_IR_DYNAMIC) {
#pragma unroll
                for (int c = 0; c < 4; ++c) excess = fmaxf(excess, fabsf(y[c]) - Bv[c]);
              } else {   // one bound for the whole unit
                excess = fmaxf(excess, fmaxf(fmaxf(fabsf(y[0]), fabsf(y[1])), fmaxf(fabsf(y[2]), fabsf(y[3]))) - Bv[0]);
              }
            }
            // total = rd(total + y), bf16 pairs
#pragma unroll
            for (int pr = 0; pr < 2; ++pr) {
              const uint32_t tp = totp[bi][bj][2 * g + pr];
              tpo[2 * gg + pr] = tp;
              totp[bi][bj][2 * g + pr] =
                  D::pack2(D::lo(tp) + y[2 * pr], D::hi(tp) + y[2 * pr + 1]);
            }
          }
          if (CLAMP) {
            const bool over = excess > 0.0f;
            if (__builtin_expect(__any(over), 0)) {
              if (a.keep != nullptr) {
                // the compare's scalar result is the wave's mask bits of two rows
                const uint64_t cols = __builtin_amdgcn_ballot_w64(nvalid);
#pragma unroll
                for (int e = 0; e < 8; ++e)
                  clamp_record_bits(__builtin_amdgcn_ballot_w64(fabsf(y8[e]) > B8[e]) & cols,
                                    32 * bi + 8 * (2 * gp + (e >> 2)) + (e & 3), cwords[bj]);
              }
#pragma unroll
              for (int e = 0; e < 8; ++e) y8[e] = __builtin_amdgcn_fmed3f(y8[e], -B8[e], B8[e]);
#pragma unroll
              for (int q = 0; q < 4; ++q)
                totp[bi][bj][4 * gp + q] =
                    D::pack2(D::lo(tpo[q]) + y8[2 * q], D::hi(tpo[q]) + y8[2 * q + 1]);
              any_clamp = 1u;   // wave-uniform here; only "any lane" is read at the end
            }
          }
          // keep the scheduler from interleaving the 8 Philox/Box-Muller chains of a block:
          // that only lengthens live ranges (the chains of different waves overlap anyway)
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
    if (CLAMP && a.keep != nullptr) {
      // the clamp-mask words of this tile: per 32-column block, the 64 rows of the wave are
      // 256 contiguous bytes
      uint32_t* plane = a.keep + (int64_t)t * clamp_plane_words(a.M, a.N);
      const int64_t m = m0 + wm * 64 + lane;
#pragma unroll
      for (int bj = 0; bj < NBJ; ++bj) {
        const int64_t nb0 = n0 + wn * WN + bj * 32;
        if (m < a.M && nb0 < a.N) plane[clamp_word(m, nb0, a.M)] = cwords[bj];
        cwords[bj] = 0u;
      }
    }
    t += 1;
  }

  // most waves find the flag already set and skip the atomic (atomics on one address are served
  // one after the other)
  if (a.clamp_flag != nullptr && __any(any_clamp != 0u) && lane == 0 &&
      __hip_atomic_load(a.clamp_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != a.flag_value)
    __hip_atomic_store(a.clamp_flag, a.flag_value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);

  // ---- store y = total (+ bias): transposed through LDS, 16-byte row-contiguous stores ----
  {
    constexpr int kOutStride = BN * 2 + 16;  // BN bf16 + 16 bytes pad
    __syncthreads();                         // every wave is done with the operand buffers
    char* obase = lds + (wm * 64 + 4 * h) * kOutStride + (wn * WN + (lane & 31)) * 2;
#pragma unroll
    for (int bj = 0; bj < NBJ; ++bj) {
      const int64_t n = n0 + wn * WN + bj * 32 + (lane & 31);
      const bool add_bias = a.bias != nullptr && !one_tile;
      const float b = (add_bias && n < a.N) ? D::load(a.bias, n) : 0.0f;
#pragma unroll
      for (int bi = 0; bi < 2; ++bi)
#pragma unroll
        for (int pr = 0; pr < 8; ++pr) {
          uint32_t tp = totp[bi][bj][pr];
          if (add_bias) tp = D::pack2(D::lo(tp) + b, D::hi(tp) + b);
          const int ro = bi * 32 + 8 * (pr >> 1) + 2 * (pr & 1);
          *(uint16_t*)(obase + ro * kOutStride + bj * 64) = (uint16_t)tp;
          *(uint16_t*)(obase + (ro + 1) * kOutStride + bj * 64) = (uint16_t)(tp >> 16);
        }
    }
    __syncthreads();
    constexpr int VPR = BN / 8;          // 16-byte vectors per row
    constexpr int RPP = 256 / VPR;       // rows per pass
    const int vcol = tid % VPR, vrow = tid / VPR;
    const int64_t n = n0 + vcol * 8;
    uint16_t* yout = one_tile ? a.part + (int64_t)t_first * a.M * a.N : (uint16_t*)a.y;
    const int64_t ldy = one_tile ? a.N : a.ldy;
#pragma unroll
    for (int j = 0; j < 128 / RPP; ++j) {
      const int row = vrow + RPP * j;
      const int64_t m = m0 + row;
      if (m < a.M && n < a.N)
        st16(yout + m * ldy + n, *(const u32x4*)(lds + row * kOutStride + vcol * 16));
    }
  }
}

// y[m, n] = rd(...rd(rd(0 + part[0]) + part[1])... ) (+ bias): the running total of k_fwd_fast over
// the tiles, for results that were computed one tile per block. One 16-byte vector per thread.
template <class D>
__global__ __launch_bounds__(256) void k_tile_sum(const uint16_t* __restrict__ part, int32_t n_tiles,
                                                  int64_t M, int64_t N, const uint16_t* __restrict__ bias,
                                                  uint16_t* __restrict__ y, int64_t ldy) {
  const int64_t v = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t nv = N / 8;
  if (v >= M * nv) return;
  const int64_t m = v / nv, n = (v - m * nv) * 8;
  float tot[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  for (int t = 0; t < n_tiles; ++t) {
    float e[8];
    D::unpack(ld16(part + ((int64_t)t * M + m) * N + n), e);
#pragma unroll
    for (int i = 0; i < 8; ++i) tot[i] = D::rd(tot[i] + e[i]);
  }
  if (bias != nullptr) {
    float b[8];
    D::unpack(ld16(bias + n), b);
#pragma unroll
    for (int i = 0; i < 8; ++i) tot[i] = D::rd(tot[i] + b[i]);
  }
  st16(y + m * ldy + n, D::pack(tot));
}

__global__ void k_zero_u32(uint32_t* p) { *p = 0u; }

}  // namespace ahl

using namespace ahl;

// number of significant bits of a positive float's significand
static int significant_bits(float v) {
  uint32_t u;
  memcpy(&u, &v, 4);
  uint32_t man = (u & 0x7fffffu) | 0x800000u;
  int bits = 24;
  while (bits > 1 && (man & 1u) == 0u) { man >>= 1; --bits; }
  return bits;
}

template <class D, int IRMODE, int NBJ>
static void launch_fast(const FastFwdArgs& a, bool noise, int qm, hipStream_t s) {
  constexpr int lds_bytes = (128 + 64 * NBJ) * kLdsStrideF + 2 * 384 * (int)sizeof(float);
  const dim3 block(256), grid((unsigned)(cdiv(a.M, 128) * cdiv(a.N, 64 * NBJ) * (a.part ? a.n_tiles : 1)));
#define AHL_FWD(NZ, Q) hipLaunchKernelGGL((k_fwd_fast<D, IRMODE, NZ, Q, NBJ>), grid, block, lds_bytes, s, a)
  if (noise) {
    if (qm == 0) AHL_FWD(true, 0); else if (qm == 1) AHL_FWD(true, 1);
    else if (qm == 2) AHL_FWD(true, 2); else AHL_FWD(true, 3);
  } else {
    if (qm == 0) AHL_FWD(false, 0); else if (qm == 1) AHL_FWD(false, 1);
    else if (qm == 2) AHL_FWD(false, 2); else AHL_FWD(false, 3);
  }
#undef AHL_FWD
}

template <class D>
static void launch_fast_modes(const FastFwdArgs& a, int ir_mode, bool few, bool noise, int qm, hipStream_t s) {
  if (ir_mode == AHL_IR_NONE) few ? launch_fast<D, 0, 1>(a, noise, qm, s) : launch_fast<D, 0, 2>(a, noise, qm, s);
  else if (ir_mode == AHL_IR_STATIC) few ? launch_fast<D, 1, 1>(a, noise, qm, s) : launch_fast<D, 1, 2>(a, noise, qm, s);
  else few ? launch_fast<D, 2, 1>(a, noise, qm, s) : launch_fast<D, 2, 2>(a, noise, qm, s);
}

namespace ahl {

// ahl_fwd_pipe.hip: the kernel for large grids
bool pipe_fwd_eligible(const FastFwdArgs& a, int ir_mode);
bool launch_pipe_fwd(int32_t dtype, const FastFwdArgs& a, int ir_mode, bool noise, int qm, hipStream_t s);

// Few rows (a recurrent step, a decoding step): the 128 x 64 output blocks alone leave most CUs
// idle and every block walks the whole contraction with one chunk in flight. With a workspace
// the K-tiles of an output block go to different blocks as well.
bool fast_fwd_split(int64_t M, int64_t N, int32_t n_tiles) {
  return n_tiles > 1 && cdiv(M, 128) * cdiv(N, 64) <= 256;
}

int64_t fast_fwd_ws_bytes(int64_t M, int64_t N, int32_t n_tiles) {
  return fast_fwd_split(M, N, n_tiles) ? (int64_t)n_tiles * M * N * 2 : 0;
}

// Whether ahl_linear_fwd can take the bf16 fast path for these arguments.
bool fast_fwd_eligible(const AhlLinearCfg* cfg, const void* xq, int64_t ldxq, const void* w,
                       int64_t ldw, int64_t K, const Tiling& tl) {
  if ((cfg->dtype != AHL_BF16 && cfg->dtype != AHL_F16) || xq == nullptr) return false;
  if (cfg->out_res > 0.0f && !(cfg->out_bound > 0.0f)) return false;  // an ADC needs its bound
  if (!aligned16(xq) || !aligned16(w) || ldxq % 8 != 0 || ldw % 8 != 0) return false;
  if (cfg->tile_stride > 0) {  // padded tile layout: any split
    const int64_t padded = (int64_t)tl.n_tiles * cfg->tile_stride;
    return cfg->tile_stride % 256 == 0 && cfg->tile_stride >= widest_tile(tl) && ldxq >= padded &&
           ldw >= padded && padded <= 0x3fffffff;
  }
  if (tl.extra != 0 || tl.base % 64 != 0) return false;
  return K % 64 == 0;  // the caller also checks N % 8, ldy % 8 and the alignment of y and the clamp mask
}

int launch_fast_fwd(const void* xq, int64_t ldxq, const void* w_eff, int64_t ldw, const void* bias,
                    void* y, int64_t ldy, uint32_t* keep, uint32_t* clamp_flag, const void* ir,
                    const void* wmax, const float* tile_max, int64_t M, int64_t K, int64_t N,
                    const Tiling& tl, const AhlLinearCfg* cfg, void* ws, hipStream_t s,
                    const ConvMap* conv) {
  FastFwdArgs a;
  a.xq = xq; a.ldx = ldxq; a.w = w_eff; a.ldw = ldw; a.bias = bias; a.y = y; a.ldy = ldy;
  a.keep = keep; a.clamp_flag = clamp_flag; a.ir = ir; a.wmax = wmax; a.tile_max = tile_max;
  a.M = M; a.N = N; a.n_tiles = tl.n_tiles;
  memset(&a.conv, 0, sizeof(a.conv));
  if (conv != nullptr) a.conv = *conv;
  if (cfg->tile_stride > 0) {  // padded tile layout: only the chunks that hold data are visited
    a.tile = (int32_t)cdiv(widest_tile(tl), 64) * 64;
    a.tile_stride = cfg->tile_stride;
  } else {
    a.tile = tl.base;
    a.tile_stride = tl.base;
  }
  (void)K;
  a.out_bound = cfg->out_bound; a.out_res = cfg->out_res;
  const bool noise = cfg->training && cfg->out_noise > 0.0f;
  const bool adc = cfg->out_res > 0.0f;
  a.noise_scale = noise ? (float)((double)cfg->out_noise / sqrt((double)tl.n_tiles)) : 0.0f;
  a.noise_per_channel = cfg->out_noise_per_channel; a.bound_per_channel = cfg->bound_per_channel;
  a.skip_rounding = cfg->skip_rounding; a.clamp_on = cfg->out_bound > 0.0f ? 1 : 0;
  const bool states = cfg->out_res > 1.0f;
  const int exact_bits = cfg->dtype == AHL_F16 ? F16::kExactStepBits : BF16::kExactStepBits;
  a.step_by_division = (adc && states && significant_bits(cfg->out_res) > exact_bits) ? 1 : 0;
  a.step_factor = !adc ? 0.0f : states ? 2.0f / cfg->out_res : 2.0f * cfg->out_res;
  a.seed = cfg->seed; a.offset = cfg->offset; a.seed_state = cfg->seed_state;
  if (cdiv(M, 128) * cdiv(N, 64) > 0x7fffffff) return AHL_ERR_ARG;
  // the caller's token needs no cleared word: whatever the word holds, it is not the token
  // (or it is by accident, and the backward then applies a mask that clamps nothing)
  a.flag_value = cfg->flag_token ? cfg->flag_token : 1u;
  if (clamp_flag && !cfg->flag_token) hipLaunchKernelGGL(k_zero_u32, dim3(1), dim3(1), 0, s, clamp_flag);
  // 128 x 128 blocks (NBJ = 2). Measured alternatives: 128 x 64 blocks (NBJ = 1, three to four
  // blocks per CU) are ~10 % slower, 256 x 128 blocks (one block of 8 waves per CU) ~15 % slower.
  // When those are too few to give every CU a block (few rows: a recurrent step, a small batch),
  // the 128 x 64 blocks double the count.
  const bool few = cdiv(M, 128) * cdiv(N, 128) < 200;
  const bool split = ws != nullptr && aligned16(ws) && (!bias || aligned16(bias)) && !a.conv.on &&
                     fast_fwd_split(M, N, tl.n_tiles);
  a.part = split ? (uint16_t*)ws : nullptr;
  const int qm = adc ? (cfg->skip_rounding ? 3 : 2) : (a.clamp_on ? 1 : 0);
  // Large grids go to the kernel that runs a tile's epilogue inside the next tile's product loop
  // (same results bit for bit); AHL_FORWARD_KERNEL=blocks in the environment keeps them here.
  const char* pick = getenv("AHL_FORWARD_KERNEL");
  if (!(pick != nullptr && strcmp(pick, "blocks") == 0) && pipe_fwd_eligible(a, cfg->ir_mode) &&
      launch_pipe_fwd(cfg->dtype, a, cfg->ir_mode, noise, qm, s))
    return check_launch("ahl_linear_fwd(pipe)");
  const dim3 sum_grid((unsigned)cdiv(M * (N / 8), 256));
  if (cfg->dtype == AHL_F16) {
    launch_fast_modes<F16>(a, cfg->ir_mode, few, noise, qm, s);
    if (split)
      hipLaunchKernelGGL(k_tile_sum<F16>, sum_grid, dim3(256), 0, s, a.part, tl.n_tiles, M, N,
                         (const uint16_t*)bias, (uint16_t*)y, ldy);
  } else {
    launch_fast_modes<BF16>(a, cfg->ir_mode, few, noise, qm, s);
    if (split)
      hipLaunchKernelGGL(k_tile_sum<BF16>, sum_grid, dim3(256), 0, s, a.part, tl.n_tiles, M, N,
                         (const uint16_t*)bias, (uint16_t*)y, ldy);
  }
  return check_launch("ahl_linear_fwd(fast)");
}

}  // namespace ahl

#define AHL_DAC(V, I)                                                                          \
  hipLaunchKernelGGL((k_dac_rows<D, V, I>), grid, block, 0, s, x, ldx, xq, ldxq, ir_in, ir_out, M, \
                     tl, cfg->inp_res, dac_on, cfg->skip_rounding, qstride)

extern "C" {

int ahl_dac(const void* x, int64_t ldx, void* xq, int64_t ldxq, const void* ir_in, void* ir_out,
            int64_t M, int64_t K, const int32_t* tile_ends_host, int32_t n_tiles,
            const AhlLinearCfg* cfg, void* stream) {
  if (!cfg || !x || !xq || M <= 0 || K <= 0 || ldx < K || ldxq < K) return AHL_ERR_ARG;
  if (cfg->ir_mode == AHL_IR_STATIC && !ir_in) return AHL_ERR_ARG;
  if (cfg->ir_mode == AHL_IR_DYNAMIC && !ir_out) return AHL_ERR_ARG;
  if (cfg->ir_mode == AHL_IR_NONE && cfg->inp_res > 0.0f) return AHL_ERR_ARG;
  Tiling tl;
  if (!make_tiling(tile_ends_host, n_tiles, K, &tl)) return AHL_ERR_TILING;
  const int32_t qstride = cfg->tile_stride;
  if (qstride < 0 || qstride % 256 != 0) return AHL_ERR_ARG;
  if (qstride > 0 && (qstride < widest_tile(tl) || ldxq < (int64_t)n_tiles * qstride)) return AHL_ERR_ARG;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)cdiv(M, 4)), block(256);
  const int32_t dac_on = cfg->inp_res > 0.0f ? 1 : 0;
  AHL_DISPATCH_DTYPE(cfg->dtype, {
    const bool vec = aligned16(x) && aligned16(xq) && ldx % D::EPV == 0 && ldxq % D::EPV == 0 &&
                     tl.extra == 0 && tl.base % D::EPV == 0;
    if (vec) {
      if (cfg->ir_mode == AHL_IR_NONE) { AHL_DAC(true, 0); }
      else if (cfg->ir_mode == AHL_IR_STATIC) { AHL_DAC(true, 1); }
      else { AHL_DAC(true, 2); }
    } else {
      if (cfg->ir_mode == AHL_IR_NONE) { AHL_DAC(false, 0); }
      else if (cfg->ir_mode == AHL_IR_STATIC) { AHL_DAC(false, 1); }
      else { AHL_DAC(false, 2); }
    }
  });
  return check_launch("ahl_dac");
}

}  // extern "C"
