// Analog forward in a 16-bit type (bf16, float16) for large grids with a learned (static) input
// range ("bf16" below stands for either: same registers, same packing). The per-K-tile
// epilogue of tile t - 1 runs inside the product loop of tile t, and the operands go from global
// memory straight into LDS two chunks ahead.
//
//   block = 8 waves (two per SIMD), output tile 256 x 128, wave tile 64 x 64 = 2 x 2 MFMA blocks of
//   32 x 32 (64 fp32 accumulators). A 256 x 128 block moves 3/4 of the operand bytes per flop of
//   the 128 x 128 blocks of k_fwd_fast.
//   Operands: 64-wide k chunks, buffer_load ... lds (no staging registers, no LDS write
//   instructions), three LDS stages, one barrier per chunk. While chunk c is multiplied the
//   loads of chunks c + 1 and c + 2 are in flight: with one chunk ahead (48 KB per CU in flight)
//   the product alone is bound by the latency of those loads (about 1 us under load). Rows are
//   128 bytes, their eight 16-byte slots XOR-swizzled with bits 1-3 of the row number so that the
//   16-byte fragment reads are conflict-free. Rows beyond the matrix read as zero (buffer
//   descriptor bounds).
//   At the end of K-tile t the accumulators are rounded to bf16 (the first step of the epilogue
//   anyway) and parked as 32 registers of bf16 pairs; the accumulators start K-tile t + 1 from
//   zero. The parked tile is worked off in 8 "units" of 8 elements per lane (one Philox call
//   each), a unit per 64-wide chunk of the next tile (512-wide tiles), its pieces alternating
//   with the chunk's MFMAs in the instruction stream. The first tile's product and the last
//   tile's epilogue run alone.
//   "Did an output leave the ADC range" is a running maximum in a vector register and one
//   compare per unit, looked at in the middle of the next unit: compares that write scalar
//   registers, the scalar ORs that collect them and a branch right behind them cost this kernel
//   a quarter of its epilogue time when they were done per element.
//
// Measured on MI355X at 8192 x 4096 x 4096, 8 tiles of 512 (alternating launches, same box):
// 405 us against 422 us for k_fwd_fast with output noise, ADC and clamp mask; 335 against 360
// without the noise; 272 against 315 for the bare product with running totals. What is left is
// the vector work of the epilogue (about 290 us of this kernel's time without the MFMAs) plus
// the matrix time (about 100 us): the two do not overlap on this hardware beyond that, wherever
// the MFMAs sit in the stream (next to the integer work of Philox, next to the fp32 work of the
// ADC, with accumulators in vector or in accumulation registers; all measured).
//
// Results are bit-identical to k_fwd_fast (ahl_fast.hip), which stays for small grids, few rows,
// the dynamic input range (no gain measured there) and other tile widths: same arithmetic per
// element, same Philox counters (tile, row group, column).
#include "ahl_fwd_common.h"
#include "ahl_lds_direct.h"
#include <type_traits>

namespace ahl {

static constexpr int kPRow = 128;                     // bytes per LDS operand row: 64 bf16, no padding
static constexpr int kPLdsA = 256 * kPRow;
static constexpr int kPLdsB = 128 * kPRow;
static constexpr int kPStage = kPLdsA + kPLdsB;       // 49152
static constexpr int kPStages = 3;
static constexpr int kPRowc = kPStages * kPStage;     // dynamic range: [2][2][256] per-row constants
static constexpr int kPColc = kPRowc + 2 * 2 * 256 * (int)sizeof(float);   // [8 waves][2][32][4] per-column constants
static constexpr int kPColw = kPColc + 8 * 2 * 32 * 4 * (int)sizeof(float);  // [8 waves][2][32][2] (dynamic range)
static constexpr int kPLdsBytes = kPColw + 8 * 2 * 32 * 2 * (int)sizeof(float);

template <bool V> using flag = std::integral_constant<bool, V>;

// CPT: 64-wide chunks per K-tile (4 or 8: tiles of 256 or 512 columns).
// NBI: 32-row MFMA blocks per wave: 2 (eight waves of 64 x 64, two per SIMD) is what is built. 4
// (four waves of 128 x 64, one per SIMD, accumulators in accumulation registers) halves the LDS
// reads per flop but was 25 % slower: a SIMD issues at most one instruction of ONE wave per 4-5
// cycles whatever its kind, and vector throughput for the epilogue's instruction mix is up to
// 1.9 x higher with two waves.
// EXTRA: K-tiles of more than CPT chunks (any multiple of 64 columns from 576 up; the K-tiles of a
// convolution read off the image, whose A operand takes its chunk offsets from the ConvMap): the
// first CPT chunks of a tile carry the epilogue of the tile before, the others are product only.
template <class D, int IRMODE, bool NOISE, int QM, int CPT, int NBI, bool EXTRA = false>
__global__ __launch_bounds__(1024 / NBI, NBI == 4 ? 1 : 2) void k_fwd_pipe(FastFwdArgs a) {
  constexpr bool ADC = QM >= 2, CLAMP = QM >= 1, ROUND = QM != 3;
  constexpr bool bound_on = CLAMP;
  constexpr int NT = 1024 / NBI;       // threads
  constexpr int NU = 4 * NBI;          // epilogue units per tile
  constexpr int KPU = CPT / NBI;       // k-steps of 16 that share a region with one epilogue unit
  extern __shared__ __attribute__((aligned(16))) char lds[];
  float* rowc = (float*)(lds + kPRowc);

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int h = lane >> 5, r = lane & 31;

  int64_t bm, bn;
  block_to_tile(blockIdx.x, gridDim.x, cdiv_dev(a.M, 256), cdiv_dev(a.N, 128), 4, bm, bn);
  const int64_t m0 = bm * 256, n0 = bn * 128;
  const NoiseKey nk = noise_key(a.seed, a.offset, a.seed_state);

  f32x16 acc[NBI][2];
  uint32_t pend[NBI][2][8];   // the finished K-tile, bf16 pairs: [g*2 + (c>>1)] = rows c, c+1 of group g
  uint32_t totp[NBI][2][8];   // running total, same layout
  uint32_t cwords[NBI / 2][2];   // [half][bj], lane L: clamp-mask word of row wm*32*NBI + half*64 + L
#pragma unroll
  for (int i = 0; i < NBI; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
#pragma unroll
      for (int v = 0; v < 8; ++v) { totp[i][j][v] = 0u; pend[i][j][v] = 0u; }
    }
#pragma unroll
  for (int i = 0; i < NBI / 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) cwords[i][j] = 0u;
  uint32_t any_clamp = 0u;

  // operand loads through buffer descriptors (see k_fwd_fast)
  const int64_t rowsA = (EXTRA && a.conv.on ? a.conv.alloc_rows : a.M) - m0, rowsB = a.N - n0;
  const uint64_t bytesA = (uint64_t)rowsA * (uint64_t)a.ldx * 2u, bytesB = (uint64_t)rowsB * (uint64_t)a.ldw * 2u;
  const __amdgpu_buffer_rsrc_t rsA = __builtin_amdgcn_make_buffer_rsrc(
      (void*)((const uint16_t*)a.xq + m0 * a.ldx), 0,
      (int)(bytesA > 0xffffffffull ? 0xffffffffu : (uint32_t)bytesA), 0x00020000);
  const __amdgpu_buffer_rsrc_t rsB = __builtin_amdgcn_make_buffer_rsrc(
      (void*)((const uint16_t*)a.w + n0 * a.ldw), 0,
      (int)(bytesB > 0xffffffffull ? 0xffffffffu : (uint32_t)bytesB), 0x00020000);
  // Operands go from global memory straight into LDS (buffer_load_dwordx4 ... lds: no staging
  // registers, no LDS write instructions), three stages of one 64-wide chunk each. One wave
  // instruction moves 8 rows of 128 bytes: lane L brings what lies in 16-byte slot L & 7 of row
  // L >> 3, which is the row's logical slot (L & 7) ^ key(row), key(row) = (row >> 1) & 7; with
  // that swizzle the 16-byte fragment reads of 16 consecutive rows hit 16 different bank groups.
  constexpr int NW = 16 / NBI;             // waves
  constexpr int NLA = 32 / NW, NLB = 16 / NW;   // load instructions per wave and chunk
  int voA[NLA], voB[NLB];
#pragma unroll
  for (int j = 0; j < NLA; ++j) {
    const int row = wave * (8 * NLA) + 8 * j + (lane >> 3);
    voA[j] = (int)(((int64_t)row * a.ldx + (((lane & 7) ^ ((row >> 1) & 7)) * 8)) * 2);
  }
#pragma unroll
  for (int j = 0; j < NLB; ++j) {
    const int row = wave * (8 * NLB) + 8 * j + (lane >> 3);
    voB[j] = (int)(((int64_t)row * a.ldw + (((lane & 7) ^ ((row >> 1) & 7)) * 8)) * 2);
  }
  int st_load = 0;   // stage the next chunk is loaded into
  const int cpt = EXTRA ? a.tile / 64 : CPT;   // chunks per K-tile
  const int nchunks = a.n_tiles * cpt;
  int32_t knext = 0;   // k offset of the next chunk to load
  int lcin = 0;        // its position inside its tile
  int lt = 0;          // its tile (EXTRA)
  auto load = [&](int32_t kc) __attribute__((always_inline)) {
    char* sa = lds + st_load * kPStage + wave * (8 * NLA * kPRow);
    char* sb = lds + st_load * kPStage + kPLdsA + wave * (8 * NLB * kPRow);
    // an image operand: the chunk's (tap, channels) position instead of the weights' column
    const int32_t kcA = (EXTRA && a.conv.on) ? conv_chunk_offset(a.conv, lt, lcin, (int32_t)a.ldx) : kc;
#pragma unroll
    for (int j = 0; j < NLA; ++j)
      load_to_lds16(rsA, sa + j * 8 * kPRow, voA[j], kcA * 2);
#pragma unroll
    for (int j = 0; j < NLB; ++j)
      load_to_lds16(rsB, sb + j * 8 * kPRow, voB[j], kc * 2);
    st_load = st_load == kPStages - 1 ? 0 : st_load + 1;
  };
  constexpr int kLoads = NLA + NLB;   // vector memory operations of one chunk, per wave

  auto advance = [&]() __attribute__((always_inline)) {
    knext += 64;
    if (++lcin == cpt) { lcin = 0; ++lt; knext += a.tile_stride - a.tile; }
  };
  // dynamic range: the per-row constants of tile tt, one row per thread
  auto write_rowc = [&](int tt) __attribute__((always_inline)) {
    if (IRMODE == AHL_IR_DYNAMIC && (NOISE || bound_on) && tid < 256) {
      const int64_t m = m0 + tid;
      const float irm = m < a.M ? D::load(a.ir, (int64_t)tt * a.M + m) : 0.0f;
      float* rc = rowc + (tt & 1) * 512;
      rc[tid] = D::rd(a.noise_scale * irm);
      rc[256 + tid] = D::rd(irm * a.out_bound);
    }
  };

  // Chunk c lives in stage c % 3. While chunk c is multiplied the loads of chunks c + 1 and c + 2
  // are in flight; the barrier at the end of chunk c follows "this wave's part of chunk c + 1 has
  // landed" (at most the loads of chunk c + 2 still fly), and after it the stage of chunk c takes
  // chunk c + 3.
  load(0); advance();
  load(knext); advance();   // chunks 1 and 2 (a tile has at least 4 chunks)
  load(knext); advance();
  write_rowc(0);
  lds_barrier<2 * kLoads>();
  int ch = 0;               // chunk being multiplied

  // LDS offsets in the stage being read, with the lane's share of the slot swizzle folded in:
  // the fragment of k-step s lies at offset ^ (s << 5)
  uint32_t rdA = (wm * 32 * NBI + r) * kPRow + ((h ^ ((r >> 1) & 7)) << 4);
  uint32_t rdB = kPLdsA + (wn * 64 + r) * kPRow + ((h ^ ((r >> 1) & 7)) << 4);
  int st_read = 0;
  asm volatile("" : "+v"(rdA), "+v"(rdB));
  const int64_t nbase = n0 + wn * 64 + r;   // this lane's column in MFMA block bj: nbase + 32 bj
  const bool ncheck = (a.N & 63) != 0;      // some block of 64 columns is not whole
  float wch[2] = {0.0f, 0.0f};              // per-channel abs-max of the tile whose product is running
  // per-column constants of the tile in the epilogue, 8 floats per column: noise scale, bound,
  // ADC step, its reciprocal, abs-max for the noise, abs-max for the bound
  float* colc = (float*)(lds + kPColc) + wave * 256 + r * 4;
  float* colw = (float*)(lds + kPColw) + wave * 128 + r * 2;

  // Fragment registers of two consecutive k-steps (k-step sg uses set sg & 1): the reads of
  // k-step sg + 1 are issued when the first MFMA of k-step sg is.
  u32x4 fa[2][NBI], fb[2][2];
  auto read_frags = [&](int s, int buf) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < NBI; ++i) fa[buf][i] = *(const u32x4*)(lds + (rdA ^ (s << 5)) + i * 32 * kPRow);
#pragma unroll
    for (int j = 0; j < 2; ++j) fb[buf][j] = *(const u32x4*)(lds + (rdB ^ (s << 5)) + j * 32 * kPRow);
  };
  // end of a chunk: the stage it occupied takes the chunk after next; the next chunk must have
  // landed before anyone reads it
  auto end_chunk = [&]() __attribute__((always_inline)) {
    if (ch + 2 < nchunks) lds_barrier<kLoads>(); else lds_barrier<0>();
    if (ch + 3 < nchunks) { load(knext); advance(); }
    const bool wrap = st_read == kPStages - 1;
    st_read = wrap ? 0 : st_read + 1;
    rdA += wrap ? -(kPStages - 1) * kPStage : kPStage;
    rdB += wrap ? -(kPStages - 1) * kPStage : kPStage;
    asm volatile("" : "+v"(rdA), "+v"(rdB));
    ++ch;
  };

  // EXTRA: the chunks of a tile beyond the first CPT, product only
  auto plain_chunks = [&]() __attribute__((always_inline)) {
    if (!EXTRA) return;
    for (int x = CPT; x < cpt; ++x) {
      read_frags(0, 0);
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        if (s < 3) read_frags(s + 1, (s + 1) & 1);
#pragma unroll
        for (int i = 0; i < NBI; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j) Mma16<D>::run(fa[s & 1][i], fb[s & 1][j], acc[i][j]);
      }
      end_chunk();
    }
  };

  // One K-tile phase: the product of tile t (MMA) and the epilogue of tile t - 1 (EPI).
  //
  // The epilogue of the parked tile is 4 NBI units (MFMA block bi, bj and half gp of its row
  // groups: 8 elements per lane, one Philox call); a unit is cut into 16 pieces of 8-20 vector
  // instructions, and the KPU k-steps that belong to the unit are dealt out over its pieces 2..15,
  // with a scheduling barrier after every piece. That order matters with one wave per SIMD (left
  // alone the compiler issues the MFMAs of a region back to back, and the SIMD then does nothing
  // else for their 32 cycles each); with two waves per SIMD no placement of the MFMAs inside the
  // unit made a measurable difference.
  auto phase = [&](auto mma_c, auto epi_c, const int t) __attribute__((always_inline)) {
    constexpr bool MMA = decltype(mma_c)::value, EPI = decltype(epi_c)::value;
    const int te = t - 1;
    if (EPI && (NOISE || bound_on)) {
      const float ir_t = IRMODE == AHL_IR_STATIC ? D::load(a.ir, te) : 0.0f;
      const float tmax = a.tile_max[te];
#pragma unroll
      for (int bj = 0; bj < 2; ++bj) {
        const float wr_ = a.noise_per_channel ? wch[bj] : tmax;
        const float wb_ = a.bound_per_channel ? wch[bj] : tmax;
        float nscale = 0.0f, Bc = 0.0f, rc = 1.0f, rcpc = 1.0f;
        if (IRMODE == AHL_IR_STATIC) {
          if (NOISE) nscale = D::rd(wr_ * D::rd(a.noise_scale * ir_t));
          if (bound_on) {
            Bc = D::rd(D::rd(ir_t * a.out_bound) * wb_);
            if (ADC) {
              rc = adc_step<D>(Bc, a);
              rcpc = __fdiv_rn(1.0f, fmaxf(rc, D::tiny()));
            }
          }
        }
        const f32x4 c0 = {nscale, Bc, rc, rcpc};
        *(f32x4*)(colc + bj * 128) = c0;
        if (IRMODE == AHL_IR_DYNAMIC) {
          const f32x2 c1 = {wr_, wb_};
          *(f32x2*)(colw + bj * 64) = c1;
        }
      }
    }
    if (MMA && (NOISE || bound_on)) {
#pragma unroll
      for (int bj = 0; bj < 2; ++bj)
        wch[bj] = nbase + 32 * bj < a.N ? D::load(a.wmax, (int64_t)t * a.N + nbase + 32 * bj) : 0.0f;
    }
    const float* rc_t = rowc + (te & 1) * 512;

    if (MMA && !EPI) {
      // the first tile: product only
#pragma unroll
      for (int sg = 0; sg < 4 * CPT; ++sg) {
        const int s = sg & 3;
        if (s == 0) read_frags(0, 0);
        if (s < 3) read_frags(s + 1, (s + 1) & 1);
#pragma unroll
        for (int i = 0; i < NBI; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            if (sg == 0) Mma16<D>::run_zero(fa[s & 1][i], fb[s & 1][j], acc[i][j]);
            else Mma16<D>::run(fa[s & 1][i], fb[s & 1][j], acc[i][j]);
          }
        if (s == 3) end_chunk();
      }
      plain_chunks();
      if (t + 1 < a.n_tiles) write_rowc(t + 1);
    } else {
      // The "did an output leave the range" branch of unit u is taken in the middle of unit
      // u + 1: a branch on a vector compare waits for the compare to leave the pipeline. The
      // unit's outputs stay in registers until then and join the running totals after it, so
      // that the (not so rare, with clipped weights) clamp path has no sums to redo.
      float yp[8], Bp[8];
      bool overp = false;
      auto resolve = [&](int pu) __attribute__((always_inline)) {
        if (!(EPI && CLAMP)) return;
        const int pbi = pu >> 2, pbj = (pu >> 1) & 1, pgp = pu & 1;
        // rare: an output of that unit left the range; its sums are redone with the clamped values
        // (not rare at all with wide weight distributions: kept to a compare, two lane writes and a
        // median per element; the compare's scalar result IS the wave's mask bits of two rows)
        if (__builtin_expect(__any(overp), 0)) {
          if (a.keep != nullptr) {
            if (__builtin_expect(ncheck, 0)) {
              const uint64_t cols = __builtin_amdgcn_ballot_w64(nbase + 32 * pbj < a.N);   // columns that exist
#pragma unroll
              for (int e = 0; e < 8; ++e)
                clamp_record_bits(__builtin_amdgcn_ballot_w64(fabsf(yp[e]) > Bp[e]) & cols,
                                  32 * (pbi & 1) + 8 * (2 * pgp + (e >> 2)) + (e & 3), cwords[pbi >> 1][pbj]);
            } else {
              // four compares, then their eight lane writes: a lane write right behind the compare
              // whose scalar result it takes waits out the distance
#pragma unroll
              for (int e0 = 0; e0 < 8; e0 += 4) {
                uint64_t bits[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) bits[e] = __builtin_amdgcn_ballot_w64(fabsf(yp[e0 + e]) > Bp[e0 + e]);
                asm volatile("" : "+s"(bits[0]), "+s"(bits[1]), "+s"(bits[2]), "+s"(bits[3]));
#pragma unroll
                for (int e = 0; e < 4; ++e)
                  clamp_record_bits(bits[e], 32 * (pbi & 1) + 8 * (2 * pgp + (e0 >> 2)) + e, cwords[pbi >> 1][pbj]);
              }
            }
          }
#pragma unroll
          for (int e = 0; e < 8; ++e) yp[e] = __builtin_amdgcn_fmed3f(yp[e], -Bp[e], Bp[e]);
          any_clamp = 1u;   // wave-uniform here; only "any lane" is read at the end
        }
        // total = rd(total + y), bf16 pairs
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const uint32_t tp = totp[pbi][pbj][4 * pgp + q];
          totp[pbi][pbj][4 * pgp + q] = D::pack2(D::lo(tp) + yp[2 * q], D::hi(tp) + yp[2 * q + 1]);
        }
      };
#pragma unroll
      for (int u = 0; u < NU; ++u) {
        const int bi = u >> 2, bj = (u >> 1) & 1, gp = u & 1;
        const int rbase = wm * 32 * NBI + bi * 32 + 4 * h;
        constexpr int MPS = 2 * NBI;    // MFMAs of a k-step
        constexpr int NM = MPS * KPU;   // MFMAs of a unit
        // MFMA m of the unit (k-step m / MPS, block (m / 2) % NBI, m % 2) goes in front of piece
        // 2 + m * 14 / NM; with it, when it opens a k-step, the fragment reads of the next one
        auto mfmas = [&](int piece) __attribute__((always_inline)) {
          if (!MMA) return;
          if (piece == 0 && (u * KPU) % 4 == 0) read_frags(0, 0);   // first k-step after a barrier
#pragma unroll
          for (int m = 0; m < NM; ++m) {
            if (2 + m * 14 / NM != piece) continue;
            const int sg = u * KPU + m / MPS, s = sg & 3;
            if (m % MPS == 0 && s < 3) read_frags(s + 1, (s + 1) & 1);
            const int i = (m >> 1) % NBI, j = m & 1;
            if (sg == 0) Mma16<D>::run_zero(fa[s & 1][i], fb[s & 1][j], acc[i][j]);
            else Mma16<D>::run(fa[s & 1][i], fb[s & 1][j], acc[i][j]);
          }
        };
        float y[8], xi[8], ns[8], Bv[8], rv[8], rcpv[8];
        float wr_ = 0.0f, wb_ = 0.0f;
        u32x4 pc = {0u, 0u, 0u, 0u};
        uint32_t k0 = (uint32_t)nk.seed, k1 = (uint32_t)(nk.seed >> 32);
        // noise, ADC of elements e, e + 1
        auto element_pair = [&](int e) __attribute__((always_inline)) {
          if (NOISE) {
            // y + scale * xi with one rounding: xi is an fp32 normal, so there is no bf16 product
            // of the reference to reproduce, and the sum is rounded once
            y[e] = __builtin_fmaf(ns[e], xi[e], y[e]);
            y[e + 1] = __builtin_fmaf(ns[e + 1], xi[e + 1], y[e + 1]);
            round2<D>(y[e], y[e + 1]);
          }
          if (ADC) {
            if (IRMODE == AHL_IR_STATIC) {   // the per-column reciprocal is correctly rounded
              y[e] = ROUND ? D::div_to_round(y[e], fmaxf(rv[e], D::tiny()), rcpv[e])
                           : D::div_exact_rcp(y[e], fmaxf(rv[e], D::tiny()), rcpv[e]);
              y[e + 1] = ROUND ? D::div_to_round(y[e + 1], fmaxf(rv[e + 1], D::tiny()), rcpv[e + 1])
                               : D::div_exact_rcp(y[e + 1], fmaxf(rv[e + 1], D::tiny()), rcpv[e + 1]);
            } else {
              y[e] = D::div(y[e], fmaxf(rv[e], D::tiny()), rcpv[e]);
              y[e + 1] = D::div(y[e + 1], fmaxf(rv[e + 1], D::tiny()), rcpv[e + 1]);
            }
            round2<D>(y[e], y[e + 1]);
            if (ROUND) { y[e] = rintf(y[e]); y[e + 1] = rintf(y[e + 1]); }
            y[e] *= rv[e]; y[e + 1] *= rv[e + 1];
            round2<D>(y[e], y[e + 1]);
          }
        };
        // dynamic range: the constants of the four consecutive rows of group gg
        auto row_consts = [&](int gg) __attribute__((always_inline)) {
          if (IRMODE == AHL_IR_DYNAMIC && (NOISE || bound_on)) {
            const int rl0 = rbase + 8 * (2 * gp + gg);
            float* nsg = ns + 4 * gg; float* Bg = Bv + 4 * gg; float* rg = rv + 4 * gg; float* rcg = rcpv + 4 * gg;
            if (NOISE) {
              const f32x4 nr = *(const f32x4*)(rc_t + rl0);
#pragma unroll
              for (int c = 0; c < 4; ++c) nsg[c] = wr_ * nr[c];
              round2<D>(nsg[0], nsg[1]); round2<D>(nsg[2], nsg[3]);
            }
            if (bound_on) {
              const f32x4 br = *(const f32x4*)(rc_t + 256 + rl0);
#pragma unroll
              for (int c = 0; c < 4; ++c) Bg[c] = br[c] * wb_;
              round2<D>(Bg[0], Bg[1]); round2<D>(Bg[2], Bg[3]);
              if (ADC) {
                if (__builtin_expect(a.step_by_division != 0, 0)) {
#pragma unroll
                  for (int c = 0; c < 4; ++c) rg[c] = adc_step<D>(Bg[c], a);
                } else {
                  adc_step4<D>(Bg, rg, a);
                }
#pragma unroll
                for (int c = 0; c < 4; ++c) rcg[c] = __builtin_amdgcn_rcpf(fmaxf(rg[c], D::tiny()));
              }
            }
          }
        };
        auto totals = [&](int gg) __attribute__((always_inline)) {
          // without a clamp there is nothing to wait for: total = rd(total + y) right away
#pragma unroll
          for (int pr = 0; pr < 2; ++pr) {
            const int idx = 2 * (2 * gp + gg) + pr;
            const uint32_t tp = totp[bi][bj][idx];
            totp[bi][bj][idx] = D::pack2(D::lo(tp) + y[4 * gg + 2 * pr], D::hi(tp) + y[4 * gg + 2 * pr + 1]);
          }
        };
        bool over = false;
#pragma unroll
        for (int piece = 0; piece < 16; ++piece) {
          mfmas(piece);
          if (EPI) {
            if (piece == 0) {
              const f32x4 cc = (NOISE || bound_on) ? *(const f32x4*)(colc + bj * 128) : f32x4{0.f, 0.f, 1.f, 1.f};
#pragma unroll
              for (int e = 0; e < 8; ++e) { ns[e] = cc[0]; Bv[e] = cc[1]; rv[e] = cc[2]; rcpv[e] = cc[3]; }
              if (IRMODE == AHL_IR_DYNAMIC && (NOISE || bound_on)) {
                const f32x2 cw = *(const f32x2*)(colw + bj * 64);
                wr_ = cw[0]; wb_ = cw[1];
              }
#pragma unroll
              for (int q = 0; q < 4; ++q) {
                const uint32_t pv = pend[bi][bj][4 * gp + q];
                y[2 * q] = D::lo(pv);
                y[2 * q + 1] = D::hi(pv);
              }
              if (NOISE) {
                const uint32_t mrow = (uint32_t)(m0 + rbase + 16 * gp);
                pc = u32x4{(uint32_t)(nbase + 32 * bj), (mrow >> 4) * 2 + ((mrow >> 2) & 1), (uint32_t)te,
                           (uint32_t)nk.offset};
                philox_round(pc, k0, k1);
              }
            }
            if (NOISE && piece >= 1 && piece <= 4) { philox_round(pc, k0, k1); philox_round(pc, k0, k1); }
            if (NOISE && piece == 5) { philox_round(pc, k0, k1); box_muller16(pc.x, xi[0], xi[1]); }
            if (NOISE && piece == 6) box_muller16(pc.y, xi[2], xi[3]);
            if (NOISE && piece == 7) box_muller16(pc.z, xi[4], xi[5]);
            if (NOISE && piece == 8) box_muller16(pc.w, xi[6], xi[7]);
            if (piece == 8 && u > 0) resolve(u - 1);
            if (piece == 9) { row_consts(0); element_pair(0); }
            if (piece == 10) element_pair(2);
            if (piece == 11) { row_consts(1); element_pair(4); }
            if (piece == 12) element_pair(6);
            if (!CLAMP && piece == 13) totals(0);
            if (!CLAMP && piece == 14) totals(1);
            if (CLAMP && piece == 15) {
              // a running maximum in a vector register and ONE compare: compares whose results
              // go to scalar registers, and the scalar ORs that collect them, stall the wave
              float excess;
              if (IRMODE == AHL_IR_DYNAMIC) {
                excess = fabsf(y[0]) - Bv[0];
#pragma unroll
                for (int e = 1; e < 8; ++e) excess = fmaxf(excess, fabsf(y[e]) - Bv[e]);
              } else {
                excess = fmaxf(fmaxf(fmaxf(fabsf(y[0]), fabsf(y[1])), fmaxf(fabsf(y[2]), fabsf(y[3]))),
                               fmaxf(fmaxf(fabsf(y[4]), fabsf(y[5])), fmaxf(fabsf(y[6]), fabsf(y[7])))) - Bv[0];
              }
              over = excess > 0.0f;
            }
          }
          if (MMA && EPI) __builtin_amdgcn_sched_barrier(0);
        }
        if (EPI && CLAMP) {
#pragma unroll
          for (int e = 0; e < 8; ++e) { yp[e] = y[e]; Bp[e] = Bv[e]; }
          overp = over;
        }
        if (!MMA) __builtin_amdgcn_sched_barrier(0);
        if (MMA && ((u + 1) * KPU) % 4 == 0) {
          end_chunk();
          // every wave has read the constants of tile t - 1: their place takes those of tile t + 1
          if (u == NU - 1 && t + 1 < a.n_tiles) write_rowc(t + 1);
        }
      }
      resolve(NU - 1);
      if (MMA) plain_chunks();
    }
    if (EPI && CLAMP && a.keep != nullptr) {
      // the clamp-mask words of tile te: per 32-column block, 64 rows are 256 contiguous bytes
      uint32_t* plane = a.keep + (int64_t)te * clamp_plane_words(a.M, a.N);
#pragma unroll
      for (int hf = 0; hf < NBI / 2; ++hf) {
        const int64_t m = m0 + wm * 32 * NBI + hf * 64 + lane;
#pragma unroll
        for (int bj = 0; bj < 2; ++bj) {
          const int64_t nb0 = n0 + wn * 64 + bj * 32;
          if (m < a.M && nb0 < a.N) plane[clamp_word(m, nb0, a.M)] = cwords[hf][bj];
          cwords[hf][bj] = 0u;
        }
      }
    }
    if (MMA) {
      // the tile is complete: y = rd(acc), parked as bf16 pairs
#pragma unroll
      for (int i = 0; i < NBI; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int v = 0; v < 8; ++v) pend[i][j][v] = D::pack2(acc[i][j][2 * v], acc[i][j][2 * v + 1]);
    }
  };

  phase(flag<true>{}, flag<false>{}, 0);
  for (int t = 1; t < a.n_tiles; ++t) phase(flag<true>{}, flag<true>{}, t);
  phase(flag<false>{}, flag<true>{}, a.n_tiles);

  // most waves find the flag already set and skip the atomic
  if (a.clamp_flag != nullptr && __any(any_clamp != 0u) && lane == 0 &&
      __hip_atomic_load(a.clamp_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != a.flag_value)
    __hip_atomic_store(a.clamp_flag, a.flag_value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);

  // ---- store y = total (+ bias): transposed through LDS, 16-byte row-contiguous stores ----
  {
    constexpr int kOutStride = 128 * 2 + 16;
    __syncthreads();   // every wave is done with the operand buffers
    char* obase = lds + (wm * 32 * NBI + 4 * h) * kOutStride + (wn * 64 + r) * 2;
#pragma unroll
    for (int bj = 0; bj < 2; ++bj) {
      const bool add_bias = a.bias != nullptr;
      const float b = (add_bias && nbase + 32 * bj < a.N) ? D::load(a.bias, nbase + 32 * bj) : 0.0f;
#pragma unroll
      for (int bi = 0; bi < NBI; ++bi)
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
    const int vcol = tid & 15, vrow = tid >> 4;   // 16 vectors per row, NT / 16 rows per pass
    const int64_t n = n0 + vcol * 8;
#pragma unroll
    for (int j = 0; j < 4096 / NT; ++j) {
      const int row = vrow + (NT / 16) * j;
      const int64_t m = m0 + row;
      if (m < a.M && n < a.N)
        st16((uint16_t*)a.y + m * a.ldy + n, *(const u32x4*)(lds + row * kOutStride + vcol * 16));
    }
  }
}

// Grids of at least one block per CU, tiles of 256 / 512 columns, no split over K-tiles.
bool pipe_fwd_eligible(const FastFwdArgs& a, int ir_mode) {
  if (a.part != nullptr || ir_mode == AHL_IR_NONE) return false;
  // tiles of 256 or 512 columns, or any multiple of 64 from 576 up (the chunks beyond the eighth
  // are product only); an image operand only in the latter form
  const bool longer = a.tile > 512 && a.tile % 64 == 0;
  if (a.tile != 256 && a.tile != 512 && !longer) return false;
  if (a.conv.on && !longer) return false;
  // at least one block per CU, and no round of blocks that leaves more than a fifth of the CUs idle
  const int64_t nb = cdiv(a.M, 256) * cdiv(a.N, 128);
  if (nb < 256 || nb * 5 < cdiv(nb, 256) * 256 * 4) return false;
  // byte offsets inside a block's 256-row operand panel are 32-bit
  return a.ldx <= (1 << 21) && a.ldw <= (1 << 21);
}

template <class D, int IRMODE, bool NOISE, int QM, int CPT, bool EXTRA = false>
static void launch_pipe_one(const FastFwdArgs& a, hipStream_t s) {
  constexpr int NBI = 2;
  const dim3 block(1024 / NBI), grid((unsigned)(cdiv(a.M, 256) * cdiv(a.N, 128)));
  // a refusal shows at the launch that follows (check_launch reads the last error)
  (void)hipFuncSetAttribute((const void*)k_fwd_pipe<D, IRMODE, NOISE, QM, CPT, NBI, EXTRA>,
                      hipFuncAttributeMaxDynamicSharedMemorySize, kPLdsBytes);
  hipLaunchKernelGGL((k_fwd_pipe<D, IRMODE, NOISE, QM, CPT, NBI, EXTRA>), grid, block, kPLdsBytes, s, a);
}

// Launches the kernel if this combination is built; false otherwise (the caller falls back).
bool launch_pipe_fwd(int32_t dtype, const FastFwdArgs& a, int ir_mode, bool noise, int qm, hipStream_t s) {
  const int cpt = a.tile / 64;
#define AHL_PIPE(I, NZ, Q, C)                                                          \
  if (ir_mode == I && noise == NZ && qm == Q && cpt == C) {                            \
    if (dtype == AHL_F16) launch_pipe_one<F16, I, NZ, Q, C>(a, s);                     \
    else launch_pipe_one<BF16, I, NZ, Q, C>(a, s);                                     \
    return true;                                                                       \
  }
  AHL_PIPE(1, true, 2, 8)
  AHL_PIPE(1, false, 2, 8)
  AHL_PIPE(1, true, 0, 8)
  AHL_PIPE(1, false, 0, 8)
  AHL_PIPE(1, true, 2, 4)
  AHL_PIPE(1, false, 2, 4)
  AHL_PIPE(1, true, 0, 4)
  AHL_PIPE(1, false, 0, 4)
#undef AHL_PIPE
  // longer tiles: with the ADC (the configurations that are measured); others stay on k_fwd_fast
#define AHL_PIPE_LONG(NZ)                                                              \
  if (ir_mode == 1 && noise == NZ && qm == 2 && cpt > 8) {                             \
    if (dtype == AHL_F16) launch_pipe_one<F16, 1, NZ, 2, 8, true>(a, s);               \
    else launch_pipe_one<BF16, 1, NZ, 2, 8, true>(a, s);                               \
    return true;                                                                       \
  }
  AHL_PIPE_LONG(true)
  AHL_PIPE_LONG(false)
#undef AHL_PIPE_LONG
  return false;
}

}  // namespace ahl
