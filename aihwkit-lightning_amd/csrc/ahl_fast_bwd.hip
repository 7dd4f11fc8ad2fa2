// bf16 fast path of the backward products.
//
//   dX[m, k] = sum_n gy[m, n] * W_eff[n, k]        (MODE_DX)   gy = g, zeroed where tile t(k) was clamped
//   dW[n, k] = sum_m gy[m, n] * xq[m, k]           (MODE_DW)
//
// Neither product has both operands contiguous along the contraction index in memory: W_eff
// and xq (and g for dW) are stored with the contraction index as the ROW. Instead of
// materialising transposed copies, those operands are staged in LDS as they are ("k-major":
// [64 contraction rows][256 output columns]) and read with ds_read_b64_tr_b16, the CDNA4
// transposing LDS read: within each group of 16 lanes, lane r supplies the address of 4
// consecutive b16 of contraction row (r / 4), columns 4 * (r % 4) ..; lane i receives, for
// column i of the 16-column block, the 4 values of the 4 contraction rows -- exactly the
// "one column, consecutive k" shape of an MFMA operand register pair. Two such reads give the 8
// bf16 of one v_mfma_f32_32x32x16_bf16 operand.
//
// Block: 512 threads = 8 waves as 2 (rows) x 4 (columns); block tile 256 x 256, wave tile
// 128 x 64 (4 x 2 MFMA blocks, 128 fp32 accumulators), 64 contraction steps per chunk,
// double-buffered LDS (2 x 72 KB), one barrier per chunk, next chunk's global loads in flight
// during the MFMAs of the current one. The weight gradient also exists with a block tile of
// 256 x 192 (4 x 2 waves of 64 x 96), for K-tiles that 192 divides and 256 does not.
#include "ahl_host.h"
#include <type_traits>

namespace ahl {

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) s16x4* lds_s16x4_ptr;

static constexpr int kRowkStride = 144;               // k-contiguous operand: 128 B + 16 B pad
static constexpr int kKmajStride = 576;               // k-major operand: 512 B + 64 B pad
static constexpr int kOperandLds = 256 * kRowkStride; // == 64 * kKmajStride == 36864
static constexpr int kMaskLut = 4 * kOperandLds;      // LDS offset of the clamp-mask table
static constexpr int kBwdLds = kMaskLut + 256 * 16;   // 2 operands x 2 stages + the table

static constexpr int MODE_DX = 0;
static constexpr int MODE_DW = 1;

struct BwdArgs {
  const uint16_t* g; int64_t ldg;      // [M, N]
  const uint32_t* keep;                // clamp mask [T, ceil(N/32), M] or null
  const uint32_t* clamp_flag;          // null or the forward's flag
  uint32_t flag_token;                 // 0: "clamped" reads non-zero; else: reads this value
  const uint16_t* b; int64_t ldb;      // DX: W_eff [N, K]; DW: xq [M, K]
  const uint16_t* x; int64_t ldx;      // DX static range: the forward input [M, K]
  const uint16_t* ir;                  // DX static range: [T]
  uint16_t* out; int64_t ldo;          // DX: dx [M, K]; DW: dw [N, K]
  float* partial;                      // DX static range: [blocks][4]
  float* bias_partial;                 // DW: [K / 256][N] partial column sums of g, or null
  int64_t M, N, K;
  int32_t tile;                        // K-tile width (a multiple of the block width: 256, or 192)
  int32_t ir_static;                   // 0: no range gradient; 1 + AHL_IR_GRAD_* otherwise
  int32_t dense_tile;                  // DX: 0, or the true tile width when x and dx are dense
                                       // while W_eff is in the padded tile layout (K, tile then
                                       // describe the padded columns); a multiple of 8
  int32_t dense_base, dense_extra;     // DX: dense_base > 0: x and dx are dense with the split
                                       // (base, extra) of any widths; the epilogue then works
                                       // element by element instead of in 16-byte vectors
  int32_t slices;                      // the contraction (DW: rows m; DX: channels n) is cut
                                       // into this many slices, one block each; > 1 when the
                                       // output tiles alone are too few to fill the chip
  float* split;                        // slices > 1: fp32 partial results [slices][rows][K]
  ConvMap conv;                        // DW, conv.on: b is a padded channels-last image [pixels, C] and
                                       // output column c of tile t (at t * tile + c, c < conv_cols) is
                                       // (tap c / tile_base, channel t * tile_base + c % tile_base)
  int32_t conv_cols;                   // columns of a tile that hold data (taps x channels per tile)
  int64_t col_base;                    // DW on a column range of the weights: the range's first column
                                       // (the K-tile of a block is (col_base + its first column) / tile)
  int64_t mask_N;                      // output channels the clamp-mask planes were laid out for (N, also
                                       // when this launch covers a range of them)
};


// Everything after the product loop: the fp32 partial result of a slice, or the 256 x 256 result
// written through LDS with the input-range epilogue of the input gradient.
struct BwdPos {
  int64_t r0, c0, R, brow, bcol, nkb;
  int t, slice;
};

template <class D, int MODE, int BN, int TI, int TJ>
AHL_DEV void bwd_finish(const BwdArgs& a, const BwdPos& pos, f32x16 (&acc)[TI][TJ], char* lds,
                        float (*red)[3]) {
  constexpr int WN = BN / (32 * TJ);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;
  const int h = lane >> 5;
  const int64_t r0 = pos.r0, c0 = pos.c0, R = pos.R, brow = pos.brow, bcol = pos.bcol, nkb = pos.nkb;
  const int t = pos.t, slice = pos.slice;
  if (a.slices > 1) {
    // partial result of this slice, fp32, straight from the accumulators: for fixed (bi, bj, v)
    // the 32 lanes of a half wave write 128 contiguous bytes of one row
    float* sp = a.split + ((int64_t)slice * R) * a.K;
#pragma unroll
    for (int bi = 0; bi < TI; ++bi)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int64_t row = r0 + wm * (TI * 32) + bi * 32 + 8 * (v >> 2) + 4 * h + (v & 3);
        if (row >= R) continue;
#pragma unroll
        for (int bj = 0; bj < TJ; ++bj)
          sp[row * a.K + c0 + wn * (TJ * 32) + bj * 32 + (lane & 31)] = acc[bi][bj][v];
      }
    return;
  }
  // the narrower block only exists with a sliced contraction (the launcher sees to it)
  if constexpr (BN == 256) {

  // ---- epilogue: the 256 x 256 result goes through LDS (the operand buffers are free after
  // the loop's last barrier) so that global memory is touched in row-contiguous 16-byte vectors;
  // the forward input needed by the input-range gradient is fetched the same way ----
  float s_up = 0.0f, s_lo = 0.0f, cnt = 0.0f;
  const bool do_ir = MODE == MODE_DX && a.ir_static != 0;
  const float ir_t = do_ir ? D::load(a.ir, t) : 0.0f;
  constexpr int kOutStride = 256 * 2 + 16;
  const int vcol = tid & 31, vrow = tid >> 5;  // 16-byte vector column, row within a pass of 16
  // column of this thread's vectors in x / dx: the operand column itself, or, with dense x / dx
  // next to a padded W_eff, the same offset inside the dense tile (padding columns: no vector)
  int64_t ocol = c0 + vcol * 8;
  bool ovalid = true;
  if (MODE == MODE_DX && a.dense_tile > 0) {
    const int64_t in_tile = ocol - (int64_t)t * a.tile;
    ovalid = in_tile < a.dense_tile;
    ocol = ovalid ? (int64_t)t * a.dense_tile + in_tile : 0;
  }
  uint16_t* op = a.out + (r0 + vrow) * a.ldo + ocol;
  {
    char* obase = lds + (wm * 128 + 4 * h) * kOutStride + (wn * 64 + (lane & 31)) * 2;
#pragma unroll
    for (int bj = 0; bj < 2; ++bj)
#pragma unroll
      for (int bi = 0; bi < 4; ++bi)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int ro = bi * 32 + 8 * (v >> 2) + (v & 3);
          *(uint16_t*)(obase + ro * kOutStride + bj * 64) = D::to_elem(acc[bi][bj][v]);
        }
  }
  __syncthreads();
  if (MODE == MODE_DX && a.dense_base > 0) {
    // Dense x / dx whose tiles start at arbitrary columns. Per output row the block owns one
    // contiguous run of dense columns; it is written as 16-byte vectors from the first 16-byte
    // boundary of dx on (x has the same alignment: the launcher checks ldx == ldo and the base
    // pointers), the few elements before and after as single 2-byte accesses. Sub-dword
    // accesses for everything cost more than the padded copies they replace. A half wave
    // handles one row per pass; wave w owns rows 32 w .. 32 w + 31.
    const int32_t tw = a.dense_base + (t < a.dense_extra ? 1 : 0);
    const int64_t dstart = (int64_t)t * a.dense_base + (t < a.dense_extra ? t : a.dense_extra);
    const int64_t in0 = c0 - (int64_t)t * a.tile;  // block's first column inside the padded tile
    const int count = (int)(tw - in0 < 256 ? tw - in0 : 256);  // columns with data (may be <= 0)
    const int hw = lane >> 5, l32 = lane & 31;
    auto element = [&](float d, float x1) -> float {
      if (a.ir_static == 1 + AHL_IR_GRAD_LEARNED) {
        const bool up = x1 >= ir_t, lo = x1 <= -ir_t;
        if (up) s_up += fminf(d, 0.0f);
        if (lo) s_lo += fmaxf(d, 0.0f);
        if (up || lo) cnt += 1.0f;
      } else {
        if (x1 > ir_t) s_up += d;
        if (x1 < -ir_t) s_lo += d;
      }
      return fabsf(x1) > ir_t ? 0.0f : d;
    };
    for (int rr = 0; rr < 32; rr += 2) {
      const int row = wave * 32 + rr + hw;
      if (count <= 0 || r0 + row >= R) continue;
      const int64_t e0 = (r0 + row) * a.ldo + dstart + in0;   // first element of the run in dx (and x)
      const int head = (int)((8 - (e0 & 7)) & 7) < count ? (int)((8 - (e0 & 7)) & 7) : count;
      const int nv = (count - head) >> 3;
      const int tail0 = head + 8 * nv;                        // first column of the tail
      const char* lrow = lds + row * kOutStride;
      if (l32 < nv) {
        const int j = head + 8 * l32;
        float d[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) d[i] = D::load(lrow, j + i);
        if (do_ir) {
          float xv[8];
          D::unpack(ld16(a.x + e0 + j), xv);
#pragma unroll
          for (int i = 0; i < 8; ++i) d[i] = element(d[i], xv[i]);
        }
        st16(a.out + e0 + j, D::pack(d));
      }
      // up to 7 elements before the first and after the last vector
      const int j1 = l32 < head ? l32 : tail0 + (l32 - head);
      if (l32 < head + (count - tail0)) {
        float d = D::load(lrow, j1);
        if (do_ir) d = element(d, D::load(a.x, e0 + j1));
        a.out[e0 + j1] = D::to_elem(d);
      }
    }
  } else
#pragma unroll
  for (int half = 0; half < 2; ++half) {
    u32x4 xr[8];
    if (do_ir && ovalid) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int row = vrow + 16 * (8 * half + j);
        // rows beyond the matrix re-read the last row (the values are not used)
        const int64_t xrow = r0 + row < R ? r0 + row : R - 1;
        xr[j] = ld16(a.x + xrow * a.ldx + ocol);
      }
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int row = vrow + 16 * (8 * half + j);
      u32x4 d4 = *(const u32x4*)(lds + row * kOutStride + vcol * 16);
      if (r0 + row >= R || !ovalid) continue;
      if (do_ir) {
        float d[8], xv[8];
        D::unpack(d4, d);
        D::unpack(xr[j], xv);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          if (a.ir_static == 1 + AHL_IR_GRAD_LEARNED) {
            const bool up = xv[i] >= ir_t, lo = xv[i] <= -ir_t;
            if (up) s_up += fminf(d[i], 0.0f);
            if (lo) s_lo += fmaxf(d[i], 0.0f);
            if (up || lo) cnt += 1.0f;
          } else {
            if (xv[i] > ir_t) s_up += d[i];
            if (xv[i] < -ir_t) s_lo += d[i];
          }
          if (fabsf(xv[i]) > ir_t) d[i] = 0.0f;
        }
        d4 = D::pack(d);
      }
      st16(op + (int64_t)(16 * (8 * half + j)) * a.ldo, d4);
    }
  }
  if (do_ir) {
    s_up = wave_sum(s_up); s_lo = wave_sum(s_lo); cnt = wave_sum(cnt);
    if (lane == 0) { red[wave][0] = s_up; red[wave][1] = s_lo; red[wave][2] = cnt; }
    __syncthreads();
    if (tid == 0) {
      float u = 0.f, l = 0.f, c = 0.f;
      for (int w = 0; w < 8; ++w) { u += red[w][0]; l += red[w][1]; c += red[w][2]; }
      float* p = a.partial + (brow * nkb + bcol) * 4;
      p[0] = u; p[1] = l; p[2] = c; p[3] = 0.0f;
    }
  }
  }
}

// TAIL: the contraction length is not a multiple of 64 (its last chunk is loaded with
// predicates); the TAIL = false instantiation has no trace of that in its hot loop.
//
// BN: output columns per block. 256: 2 x 4 waves of 128 x 64. 192 (weight gradient with a sliced
// contraction only): 4 x 2 waves of 64 x 96, for K-tiles of 3 x 64 columns and their multiples that
// blocks of 256 would cover with a quarter of their columns empty.
template <class D, int MODE, bool TAIL, int BN>
__global__ __launch_bounds__(512, 2) void k_bwd_fast(BwdArgs a) {
  static_assert(BN == 256 || (BN == 192 && MODE == MODE_DW), "block widths: 256, or 192 for the weight gradient");
  constexpr int WN = BN == 256 ? 4 : 2, WM = 8 / WN;  // waves along the columns / the rows
  constexpr int TI = 256 / (32 * WM), TJ = BN / (32 * WN);  // 32 x 32 tiles of a wave
  extern __shared__ __attribute__((aligned(16))) char lds[];
  __shared__ float red[8][3];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;
  const int h = lane >> 5;

  // ---- block -> output tile. columns of the output are k (both modes), BN per block ----
  const int64_t nkb = a.K / BN;
  const int64_t nb = gridDim.x / a.slices;            // output tiles
  const int slice = (int)(blockIdx.x / nb);
  int64_t brow, bcol;
  block_to_tile(blockIdx.x % nb, nb, nb / nkb, nkb, 4, brow, bcol);
  const int64_t r0 = brow * 256;                     // DX: m0; DW: n0
  const int64_t c0 = bcol * BN;                      // k0
  const int t = (int)((c0 + (MODE == MODE_DW ? a.col_base : 0)) / a.tile);
  const int64_t R = MODE == MODE_DX ? a.M : a.N;      // output rows
  const int64_t L = MODE == MODE_DX ? a.N : a.M;      // contraction length
  const bool use_keep = a.keep != nullptr && clamp_flag_says_clamped(a.clamp_flag, a.flag_token);
  const uint32_t* plane = use_keep ? a.keep + (int64_t)t * clamp_plane_words(a.M, a.mask_N) : nullptr;

  f32x16 acc[TI][TJ];
#pragma unroll
  for (int i = 0; i < TI; ++i)
#pragma unroll
    for (int j = 0; j < TJ; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  // ---- staging maps ----
  // operand A (g): a thread owns 4 consecutive rows, so that the clamp-mask words of its four
  // vectors are 16 contiguous bytes (one load per chunk):
  //   DX (k-contiguous, rows m):      vector j -> row 4 (tid/8) + j,  16-byte column tid%8
  //   DW (k-major, contraction rows): vector j -> row 4 (tid/32) + j, 16-byte column tid%32
  // operand B (k-major): vector j -> contraction row tid/32 + 16 j, 16-byte column tid%32
  const int rk_row = tid >> 3, rk_cv = tid & 7;
  const int km_row = tid >> 5, km_cv = tid & 31;
  u32x4 rawA[4], rawB[4];
  u32x4 rawK = {0u, 0u, 0u, 0u};  // mask words of the vectors in rawA

  // Rows of the output tile that lie beyond the matrix are redirected to the last valid row:
  // they only feed accumulators that are never stored. No predicates in the hot loop.
  // Clamp mask: the 8 gradient values of one 16-byte vector are one byte of a mask word.
  const uint16_t* pa[4];
  const uint32_t* pk = nullptr;
  int psh = 0;
  const uint16_t* pb[4];
  if (MODE == MODE_DX) {
    int64_t mq = r0 + 4 * rk_row;          // first row of this thread's quad
    mq = mq < a.M ? mq : (a.M - 1) & ~(int64_t)3;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int64_t mr = mq + j < a.M ? mq + j : a.M - 1;
      pa[j] = a.g + mr * a.ldg + rk_cv * 8;                                  // + l0 (contraction n)
    }
    if (plane) pk = plane + clamp_word(mq, rk_cv * 8, a.M);                  // + (l0 / 32) * rows
    psh = 8 * (rk_cv & 3);
  } else {
    int64_t n = r0 + km_cv * 8;
    n = n < a.N ? n : a.N - 8;
#pragma unroll
    for (int j = 0; j < 4; ++j) pa[j] = a.g + (int64_t)(4 * km_row + j) * a.ldg + n;  // + l0 * ldg
    if (plane) pk = plane + clamp_word(4 * km_row, n, a.M);                           // + l0
    psh = 8 * (int)((n >> 3) & 3);
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) pb[j] = a.b + (int64_t)(km_row + 16 * j) * a.ldb + c0 + km_cv * 8;  // + l0 * ldb
  // weight gradient of a convolution read off the image: this thread's 8 columns are 8 channels of
  // one tap, i.e. of the image rows `tap offset` further on; columns in the padding between two
  // tiles contribute zeros
  // (a block narrower than the 256 columns the threads span leaves the last vectors of a row unused)
  bool b_valid = BN == 256 || km_cv * 8 < BN;
  if (MODE == MODE_DW && a.conv.on) {
    const int32_t in_tile = (int32_t)(c0 - (int64_t)t * a.tile) + km_cv * 8;
    b_valid = b_valid && in_tile < a.conv_cols;
    const int32_t tap = b_valid ? in_tile / a.conv.tile_base : 0;
    const int32_t ch = b_valid ? in_tile - tap * a.conv.tile_base : 0;
#pragma unroll
    for (int j = 0; j < 4; ++j)
      pb[j] = a.b + (int64_t)(km_row + 16 * j + conv_tap_rows(a.conv, tap)) * a.ldb + t * a.conv.tile_base + ch;
  }
  const int64_t a_step = MODE == MODE_DX ? 64 : 64 * a.ldg;
  const int64_t k_step = MODE == MODE_DX ? 2 * clamp_rows(a.M) : 64;   // 64 columns = 2 words; or 64 rows
  const int64_t b_step = 64 * a.ldb;
  // l_next: contraction offset of the chunk the next load() fetches. Only the last chunk of a
  // contraction length that is not a multiple of 64 takes the predicated path: contraction
  // indices beyond L read as zero (and are never touched in memory).
  int64_t l_next = 0;
  // this block's share of the contraction: chunks [ch0, ch0 + nchunks)
  const int chunks_all = (int)((L + 63) / 64);  // the last chunk may be partial
  const int per_slice = (chunks_all + a.slices - 1) / a.slices;
  const int ch0 = slice * per_slice;
  const int nchunks = chunks_all - ch0 < per_slice ? chunks_all - ch0 : per_slice;
  if (ch0 > 0) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      pa[j] += (int64_t)ch0 * a_step;
      pb[j] += (int64_t)ch0 * b_step;
    }
    if (pk) pk += (int64_t)ch0 * k_step;
    l_next = (int64_t)ch0 * 64;
  }
  const u32x4 zero4 = {0u, 0u, 0u, 0u};
  auto load = [&](bool masked) {
    if (!TAIL || l_next + 64 <= L) {
      if (masked) rawK = ld16(pk);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        rawA[j] = ld16(pa[j]);
        rawB[j] = ld16(pb[j]);
      }
    } else {
      // DX: contraction = columns of g (8 per vector, L a multiple of 8) and rows of W_eff;
      // DW: contraction = rows of g and of xq
      const bool a_col_ok = l_next + rk_cv * 8 < L;
      if (masked) {
        rawK = zero4;
        if (MODE == MODE_DW || a_col_ok) rawK = ld16(pk);
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const bool a_ok = MODE == MODE_DX ? a_col_ok : (l_next + 4 * km_row + j < L);
        const bool b_ok = l_next + km_row + 16 * j < L;
        rawA[j] = zero4;
        rawB[j] = zero4;
        if (a_ok) rawA[j] = ld16(pa[j]);
        if (b_ok) rawB[j] = ld16(pb[j]);
      }
    }
    if (MODE == MODE_DW && !b_valid) {
#pragma unroll
      for (int j = 0; j < 4; ++j) rawB[j] = zero4;
    }
    if (masked) pk += k_step;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      pa[j] += a_step;
      pb[j] += b_step;
    }
    if (TAIL) l_next += 64;
  };
  // The mask is applied here, after the MFMAs of the current chunk, so that nothing waits for
  // the loads that were issued before them.
  // DW: the bias gradient is the column sum of the unmasked g over all rows. Every block of a
  // row of blocks streams the same g; block kb of the nkb sums the chunks ch = kb (mod nkb), so
  // that the extra work is spread evenly, and a small kernel adds the nkb partial sums.
  float bsum[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  const int kb_idx = (int)bcol;
  auto stage = [&](char* sa, char* sb, bool masked, bool bias) {
    // clamps are rare in most layers: a chunk whose mask words are all zero for the wave skips the
    // table reads and the ANDs
    if (masked) masked = __any((rawK[0] | rawK[1] | rawK[2] | rawK[3]) != 0u);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (bias) {
        float e[8];
        D::unpack(rawA[j], e);
#pragma unroll
        for (int i = 0; i < 8; ++i) bsum[i] += e[i];
      }
      if (masked) {
        // the mask byte of the vector selects one of 256 precomputed 16-byte AND masks
        const u32x4 km = *(const u32x4*)(lds + kMaskLut + (((rawK[j] >> psh) & 0xffu) << 4));
        rawA[j] &= km;
      }
      if (MODE == MODE_DX) *(u32x4*)(sa + (4 * rk_row + j) * kRowkStride + rk_cv * 16) = rawA[j];
      else *(u32x4*)(sa + (4 * km_row + j) * kKmajStride + km_cv * 16) = rawA[j];
      *(u32x4*)(sb + (km_row + 16 * j) * kKmajStride + km_cv * 16) = rawB[j];
    }
  };

  // transposing read of one MFMA operand (8 bf16 of column `col` at contraction rows
  // 16 s + 8 h + 0..7) from a k-major LDS tile
  const int tr_r = lane & 15, tr_g = (lane >> 4) & 1;
  auto read_kmaj = [&](const char* base, int col0, int s) -> u32x4 {
    const char* p = base + (16 * s + 8 * h + (tr_r >> 2)) * kKmajStride +
                    (col0 + 16 * tr_g + 4 * (tr_r & 3)) * 2;
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)p);
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p + 4 * kKmajStride));
    const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
    u32x4 o = {l2.x, l2.y, h2.x, h2.y};
    return o;
  };

  if (plane) {  // uniform over the block
    if (tid < 256) {
      // entry e: halfword i is all ones unless bit i of e is set
      const u32x4 ones = {0xffffffffu, 0xffffffffu, 0xffffffffu, 0xffffffffu};
      *(u32x4*)(lds + kMaskLut + tid * 16) = clamp_apply8(ones, (uint32_t)tid);
    }
    __syncthreads();
  }
  auto main_loop = [&](auto masked_tag, auto bias_tag) {
    constexpr bool kMasked = decltype(masked_tag)::value;
    constexpr bool kBias = decltype(bias_tag)::value;
    load(kMasked);
    stage(lds, lds + kOperandLds, kMasked, kBias && ch0 % (int)nkb == kb_idx);
    __syncthreads();
    for (int ch = 0; ch < nchunks; ++ch) {
      const char* sa = lds + (ch & 1) * 2 * kOperandLds;
      const char* sb = sa + kOperandLds;
      if (ch + 1 < nchunks) load(kMasked);
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        u32x4 fa[TI], fb[TJ];
#pragma unroll
        for (int bi = 0; bi < TI; ++bi) {
          if (MODE == MODE_DX)
            fa[bi] = *(const u32x4*)(sa + (wm * (TI * 32) + bi * 32 + (lane & 31)) * kRowkStride + s * 32 + h * 16);
          else
            fa[bi] = read_kmaj(sa, wm * (TI * 32) + bi * 32, s);
        }
#pragma unroll
        for (int bj = 0; bj < TJ; ++bj) fb[bj] = read_kmaj(sb, wn * (TJ * 32) + bj * 32, s);
#pragma unroll
        for (int bi = 0; bi < TI; ++bi)
#pragma unroll
          for (int bj = 0; bj < TJ; ++bj) Mma16<D>::run(fa[bi], fb[bj], acc[bi][bj]);
      }
      if (ch + 1 < nchunks) {
        char* na = lds + ((ch + 1) & 1) * 2 * kOperandLds;
        stage(na, na + kOperandLds, kMasked, kBias && (ch0 + ch + 1) % (int)nkb == kb_idx);
      }
      __syncthreads();
    }
  };
  const bool do_bias = MODE == MODE_DW && a.bias_partial != nullptr;
  if (do_bias) {
    if (plane) main_loop(std::true_type{}, std::true_type{});
    else main_loop(std::false_type{}, std::true_type{});
    // 16 threads (contraction rows km_row + 16 j) hold partial sums of the same 8 columns
    float* bred = (float*)lds;  // [16][256]; the operand buffers are free after the last barrier
#pragma unroll
    for (int i = 0; i < 8; ++i) bred[km_row * 256 + km_cv * 8 + i] = bsum[i];
    __syncthreads();
    if (tid < 256 && r0 + tid < a.N) {
      float sum = 0.0f;
#pragma unroll
      for (int r = 0; r < 16; ++r) sum += bred[r * 256 + tid];
      a.bias_partial[((int64_t)slice * nkb + kb_idx) * a.N + r0 + tid] = sum;
    }
    __syncthreads();
  } else {
    if (plane) main_loop(std::true_type{}, std::false_type{});
    else main_loop(std::false_type{}, std::false_type{});
  }

  const BwdPos pos = {r0, c0, R, brow, bcol, nkb, t, slice};
  bwd_finish<D, MODE, BN, TI, TJ>(a, pos, acc, lds, red);
}

// dbias[n] = the sum of the partial rows, rounded to the dtype: 16 columns per block, 16 threads per column that
// each add every 16th row, combined in a fixed order (the partial rows can be hundreds when the
// weight gradient is sliced)
template <class D>
AHL_DEV void bias_final_block(int64_t block, const float* partial, int rows, int64_t N, uint16_t* dbias) {
  __shared__ float part[16][17];
  const int col = threadIdx.x & 15, grp = threadIdx.x >> 4;
  const int64_t n = block * 16 + col;
  float s = 0.0f;
  if (n < N)
    for (int i = grp; i < rows; i += 16) s += partial[(int64_t)i * N + n];
  part[grp][col] = s;
  __syncthreads();
  if (grp == 0 && n < N) {
    float sum = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; ++i) sum += part[i][col];
    dbias[n] = D::to_elem(sum);
  }
}

// out[r, c] = the sum over slices of split[s][r][c], slices added in order, rounded to the dtype.
// The first bias_blocks blocks (or none) finish the bias gradient in the same launch: a few long
// chains of additions that start first and run beside the sums.
template <class D>
__global__ __launch_bounds__(256) void k_split_reduce(const float* __restrict__ split, int slices,
                                                      int64_t R, int64_t K, uint16_t* __restrict__ out,
                                                      int64_t ldo, int64_t bias_blocks, const float* bias_partial,
                                                      int bias_rows, uint16_t* dbias) {
  if ((int64_t)blockIdx.x < bias_blocks) {   // uniform over the block
    bias_final_block<D>((int64_t)blockIdx.x, bias_partial, bias_rows, R, dbias);
    return;
  }
  const int64_t idx = (((int64_t)blockIdx.x - bias_blocks) * 256 + threadIdx.x) * 4;
  if (idx >= R * K) return;
  const int64_t r = idx / K, c = idx - r * K;  // K is a multiple of 256: the 4 share a row
  f32x4 sum = {0.f, 0.f, 0.f, 0.f};
  // four slices' loads in flight at a time; the sums stay in slice order
  for (int s = 0; s < slices; s += 4) {
    f32x4 part[4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
      part[u] = *(const f32x4*)(split + (int64_t)(s + u < slices ? s + u : slices - 1) * R * K + idx);
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (s + u < slices) sum += part[u];
  }
  u32x2 pk = {D::pack2(sum.x, sum.y), D::pack2(sum.z, sum.w)};
  *(u32x2*)(out + r * ldo + c) = pk;
}

// Sliced input gradient: sums the slices' partial results in order, rounds once, and applies the
// epilogue of the unsliced kernel (input-range mask and partial sums, column mapping onto a dense
// dx). One block: 16 rows x 256 columns; partial sums go to partial[(row block, column block)].
template <class D>
__global__ __launch_bounds__(512) void k_dx_split_reduce(BwdArgs a) {
  __shared__ float red[8][3];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t nkb = a.K / 256;
  const int64_t rb = blockIdx.x / nkb, bcol = blockIdx.x % nkb;
  const int64_t c0 = bcol * 256;
  const int t = (int)(c0 / a.tile);
  const int vcol = tid & 31, vrow = tid >> 5;
  const int64_t row = rb * 16 + vrow;
  int64_t ocol = c0 + vcol * 8;
  bool ovalid = true;
  if (a.dense_tile > 0) {
    const int64_t in_tile = ocol - (int64_t)t * a.tile;
    ovalid = in_tile < a.dense_tile;
    ocol = ovalid ? (int64_t)t * a.dense_tile + in_tile : 0;
  }
  const bool do_ir = a.ir_static != 0;
  const float ir_t = do_ir ? D::load(a.ir, t) : 0.0f;
  float s_up = 0.0f, s_lo = 0.0f, cnt = 0.0f;
  if (row < a.M && ovalid) {
    f32x4 lo4 = {0.f, 0.f, 0.f, 0.f}, hi4 = {0.f, 0.f, 0.f, 0.f};
    const float* sp = a.split + row * a.K + c0 + vcol * 8;
    // four slices' loads in flight at a time; the sums stay in slice order
    for (int sl = 0; sl < a.slices; sl += 4) {
      f32x4 l[4], h[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int64_t si = sl + u < a.slices ? sl + u : a.slices - 1;
        l[u] = *(const f32x4*)(sp + si * a.M * a.K);
        h[u] = *(const f32x4*)(sp + si * a.M * a.K + 4);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u)
        if (sl + u < a.slices) { lo4 += l[u]; hi4 += h[u]; }
    }
    float d[8] = {lo4.x, lo4.y, lo4.z, lo4.w, hi4.x, hi4.y, hi4.z, hi4.w};
#pragma unroll
    for (int i = 0; i < 8; i += 2) round2<D>(d[i], d[i + 1]);
    if (do_ir) {
      float xv[8];
      D::unpack(ld16(a.x + row * a.ldx + ocol), xv);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        if (a.ir_static == 1 + AHL_IR_GRAD_LEARNED) {
          const bool up = xv[i] >= ir_t, lo = xv[i] <= -ir_t;
          if (up) s_up += fminf(d[i], 0.0f);
          if (lo) s_lo += fmaxf(d[i], 0.0f);
          if (up || lo) cnt += 1.0f;
        } else {
          if (xv[i] > ir_t) s_up += d[i];
          if (xv[i] < -ir_t) s_lo += d[i];
        }
        if (fabsf(xv[i]) > ir_t) d[i] = 0.0f;
      }
    }
    st16(a.out + row * a.ldo + ocol, D::pack(d));
  }
  if (do_ir) {
    s_up = wave_sum(s_up); s_lo = wave_sum(s_lo); cnt = wave_sum(cnt);
    if (lane == 0) { red[wave][0] = s_up; red[wave][1] = s_lo; red[wave][2] = cnt; }
    __syncthreads();
    if (tid == 0) {
      float u = 0.f, l = 0.f, c = 0.f;
      for (int w = 0; w < 8; ++w) { u += red[w][0]; l += red[w][1]; c += red[w][2]; }
      float* p = a.partial + (rb * nkb + bcol) * 4;
      p[0] = u; p[1] = l; p[2] = c; p[3] = 0.0f;
    }
  }
}

template <class D>
__global__ __launch_bounds__(256) void k_bias_final(const float* partial, int rows, int64_t N,
                                                    uint16_t* dbias) {
  bias_final_block<D>((int64_t)blockIdx.x, partial, rows, N, dbias);
}

template <class D, int MODE, bool TAIL, int BN>
static void launch_bwd_one(dim3 grid, hipStream_t s, const BwdArgs& a) {
  // a refusal shows at the launch that follows (check_launch reads the last error)
  (void)hipFuncSetAttribute((const void*)k_bwd_fast<D, MODE, TAIL, BN>, hipFuncAttributeMaxDynamicSharedMemorySize, kBwdLds);
  hipLaunchKernelGGL((k_bwd_fast<D, MODE, TAIL, BN>), grid, dim3(512), kBwdLds, s, a);
}

template <int MODE, int BN = 256>
static void launch_bwd(int32_t dtype, bool tail, dim3 grid, hipStream_t s, const BwdArgs& a) {
  if (dtype == AHL_F16) {
    if (tail) launch_bwd_one<F16, MODE, true, BN>(grid, s, a);
    else launch_bwd_one<F16, MODE, false, BN>(grid, s, a);
  } else {
    if (tail) launch_bwd_one<BF16, MODE, true, BN>(grid, s, a);
    else launch_bwd_one<BF16, MODE, false, BN>(grid, s, a);
  }
}

// Whether the fast backward kernels can be used: a 16-bit dtype, equal K-tiles of a multiple of 256
// columns, output channels in whole 16-byte vectors. Any number of rows M: a contraction length
// that is not a multiple of 64 ends in one predicated chunk.
bool fast_bwd_eligible(int32_t dtype, const Tiling& tl, int64_t M, int64_t K, int64_t N) {
  if (dtype != AHL_BF16 && dtype != AHL_F16) return false;
  if (tl.extra != 0 || tl.base % 256 != 0) return false;
  return K % 256 == 0 && N % 8 == 0 && N >= 8 && M >= 1;
}

// Slices of the contraction for the input gradient: with few rows (a recurrent step, a small
// batch) the M x K / 65536 output tiles are a handful of blocks that each walk all N channels;
// the channels are cut until there are about 256 blocks, each with at least 4 chunks of 64.
int fast_dx_slices(int64_t M, int64_t K, int64_t N) {
  const int64_t tiles = cdiv(M, 256) * (K / 256);
  if (tiles >= 128) return 1;
  int64_t s = 256 / tiles;   // one block per CU: tiles * s blocks must fit one round of 256
  const int64_t chunks = cdiv(N, 64), most = chunks / 4;
  if (s > most) s = most;
  if (s <= 1) return 1;
  return (int)cdiv(chunks, cdiv(chunks, s));
}

// Rows of the input-range partial sums [rows][K / 256][4] that launch_fast_dx writes: one per
// 256 output rows, or one per 16 when the contraction is sliced.
int64_t fast_dx_row_blocks(int64_t M, int64_t K, int64_t N, bool element_mode) {
  return !element_mode && fast_dx_slices(M, K, N) > 1 ? cdiv(M, 16) : cdiv(M, 256);
}

static int64_t fast_dx_partial_bytes(int64_t M, int64_t K, int64_t N) {
  return (fast_dx_row_blocks(M, K, N, false) * (K / 256) * 16 + 255) / 256 * 256;
}

// Workspace of launch_fast_dx: [input-range partial sums | slices > 1: slices x M x K floats]
int64_t fast_dx_ws_bytes(int64_t M, int64_t K, int64_t N) {
  const int64_t slices = fast_dx_slices(M, K, N);
  return fast_dx_partial_bytes(M, K, N) + (slices > 1 ? slices * M * K * 4 : 0);
}

int launch_fast_dx(int32_t dtype, const void* g, int64_t ldg, const uint32_t* keep, const uint32_t* clamp_flag,
                   uint32_t flag_token, const void* w_eff, int64_t ldw, const void* x, int64_t ldx, const void* ir,
                   void* dx, int64_t lddx, void* ws, int64_t M, int64_t K, int64_t N,
                   const Tiling& tl, int ir_static, int32_t dense_tile, const Tiling* dense,
                   hipStream_t s) {
  BwdArgs a;
  float* partial = (float*)ws;
  // the element-wise epilogue for arbitrary dense splits is not part of the reduction kernel
  const int slices = dense ? 1 : fast_dx_slices(M, K, N);
  a.dense_tile = dense_tile;
  a.dense_base = dense ? dense->base : 0;
  a.dense_extra = dense ? dense->extra : 0;
  memset(&a.conv, 0, sizeof(a.conv)); a.conv_cols = 0; a.col_base = 0; a.mask_N = N;
  a.g = (const uint16_t*)g; a.ldg = ldg; a.keep = keep; a.clamp_flag = clamp_flag; a.flag_token = flag_token;
  a.b = (const uint16_t*)w_eff; a.ldb = ldw; a.x = (const uint16_t*)x; a.ldx = ldx;
  a.ir = (const uint16_t*)ir; a.out = (uint16_t*)dx; a.ldo = lddx; a.partial = partial; a.bias_partial = nullptr;
  a.M = M; a.N = N; a.K = K; a.tile = tl.base; a.ir_static = ir_static;
  a.slices = slices;
  a.split = slices > 1 ? (float*)((char*)ws + fast_dx_partial_bytes(M, K, N)) : nullptr;
  const int64_t nb = cdiv(M, 256) * (K / 256) * slices;
  if (nb > 0x7fffffff) return AHL_ERR_ARG;
  const dim3 grid((unsigned)nb), reduce_grid((unsigned)(cdiv(M, 16) * (K / 256)));
  launch_bwd<MODE_DX>(dtype, N % 64 != 0, grid, s, a);
  if (slices > 1) {
    if (dtype == AHL_F16) hipLaunchKernelGGL(k_dx_split_reduce<F16>, reduce_grid, dim3(512), 0, s, a);
    else hipLaunchKernelGGL(k_dx_split_reduce<BF16>, reduce_grid, dim3(512), 0, s, a);
  }
  return check_launch("ahl_linear_bwd_dx(fast)");
}

// Slices of the contraction for the weight gradient: N x K / 65536 output tiles are too few to
// fill 256 CUs when the layer is narrow (a convolution with many patches and few channels), so
// the rows m are cut until there are about 256 blocks, each with at least 8 chunks of 64 rows.
//
// A weight gradient whose 256 x 256 output tiles fill whole rounds of the 256 CUs plus a rest of at
// most half a round is cut in two launches: the tiles of the full rounds, and the rest with its
// contraction sliced so that it fills one round of shorter blocks (1.5 rounds paid as 2 become
// 1 + 0.5). The cut runs along the columns (a range of weight columns: xq and dw shifted, K-tiles
// counted from col_base) or along the rows (a range of output channels: g, dw, the bias gradient
// and the mask words shifted), whichever leaves whole rounds in front.
struct DwPart { int64_t n0, n, k0, k; int slices; };

static int dw_slices_for(int64_t tiles, int64_t M) {
  int64_t s = 256 / tiles;   // one block per CU: 257 blocks take as long as 512
  const int64_t chunks = cdiv(M, 64), most = chunks / 8;
  if (s > most) s = most;
  if (s <= 1) return 1;
  // every slice gets ceil(chunks / s) chunks; drop the slices that would be left empty
  return (int)cdiv(chunks, cdiv(chunks, s));
}

int fast_dw_slices(int64_t M, int64_t K, int64_t N) {
  const int64_t tiles = cdiv(N, 256) * (K / 256);
  return tiles >= 128 ? 1 : dw_slices_for(tiles, M);
}

// Columns per block for the weight gradient of an image operand whose K-tiles hold `tile_cols`
// columns: 192 when that divides the tile, 256 does not, and the 192-wide blocks are few enough
// for a sliced contraction (the narrower block has no unsliced epilogue); else 256, with the tile
// padded to a multiple of it.
int fast_dw_image_block(int64_t M, int64_t tile_cols, int32_t n_tiles, int64_t N) {
  if (tile_cols % 256 == 0 || tile_cols % 192 != 0) return 256;
  const int64_t tiles = cdiv(N, 256) * (tile_cols / 192) * n_tiles;
  return tiles < 128 && dw_slices_for(tiles, M) > 1 ? 192 : 256;
}

static int dw_parts(int64_t M, int64_t K, int64_t N, bool whole_only, int bw, DwPart parts[2]) {
  const int64_t nrows = cdiv(N, 256), nkb = K / 256, tiles = nrows * nkb;
  if (bw != 256) {  // the narrower blocks of an image operand: one launch, sliced
    parts[0] = {0, N, 0, K, dw_slices_for(nrows * (K / bw), M)};
    return 1;
  }
  parts[0] = {0, N, 0, K, fast_dw_slices(M, K, N)};
  if (whole_only || tiles <= 256 || tiles % 256 == 0) return 1;
  for (int64_t kb1 = nkb - 1; kb1 >= 1; --kb1) {
    const int64_t rest = nrows * (nkb - kb1);
    if ((nrows * kb1) % 256 != 0 || rest > 128) continue;
    const int sl = dw_slices_for(rest, M);
    if (sl < 2) break;
    parts[0] = {0, N, 0, kb1 * 256, 1};
    parts[1] = {0, N, kb1 * 256, K - kb1 * 256, sl};
    return 2;
  }
  if (N % 256 != 0) return 1;
  for (int64_t r1 = nrows - 1; r1 >= 1; --r1) {
    const int64_t rest = (nrows - r1) * nkb;
    if ((r1 * nkb) % 256 != 0 || rest > 128) continue;
    const int sl = dw_slices_for(rest, M);
    if (sl < 2) break;
    parts[0] = {0, r1 * 256, 0, K, 1};
    parts[1] = {r1 * 256, N - r1 * 256, 0, K, sl};
    return 2;
  }
  return 1;
}

static int64_t dw_part_bias_bytes(const DwPart& p, int bw) { return ((int64_t)p.slices * (p.k / bw) * p.n * 4 + 255) / 256 * 256; }
static int64_t dw_part_bytes(const DwPart& p, int bw) {
  return dw_part_bias_bytes(p, bw) + (p.slices > 1 ? ((int64_t)p.slices * p.n * p.k * 4 + 255) / 256 * 256 : 0);
}

// Workspace of launch_fast_dw, per launch: [partial bias sums: slices x k/256 x n floats |
// slices > 1: partial results slices x n x k floats]
int64_t fast_dw_ws_bytes(int64_t M, int64_t K, int64_t N, int block_cols) {
  DwPart parts[2];
  const int np = dw_parts(M, K, N, false, block_cols, parts);
  int64_t bytes = 0;
  for (int i = 0; i < np; ++i) bytes += dw_part_bytes(parts[i], block_cols);
  return bytes;
}

int launch_fast_dw(int32_t dtype, const void* g, int64_t ldg, const uint32_t* keep, const uint32_t* clamp_flag,
                   uint32_t flag_token, const void* xq, int64_t ldxq, void* dw, int64_t lddw, void* dbias,
                   void* ws, int64_t M, int64_t K, int64_t N, const Tiling& tl,
                   hipStream_t s, const ConvMap* conv, int32_t conv_cols, int block_cols) {
  DwPart parts[2];
  const int bw = conv != nullptr ? block_cols : 256;
  if (bw != 256 && (bw != 192 || K % 192 != 0 || tl.base % 192 != 0)) return AHL_ERR_ARG;
  // an image operand maps its columns itself: one launch
  const int np = dw_parts(M, K, N, conv != nullptr, bw, parts);
  if (bw != 256 && parts[0].slices < 2) return AHL_ERR_ARG;
  char* wsp = (char*)ws;
  for (int i = 0; i < np; ++i) {
    const DwPart& p = parts[i];
    // the bias gradient comes from the launch(es) that cover column 0 of the weights
    void* dbias_p = (dbias && p.k0 == 0) ? (char*)dbias + p.n0 * 2 : nullptr;
    BwdArgs a;
    memset(&a.conv, 0, sizeof(a.conv)); a.conv_cols = 0;
    if (conv != nullptr) { a.conv = *conv; a.conv_cols = conv_cols; }
    float* bias_partial = (float*)wsp;
    a.g = (const uint16_t*)g + p.n0; a.ldg = ldg;
    // mask words of channel n lie at word column n / 32 of a plane laid out for all N channels
    a.keep = keep ? keep + (p.n0 >> 5) * ((M + 63) & ~(int64_t)63) : nullptr;
    a.clamp_flag = clamp_flag; a.flag_token = flag_token;
    a.b = (const uint16_t*)xq + p.k0; a.ldb = ldxq; a.x = nullptr; a.ldx = 0; a.ir = nullptr;
    a.out = (uint16_t*)dw + p.n0 * lddw + p.k0; a.ldo = lddw; a.partial = nullptr;
    a.bias_partial = dbias_p ? bias_partial : nullptr;
    a.M = M; a.N = p.n; a.K = p.k; a.tile = tl.base; a.ir_static = 0; a.dense_tile = 0;
    a.dense_base = 0; a.dense_extra = 0;
    a.col_base = p.k0; a.mask_N = N;
    a.slices = p.slices;
    a.split = p.slices > 1 ? (float*)(wsp + dw_part_bias_bytes(p, bw)) : nullptr;
    const int64_t nb = cdiv(p.n, 256) * (p.k / bw) * p.slices;
    if (nb > 0x7fffffff) return AHL_ERR_ARG;
    if (bw == 192) launch_bwd<MODE_DW, 192>(dtype, M % 64 != 0, dim3((unsigned)nb), s, a);
    else launch_bwd<MODE_DW>(dtype, M % 64 != 0, dim3((unsigned)nb), s, a);
    // a sliced launch sums its slices and finishes the bias gradient in one more launch
    const int64_t sum_blocks = cdiv(p.n * p.k, 1024), bias_blocks = dbias_p ? cdiv(p.n, 16) : 0;
    const dim3 reduce_grid((unsigned)(sum_blocks + bias_blocks)), bias_grid((unsigned)cdiv(p.n, 16));
    const int bias_rows = (int)(p.k / bw) * p.slices;
    if (dtype == AHL_F16) {
      if (p.slices > 1)
        hipLaunchKernelGGL(k_split_reduce<F16>, reduce_grid, dim3(256), 0, s, (const float*)a.split, p.slices, p.n, p.k,
                           a.out, lddw, bias_blocks, (const float*)bias_partial, bias_rows, (uint16_t*)dbias_p);
      else if (dbias_p)
        hipLaunchKernelGGL(k_bias_final<F16>, bias_grid, dim3(256), 0, s, (const float*)bias_partial, bias_rows, p.n,
                           (uint16_t*)dbias_p);
    } else {
      if (p.slices > 1)
        hipLaunchKernelGGL(k_split_reduce<BF16>, reduce_grid, dim3(256), 0, s, (const float*)a.split, p.slices, p.n, p.k,
                           a.out, lddw, bias_blocks, (const float*)bias_partial, bias_rows, (uint16_t*)dbias_p);
      else if (dbias_p)
        hipLaunchKernelGGL(k_bias_final<BF16>, bias_grid, dim3(256), 0, s, (const float*)bias_partial, bias_rows, p.n,
                           (uint16_t*)dbias_p);
    }
    wsp += dw_part_bytes(p, bw);
  }
  return check_launch("ahl_linear_bwd_dw(fast)");
}

}  // namespace ahl
