// Convolutions without the patch matrix (16-bit dtypes, stride 1, dilation 1, K-tiles that hold
// whole channels in multiples of 64): the three products read the image itself.
//
// The reference unfolds the input into a [B * L, C * kvol] patch matrix and runs the tiled analog
// operator on it (nn/modules/conv.py:310-360). Here the input is kept as ONE zero-padded,
// channels-last matrix [padded pixels, C] (quantised per K-tile on the way in: a tile holds whole
// channels, so the DAC of a pixel does not depend on the patch it is seen through), the outputs are
// numbered on the same padded pixel grid, and a kernel offset is a constant row offset (ConvMap in
// ahl_device.h). The matrix kernels are the linear layer's own:
//   forward          k_fwd_fast with the A operand's chunk offsets taken from the ConvMap;
//   weight gradient  k_bwd_fast<DW> with the B operand's columns mapped onto (tap, channel);
//   input gradient   k_conv_dx_pipe / k_conv_dx below: dimg[q, c] = sum over taps and output channels of
//                    gy[q - offset(tap), n] * w[n, c, tap], gy = g without the outputs that tile
//                    t(c) clamped. Each tap's partial is rounded to the dtype (it is the patch
//                    gradient entry the reference's product produces), then summed in fp32 in
//                    ascending tap order and rounded once -- the arithmetic of the fold of the
//                    patch path (ahl_col2im) -- and the input-range gradient's sums are taken
//                    from the per-tap values, as the reference takes them from the patch entries.
// Around them: layout kernels between [B, C, *spatial] and the padded pixel rows.
//
// Row convention of every pixel-row buffer here: `lead` rows of zeros, the P padded pixels, then
// at least lead + 256 more rows of zeros (ahl_conv_direct_rows gives the numbers); real row p is
// stored at row p + lead. Rows that are no valid output (the receptive field would leave the
// padded image) hold zeros in the gradient and are dropped from the output.
#include "ahl_host.h"
#include "ahl_fwd_common.h"
#include "ahl_lds_direct.h"
#include <type_traits>

namespace ahl {

// declared in ahl_fast.hip / ahl_fast_bwd.hip
int launch_fast_fwd(const void* xq, int64_t ldxq, const void* w_eff, int64_t ldw, const void* bias,
                    void* y, int64_t ldy, uint32_t* keep, uint32_t* clamp_flag, const void* ir,
                    const void* wmax, const float* tile_max, int64_t M, int64_t K, int64_t N,
                    const Tiling& tl, const AhlLinearCfg* cfg, void* ws, hipStream_t s,
                    const ConvMap* conv);
int launch_fast_dw(int32_t dtype, const void* g, int64_t ldg, const uint32_t* keep, const uint32_t* clamp_flag,
                   uint32_t flag_token, const void* xq, int64_t ldxq, void* dw, int64_t lddw, void* dbias,
                   void* ws, int64_t M, int64_t K, int64_t N, const Tiling& tl,
                   hipStream_t s, const ConvMap* conv, int32_t conv_cols, int block_cols);
int64_t fast_dw_ws_bytes(int64_t M, int64_t K, int64_t N, int block_cols);
int fast_dw_image_block(int64_t M, int64_t tile_cols, int32_t n_tiles, int64_t N);

struct DirectGeom {
  int32_t B, C;
  int32_t in[3], ker[3], pad[3], pin[3], out[3];  // input, kernel, padding, padded input, output extents
  int32_t kvol;
  int32_t lead;      // the largest tap offset in rows
  int64_t P;         // padded pixels = rows of the output grid
  int64_t rows;      // rows of a pixel-row buffer: lead + P + lead + 256
};

static bool make_direct(const AhlConvGeom* a, DirectGeom* g) {
  if (a == nullptr || a->batch <= 0 || a->channels <= 0) return false;
  g->B = a->batch;
  g->C = a->channels;
  int64_t P = a->batch;
  g->kvol = 1;
  for (int d = 0; d < 3; ++d) {
    if (a->in_size[d] <= 0 || a->kernel[d] <= 0 || a->stride[d] != 1 || a->dilation[d] != 1 || a->padding[d] < 0)
      return false;
    g->in[d] = a->in_size[d]; g->ker[d] = a->kernel[d]; g->pad[d] = a->padding[d];
    g->pin[d] = a->in_size[d] + 2 * a->padding[d];
    g->out[d] = g->pin[d] - a->kernel[d] + 1;
    if (g->out[d] <= 0) return false;
    g->kvol *= a->kernel[d];
    P *= g->pin[d];
  }
  const int64_t lead = ((int64_t)(g->ker[0] - 1) * g->pin[1] + (g->ker[1] - 1)) * g->pin[2] + (g->ker[2] - 1);
  // byte offsets of a tap inside an operand (lead rows x at most 16384 columns x 2 bytes) are 32-bit
  if (P > 0x3fffffff || lead > 0x7fff || a->channels > 16384) return false;
  g->lead = (int32_t)lead;
  g->P = P;
  g->rows = P + 2 * lead + 256;   // a block of 256 rows may start at the last pixel
  return true;
}

static ConvMap make_map(const DirectGeom& g, int sign, int32_t cg, int32_t tile_base, int64_t alloc_rows) {
  ConvMap m;
  m.on = 1; m.sign = sign; m.lead = g.lead; m.cg = cg; m.tile_base = tile_base;
  m.kh = g.ker[1]; m.kw = g.ker[2]; m.hp = g.pin[1]; m.wp = g.pin[2];
  m.alloc_rows = alloc_rows;
  return m;
}

// Spatial index s of a [d0, d1, d2] box -> row on the padded pixel grid of image b, the box's
// origin at padded coordinates o0, o1, o2.
struct RowMap {
  int32_t d0, d1, d2;     // extents of the box
  int32_t o0, o1, o2;     // origin of the box on the padded grid
  int32_t p0, p1, p2;     // padded extents
};
AHL_DEV int64_t row_of(const RowMap& m, int32_t b, int32_t s) {
  const int32_t w = s % m.d2, r = s / m.d2;
  const int32_t h = r % m.d1, d = r / m.d1;
  return (((int64_t)b * m.p0 + d + m.o0) * m.p1 + h + m.o1) * m.p2 + w + m.o2;
}
// The inverse: pixel p of the padded grid -> index into a [B, nch, S] tensor's (b, s), or -1 when
// p lies outside the box (padding, outputs that do not exist).
AHL_DEV bool box_of(const RowMap& m, int64_t p64, int32_t& b, int32_t& s, int32_t (&pc)[3]) {
  const uint32_t p = (uint32_t)p64;   // pixels are fewer than 2^30: 32-bit divisions
  const uint32_t q1 = p / (uint32_t)m.p2;
  const int32_t w = (int32_t)(p - q1 * (uint32_t)m.p2) - m.o2;
  const uint32_t q0 = q1 / (uint32_t)m.p1;
  const int32_t h = (int32_t)(q1 - q0 * (uint32_t)m.p1) - m.o1;
  const uint32_t qb = q0 / (uint32_t)m.p0;
  const int32_t d = (int32_t)(q0 - qb * (uint32_t)m.p0) - m.o0;
  b = (int32_t)qb;
  s = (d * m.d1 + h) * m.d2 + w;
  pc[0] = d + m.o0; pc[1] = h + m.o1; pc[2] = w + m.o2;   // coordinates on the padded grid
  return w >= 0 && w < m.d2 && h >= 0 && h < m.d1 && d >= 0 && d < m.d0;
}

static constexpr int kTileWords = 33;   // LDS row stride of the 64 x 64 transposing tiles, in dwords

// ---------------------------------------------------------------------------------------------
// [B, nch, S] -> pixel rows: dst[lead + row(b, s), c] = f(src[b, c, s]), f = the DAC of channel
// c's K-tile (clamp to the tile's range, quantise) or the identity; every other row of dst (the
// lead rows, the padding pixels, the rows behind the last pixel) is written as zeros, so dst
// need not be cleared beforehand. One block: 64 consecutive rows of dst x 64 channels, turned in
// LDS; global memory is read along s (consecutive rows of dst are consecutive s up to the padding)
// and written along c, 16 bytes at a time. ct is a multiple of 64: a block's channels share a K-tile.
// With `flags` set (static range, a backward pass will follow) the kernel also leaves what the
// input gradient needs to know about x, one byte per element in the layout of dst:
//   bit 0: x >= ir, bit 1: x <= -ir (the entries whose gradient goes to the range, reference
//   torch_utils/torch_linear.py:92-106), bit 2: |x| > ir (the straight-through mask, :44-54),
// and per block the number of PATCH ENTRIES with bit 0 or 1 (for the decay switch, :98-103): a
// pixel is seen by one patch for every tap under which some valid output lies, so it counts that
// many times.
struct TapSpan { int32_t k0, k1, k2, out0, out1, out2; };

template <class D, int IRMODE>
__global__ __launch_bounds__(256) void k_conv_scatter(const uint16_t* __restrict__ src, int32_t nch, int32_t S,
                                                      RowMap map, int32_t lead, int64_t P, int64_t rows,
                                                      uint16_t* __restrict__ dst,
                                                      uint8_t* __restrict__ flags, uint32_t* __restrict__ count,
                                                      TapSpan taps, const void* __restrict__ ir,
                                                      int32_t ct, float inp_res, int32_t skip_rounding) {
  __shared__ uint32_t tile[64 * kTileWords];
  __shared__ uint32_t ftile[64 * 17];   // flags, one byte per element, 68 bytes per row
  __shared__ uint32_t wave_count[4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t r0 = (int64_t)blockIdx.x * 64;
  const int32_t c0 = blockIdx.y * 64;
  int32_t b = 0, sp = 0;
  int32_t pc[3] = {0, 0, 0};
  const int64_t pix = r0 + lane - lead;
  const bool inside = pix >= 0 && pix < P && box_of(map, pix, b, sp, pc);
  Dac dac = {0.0f, 1.0f, 1.0f, 1.0f};
  float irv = 0.0f;
  if (IRMODE == AHL_IR_STATIC) {
    irv = D::load(ir, c0 / ct);
    dac = make_dac<D>(irv, inp_res);
  }
  // every load is issued (lanes with nothing to read load the tensor's first element) and the
  // values are selected afterwards: a load behind a branch would be waited for before the next
  const uint16_t* col = src + ((int64_t)b * nch + c0 + wave * 16) * S + sp;
  float v[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const bool ok = inside && c0 + wave * 16 + i < nch;
    v[i] = D::load(ok ? col + (int64_t)i * S : src, 0);
  }
#pragma unroll
  for (int i = 0; i < 16; ++i) v[i] = (inside && c0 + wave * 16 + i < nch) ? v[i] : 0.0f;
  uint32_t clipped = 0;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int32_t cl = wave * 16 + i;
    float q = v[i];
    if (IRMODE == AHL_IR_STATIC)
      q = inp_res > 0.0f ? dac_apply<D, true, true>(v[i], dac, skip_rounding != 0)
                         : dac_apply<D, true, false>(v[i], dac, false);
    ((uint16_t*)tile)[lane * (2 * kTileWords) + cl] = D::to_elem(q);
    if (IRMODE == AHL_IR_STATIC && flags != nullptr) {
      const bool edge = v[i] >= irv || v[i] <= -irv;
      const uint32_t f = (v[i] >= irv ? 1u : 0u) | (v[i] <= -irv ? 2u : 0u) | (fabsf(v[i]) > irv ? 4u : 0u);
      ((uint8_t*)ftile)[lane * 68 + cl] = (uint8_t)f;
      clipped += edge ? 1u : 0u;
    }
  }
  if (IRMODE == AHL_IR_STATIC && flags != nullptr) {
    // patches that see this lane's pixel: per dimension, the taps k with 0 <= coordinate - k < outputs
    auto span = [](int32_t c, int32_t k, int32_t out) {
      const int32_t lo = c - (out - 1) > 0 ? c - (out - 1) : 0, hi = c < k - 1 ? c : k - 1;
      return hi >= lo ? hi - lo + 1 : 0;
    };
    uint32_t cnt = inside ? clipped * (uint32_t)(span(pc[0], taps.k0, taps.out0) * span(pc[1], taps.k1, taps.out1) *
                                                 span(pc[2], taps.k2, taps.out2)) : 0u;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) cnt += __shfl_xor(cnt, o, 64);
    if (lane == 0) wave_count[wave] = cnt;
  }
  __syncthreads();
  if (IRMODE == AHL_IR_STATIC && flags != nullptr && tid == 0)
    count[(int64_t)blockIdx.x * gridDim.y + blockIdx.y] = (wave_count[0] + wave_count[1]) + (wave_count[2] + wave_count[3]);
  const int vec = tid & 7;
  if (c0 + vec * 8 >= nch) return;
#pragma unroll
  for (int half = 0; half < 2; ++half) {
    const int r = (tid >> 3) + 32 * half;
    const int64_t row = r0 + r;
    if (row >= rows) continue;
    const uint32_t* t0 = tile + r * kTileWords + vec * 4;
    const u32x4 v0 = {t0[0], t0[1], t0[2], t0[3]};
    st16(dst + row * nch + c0 + vec * 8, v0);
    if (IRMODE == AHL_IR_STATIC && flags != nullptr) {
      const uint32_t* f0 = ftile + r * 17 + vec * 2;
      const u32x2 fv = {f0[0], f0[1]};
      *(u32x2*)(flags + row * nch + c0 + vec * 8) = fv;
    }
  }
}

// ---------------------------------------------------------------------------------------------
// pixel rows -> [B, nch, S]: dst[b, c, s] = src[lead + row(b, s), c].
template <class D>
__global__ __launch_bounds__(256) void k_conv_gather(const uint16_t* __restrict__ src, int32_t nch, int32_t S,
                                                     RowMap map, int32_t lead, uint16_t* __restrict__ dst) {
  __shared__ uint32_t tile[64 * kTileWords];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int32_t s0 = blockIdx.x * 64, c0 = blockIdx.y * 64, b = blockIdx.z;
  const int vec = tid & 7;
#pragma unroll
  for (int half = 0; half < 2; ++half) {
    const int r = (tid >> 3) + 32 * half;
    u32x4 v = {0u, 0u, 0u, 0u};
    if (s0 + r < S && c0 + vec * 8 < nch)
      v = ld16(src + (lead + row_of(map, b, s0 + r)) * nch + c0 + vec * 8);
    uint32_t* t0 = tile + r * kTileWords + vec * 4;
    t0[0] = v.x; t0[1] = v.y; t0[2] = v.z; t0[3] = v.w;
  }
  __syncthreads();
  const int32_t s = s0 + lane;
  if (s >= S) return;
  const int64_t at0 = ((int64_t)b * nch + c0 + wave * 16) * S + s;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int32_t cl = wave * 16 + i;
    if (c0 + cl >= nch) continue;
    D::store(dst, at0 + (int64_t)i * S, D::load(tile, lane * (2 * kTileWords) + cl));
  }
}

// ---------------------------------------------------------------------------------------------
// Weight layouts. w is the layer's [N, C * kvol] matrix (channel-major, taps inside: the
// reference's weight.view(out, -1)); ct channels per K-tile.
//   mode 0: -> [N, C * kvol] with a tile's columns reordered (tap, channel): the forward's B operand
//   mode 1: the inverse, from a matrix whose tiles start every `stride` columns (the weight
//           gradient as the kernel leaves it) to the layer's order, dense
//   mode 2: -> [C, kvol * N], row c: (tap, n) -> w[n, c, tap]: the input gradient's B operand
template <class E>
__global__ __launch_bounds__(256) void k_conv_weights(const E* __restrict__ src, int64_t ld_src, int32_t N,
                                                      int32_t C, int32_t kvol, int32_t ct, int32_t stride,
                                                      int mode, E* __restrict__ dst, int64_t ld_dst,
                                                      E* __restrict__ dst_dx, int64_t ld_dx) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t K = (int64_t)C * kvol;
  if (idx >= (int64_t)N * K) return;
  if (dst_dx != nullptr) {   // mode 2, alone or (mode 0) beside the forward's layout
    const int32_t c = (int32_t)(idx / ((int64_t)kvol * N));
    const int32_t rem = (int32_t)(idx - (int64_t)c * kvol * N);
    const int32_t tap = rem / N, n = rem - tap * N;
    dst_dx[(int64_t)c * ld_dx + rem] = src[(int64_t)n * ld_src + (int64_t)c * kvol + tap];
    if (mode == 2) return;
  }
  const int32_t n = (int32_t)(idx / K);
  const int32_t k = (int32_t)(idx - (int64_t)n * K);   // position in the layer's order
  const int32_t c = k / kvol, tap = k - c * kvol;
  const int32_t t = c / ct, cl = c - t * ct;
  const int64_t tiled = (int64_t)t * (mode == 0 ? ct * kvol : stride) + (int64_t)tap * ct + cl;
  if (mode == 0) dst[(int64_t)n * ld_dst + tiled] = src[(int64_t)n * ld_src + k];
  else dst[(int64_t)n * ld_dst + k] = src[(int64_t)n * ld_src + tiled];
}

// ---------------------------------------------------------------------------------------------
// Input gradient on the padded pixel grid (see the file header). Block: 256 threads = 4 waves that
// each own a 64 x 64 output tile: 256 pixels x 64 channels when a K-tile holds 64 channels, else
// 128 x 128 (all columns of a block lie in one K-tile: the clamp mask applied to g is that
// tile's). The contraction runs tap by tap over the output channels in 64-wide chunks, operands
// staged global -> registers -> LDS like k_fwd_fast, the mask applied to g in the registers.
struct ConvDxArgs {
  const uint16_t* g; int64_t ldg;      // gradient rows [rows, N] (lead rows of zeros in front)
  const uint32_t* keep;                // clamp mask [T, ceil(N/32), rows64(P)] or null
  const uint32_t* clamp_flag; uint32_t flag_token;
  const uint16_t* w; int64_t ldw;      // [C, kvol * N] (k_conv_weights mode 2)
  const uint8_t* flags;                // per element of the padded image rows [rows, C]: bit 0 x >= ir,
                                       // bit 1 x <= -ir, bit 2 |x| > ir (k_conv_scatter); or null
  uint16_t* out; int64_t ldo;          // dimg [P, C]
  float* partial;                      // [row blocks][column blocks][2] (with flags)
  int64_t P, rows;
  int32_t N, C, ct, kvol;
  ConvMap conv;                        // sign -1
};

// v with the elements zeroed whose bit in `bits` is set (bit i: element i), four operations per
// pair of elements: the two bits sign-extended, merged into a halfword mask, applied.
AHL_DEV u32x4 zero_where_set8(const u32x4& v, uint32_t bits) {
  const int32_t keep = (int32_t)~bits;
  auto pair = [&](uint32_t x, int i) -> uint32_t {
    const uint32_t lo = (uint32_t)__builtin_amdgcn_sbfe(keep, 2 * i, 1);       // all ones: keep the even element
    const uint32_t hi = (uint32_t)__builtin_amdgcn_sbfe(keep, 2 * i + 1, 1);
    return x & ((lo & 0xffffu) | (hi & 0xffff0000u));                          // and_or + and
  };
  u32x4 o = {pair(v.x, 0), pair(v.y, 1), pair(v.z, 2), pair(v.w, 3)};
  return o;
}

template <class D, int WM, int WN>
__global__ __launch_bounds__(256, 2) void k_conv_dx(ConvDxArgs a) {
  constexpr int BM = 64 * WM, BN = 64 * WN;   // block tile; every wave owns 64 x 64 of it
  constexpr int NA = 2 * WM, NB = 2 * WN;     // 16-byte vectors per thread and chunk
  constexpr int kStride = 144;                // LDS row: 128 bytes + 16 pad
  extern __shared__ __attribute__((aligned(16))) char lds[];
  __shared__ float red[4][2];
  char* ldsA = lds;
  char* ldsB = lds + BM * kStride;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN, h = lane >> 5;
  const int row0 = tid >> 3, cv = tid & 7;
  const int64_t nbn = a.C / BN;
  const int64_t bm = blockIdx.x / nbn, bn = blockIdx.x % nbn;
  const int64_t m0 = bm * BM;
  const int32_t n0 = (int32_t)bn * BN;
  const int32_t t_out = n0 / a.ct;
  const bool use_keep = a.keep != nullptr && clamp_flag_says_clamped(a.clamp_flag, a.flag_token);
  const int64_t mask_rows = clamp_rows(a.P);
  const uint32_t* plane = use_keep ? a.keep + (int64_t)t_out * ((a.N + 31) >> 5) * mask_rows : nullptr;

  f32x16 acc[2][2];
  float tot[2][2][16];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) { acc[i][j][v] = 0.0f; tot[i][j][v] = 0.0f; }

  // which of this lane's 64 outputs have their input on or beyond the range (per tap the same pixel)
  // and which are zeroed by the straight-through rule (|x| > range)
  uint64_t up = 0, lo = 0, zr = 0;
  const bool do_ir = a.flags != nullptr;
  if (do_ir) {
    // all loads first (rows beyond the last pixel carry zero flags), then the tests
#pragma unroll
    for (int bi = 0; bi < 2; ++bi)
#pragma unroll
      for (int bj = 0; bj < 2; ++bj) {
        uint32_t fv[16];
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int64_t m = m0 + wm * 64 + bi * 32 + 8 * (v >> 2) + 4 * h + (v & 3);
          const int32_t c = n0 + wn * 64 + bj * 32 + (lane & 31);
          fv[v] = a.flags[(m + a.conv.lead) * a.C + c];
        }
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int e = (bi * 2 + bj) * 16 + v;
          up |= (uint64_t)(fv[v] & 1u) << e;
          lo |= (uint64_t)((fv[v] >> 1) & 1u) << e;
          zr |= (uint64_t)((fv[v] >> 2) & 1u) << e;
        }
      }
  }
  // bit e set: some lane of the wave has its output e clipped (most registers have none)
  uint64_t wave_bits = up | lo;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) wave_bits |= __shfl_xor(wave_bits, o, 64);
  wave_bits = __builtin_amdgcn_readfirstlane((uint32_t)wave_bits) |
              ((uint64_t)__builtin_amdgcn_readfirstlane((uint32_t)(wave_bits >> 32)) << 32);
  float s_up = 0.0f, s_lo = 0.0f;

  const uint64_t bytesA = (uint64_t)(a.rows - m0) * (uint64_t)a.ldg * 2u;
  const __amdgpu_buffer_rsrc_t rsA = __builtin_amdgcn_make_buffer_rsrc(
      (void*)(a.g + m0 * a.ldg), 0, (int)(uint32_t)(bytesA > 0xffffffffull ? 0xffffffffull : bytesA), 0x00020000);
  const __amdgpu_buffer_rsrc_t rsB = __builtin_amdgcn_make_buffer_rsrc(
      (void*)(a.w + (int64_t)n0 * a.ldw), 0, (int)(uint32_t)((uint64_t)BN * (uint64_t)a.ldw * 2u), 0x00020000);
  int voA[NA], voB[NB];
#pragma unroll
  for (int j = 0; j < NA; ++j) voA[j] = (int)(((int64_t)(row0 + 32 * j) * a.ldg + cv * 8) * 2);
#pragma unroll
  for (int j = 0; j < NB; ++j) voB[j] = (int)(((int64_t)(row0 + 32 * j) * a.ldw + cv * 8) * 2);
  u32x4 rawA[NA], rawB[NB];
  // Clamp mask of the chunk being loaded, as the MFMA fragments need it: lane (r, h) multiplies
  // rows wm * 64 + r and + 32 of the block, 8 gradient values (one mask byte) per 16-wide step;
  // the 64 columns of a chunk are two mask words per row. Output row q reads the gradient of
  // output q - shift, whose words lie at row q - shift of the plane.
  uint32_t mk[2][2] = {{0u, 0u}, {0u, 0u}}, mk_next[2][2] = {{0u, 0u}, {0u, 0u}};
  const int cg = a.N / 64, nchunks = a.kvol * cg;
  auto load = [&](int ch) {
    const int tap = ch / cg, kc = (ch - tap * cg) * 64;
    const int32_t shift = conv_tap_rows(a.conv, tap);
    const int32_t kcA = (a.conv.lead - shift) * (int32_t)a.ldg + kc;
    const int32_t kcB = ch * 64;
#pragma unroll
    for (int j = 0; j < NA; ++j)
      rawA[j] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rsA, voA[j], kcA * 2, 0));
#pragma unroll
    for (int j = 0; j < NB; ++j)
      rawB[j] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rsB, voB[j], kcB * 2, 0));
    if (plane != nullptr) {
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int64_t src = m0 + wm * 64 + i * 32 + (lane & 31) - shift;
        const bool ok = src >= 0 && src < a.P;
        const uint32_t* w = plane + (int64_t)(kc >> 5) * mask_rows + (ok ? src : 0);
        mk_next[i][0] = ok ? w[0] : 0u;
        mk_next[i][1] = ok ? w[mask_rows] : 0u;
      }
    }
  };
  auto stage = [&]() {
    __syncthreads();
#pragma unroll
    for (int j = 0; j < NA; ++j) *(u32x4*)(ldsA + (row0 + 32 * j) * kStride + cv * 16) = rawA[j];
#pragma unroll
    for (int j = 0; j < NB; ++j) *(u32x4*)(ldsB + (row0 + 32 * j) * kStride + cv * 16) = rawB[j];
#pragma unroll
    for (int i = 0; i < 2; ++i) { mk[i][0] = mk_next[i][0]; mk[i][1] = mk_next[i][1]; }
    __syncthreads();
  };

  load(0);
  int cin = 0;
  for (int ch = 0; ch < nchunks; ++ch) {
    stage();
    if (ch + 1 < nchunks) load(ch + 1);
    {
      const int r = lane & 31;
      const char* pa = ldsA + (wm * 64 + r) * kStride + h * 16;
      const char* pb = ldsB + (wn * 64 + r) * kStride + h * 16;
      // clamps are rare: most chunks have no mask bit in any of the wave's 64 x 64 gradient values
      const bool masked = plane != nullptr && __any((mk[0][0] | mk[0][1] | mk[1][0] | mk[1][1]) != 0u);
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        u32x4 a0 = *(const u32x4*)(pa + s * 32), a1 = *(const u32x4*)(pa + 32 * kStride + s * 32);
        const u32x4 b0 = *(const u32x4*)(pb + s * 32), b1 = *(const u32x4*)(pb + 32 * kStride + s * 32);
        if (masked) {   // values s * 16 + h * 8 ... + 7 of the chunk: byte (2 s + h) of the row's 8
          const int sh = 8 * ((2 * s + h) & 3);
          a0 = zero_where_set8(a0, mk[0][s >> 1] >> sh);
          a1 = zero_where_set8(a1, mk[1][s >> 1] >> sh);
        }
        Mma16<D>::run(a0, b0, acc[0][0]);
        Mma16<D>::run(a1, b0, acc[1][0]);
        Mma16<D>::run(a0, b1, acc[0][1]);
        Mma16<D>::run(a1, b1, acc[1][1]);
      }
    }
    if (++cin < cg) continue;
    cin = 0;
    // a tap is complete: its partial, rounded to the dtype, is the patch-gradient entry of the
    // reference; it joins the pixel's fp32 sum and, where the input is clipped, the range sums
#pragma unroll
    for (int bi = 0; bi < 2; ++bi)
#pragma unroll
      for (int bj = 0; bj < 2; ++bj)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const float d = D::rd(acc[bi][bj][v]);
          acc[bi][bj][v] = 0.0f;
          tot[bi][bj][v] += d;
          const uint64_t bit = 1ull << ((bi * 2 + bj) * 16 + v);
          if (wave_bits & bit) {   // wave-uniform
            if (up & bit) s_up += fminf(d, 0.0f);
            if (lo & bit) s_lo += fmaxf(d, 0.0f);
          }
        }
  }

  // ---- store: rounded once, through LDS, 16-byte row vectors ----
  {
    constexpr int kOutStride = BN * 2 + 16;
    __syncthreads();
    char* obase = lds + (wm * 64 + 4 * h) * kOutStride + (wn * 64 + (lane & 31)) * 2;
#pragma unroll
    for (int bj = 0; bj < 2; ++bj)
#pragma unroll
      for (int bi = 0; bi < 2; ++bi)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int ro = bi * 32 + 8 * (v >> 2) + (v & 3);
          const bool zero = (zr >> ((bi * 2 + bj) * 16 + v)) & 1ull;
          *(uint16_t*)(obase + ro * kOutStride + bj * 64) = D::to_elem(zero ? 0.0f : tot[bi][bj][v]);
        }
    __syncthreads();
    constexpr int VPR = BN / 8, RPP = 256 / VPR;
    const int vcol = tid % VPR, vrow = tid / VPR;
#pragma unroll
    for (int j = 0; j < BM / RPP; ++j) {
      const int row = vrow + RPP * j;
      const int64_t m = m0 + row;
      if (m < a.P) st16(a.out + m * a.ldo + n0 + vcol * 8, *(const u32x4*)(lds + row * kOutStride + vcol * 16));
    }
  }
  if (do_ir) {
    s_up = wave_sum(s_up); s_lo = wave_sum(s_lo);
    if (lane == 0) { red[wave][0] = s_up; red[wave][1] = s_lo; }
    __syncthreads();
    if (tid == 0) {
      float* p = a.partial + (bm * nbn + bn) * 2;
      p[0] = (red[0][0] + red[1][0]) + (red[2][0] + red[3][0]);
      p[1] = (red[0][1] + red[1][1]) + (red[2][1] + red[3][1]);
    }
  }
}

// The same product for channel counts that are multiples of 128, operands straight from global
// memory into LDS (the scheme of k_fwd_pipe: 64-wide chunks, three stages, one barrier per chunk,
// 16-byte slots of a row XOR-swizzled with bits 1-3 of the row number). Block: 8 waves (two per
// SIMD), 256 pixels x 128 channels, every wave 64 x 64. The gradient rows lie in LDS unmasked and
// every wave applies the clamp mask of ITS K-tile to the fragments it reads, so the two column
// halves of a block may belong to different K-tiles. The mask words of a chunk (2 K-tiles x 2
// words x 256 rows) travel through LDS with the operands; without a mask (nothing was clamped)
// their descriptor is empty and they read as zero.
static constexpr int kDxRow = 128;
static constexpr int kDxLdsA = 256 * kDxRow, kDxLdsB = 128 * kDxRow, kDxLdsK = 2 * 2 * 256 * 4;
static constexpr int kDxStage = kDxLdsA + kDxLdsB + kDxLdsK;   // 53248
static constexpr int kDxStages = 3;
static constexpr int kDxLdsBytes = kDxStages * kDxStage;       // 159744

AHL_DEV void load_to_lds4(__amdgpu_buffer_rsrc_t rsrc, char* lds_base, int voffset) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_void_ptr)lds_base, 4, voffset, 0, 0, 0);
}

template <class D>
__global__ __launch_bounds__(512, 1) void k_conv_dx_pipe(ConvDxArgs a) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  __shared__ float red[8][2];
  // four mask bits -> the two dwords that keep the elements whose bit is clear (entry n: element
  // pairs (0, 1) and (2, 3) of the nibble); 16 entries of 8 bytes lie in 32 different banks
  __shared__ uint2 keep_lut[16];
  const int tid = threadIdx.x, lane = tid & 63;
  if (tid < 16) {
    auto pair = [](uint32_t two) { return ((two & 1u) ? 0u : 0xffffu) | ((two & 2u) ? 0u : 0xffff0000u); };
    keep_lut[tid] = make_uint2(pair((uint32_t)tid & 3u), pair((uint32_t)tid >> 2));
  }
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int h = lane >> 5, r = lane & 31;
  // The grid is a multiple of 8 blocks so that every XCD gets (block b runs on XCD b % 8) (and its L2) one
  // contiguous range of row blocks, both column blocks of a row block included: neighbouring row
  // blocks share their halo rows, the taps of one block re-read the same rows. Blocks beyond the
  // last tile leave at once.
  const int64_t nbn = a.C / 128, nbm = (a.P + 255) / 256;
  const int64_t lin = (int64_t)(blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
  if (lin >= nbm * nbn) return;
  const int64_t per_band = 16 * nbn, band = lin / per_band, in_band = lin % per_band;
  const int64_t first = band * 16, gsz = nbm - first < 16 ? nbm - first : 16;
  const int64_t bm = first + in_band % gsz, bn = in_band / gsz;
  const int64_t m0 = bm * 256;
  const int32_t n0 = (int32_t)bn * 128;
  const int32_t t_wave = (n0 + wn * 64) / a.ct;   // the K-tile of this wave's 64 channels
  const bool use_keep = a.keep != nullptr && clamp_flag_says_clamped(a.clamp_flag, a.flag_token);
  const int64_t mask_rows = clamp_rows(a.P);
  const int64_t plane_words = (int64_t)((a.N + 31) >> 5) * mask_rows;

  // which of this lane's 64 outputs have their input on or beyond the range (per tap the same pixel)
  // bit e of up / lo: this lane's output e (MFMA block e >> 4, register e & 15) has its input on or
  // beyond the upper / lower end of the range (per tap the same pixel)
  // zr: the outputs that the straight-through rule zeroes (|x| > range)
  uint32_t up[2] = {0u, 0u}, lo[2] = {0u, 0u}, zr[2] = {0u, 0u};
  const bool do_ir = a.flags != nullptr;
  if (do_ir) {
    uint32_t fv[2][2][16];   // all 64 loads in flight at once (rows beyond the pixels carry zero flags)
#pragma unroll
    for (int bi = 0; bi < 2; ++bi)
#pragma unroll
      for (int bj = 0; bj < 2; ++bj)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int64_t m = m0 + wm * 64 + bi * 32 + 8 * (v >> 2) + 4 * h + (v & 3);
          const int32_t c = n0 + wn * 64 + bj * 32 + r;
          fv[bi][bj][v] = a.flags[(m + a.conv.lead) * a.C + c];
        }
#pragma unroll
    for (int bi = 0; bi < 2; ++bi)
#pragma unroll
      for (int bj = 0; bj < 2; ++bj)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int e = bj * 16 + v;
          up[bi] |= (fv[bi][bj][v] & 1u) << e;
          lo[bi] |= ((fv[bi][bj][v] >> 1) & 1u) << e;
          zr[bi] |= ((fv[bi][bj][v] >> 2) & 1u) << e;
        }
  }
  // the same for the wave: most of the 64 registers have no clipped input in any lane
  uint32_t wave_bits[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    uint32_t w = up[i] | lo[i];
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) w |= __shfl_xor(w, o, 64);
    wave_bits[i] = __builtin_amdgcn_readfirstlane(w);
  }
  f32x16 acc[2][2];
  float tot[2][2][16];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) { tot[i][j][v] = 0.0f; }

  float s_up = 0.0f, s_lo = 0.0f;

  const __amdgpu_buffer_rsrc_t rsA = make_rsrc(a.g + m0 * a.ldg, (uint64_t)(a.rows - m0) * (uint64_t)a.ldg * 2u);
  const __amdgpu_buffer_rsrc_t rsB = make_rsrc(a.w + (int64_t)n0 * a.ldw, (uint64_t)128 * (uint64_t)a.ldw * 2u);
  // mask words: wave w brings word (w >> 1) & 1 of the rows (w & 1) * 128 ... + 127 of the K-tile
  // of column half w >> 2
  const int ksel = wave >> 2, kword = (wave >> 1) & 1, krow0 = (wave & 1) * 128 + lane;
  const int32_t t_load = (n0 + ksel * 64) / a.ct;
  const __amdgpu_buffer_rsrc_t rsK =
      make_rsrc(use_keep ? a.keep + (int64_t)t_load * plane_words : a.keep, use_keep ? (uint64_t)plane_words * 4u : 0u);
  int voA[4], voB[2];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int row = wave * 32 + 8 * j + (lane >> 3);
    voA[j] = (int)(((int64_t)row * a.ldg + (((lane & 7) ^ ((row >> 1) & 7)) * 8)) * 2);
  }
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int row = wave * 16 + 8 * j + (lane >> 3);
    voB[j] = (int)(((int64_t)row * a.ldw + (((lane & 7) ^ ((row >> 1) & 7)) * 8)) * 2);
  }
  constexpr int kLoads = 4 + 2 + 2;   // vector memory operations of one chunk, per wave
  const int cg = a.N / 64, nchunks = a.kvol * cg;
  int st_load = 0, ltap = 0, lcin = 0;   // stage, tap and position in the tap of the next chunk to load
  int tap_w = 0, tap_h = 0, tap_d = 0;   // the tap's kernel coordinates (no divisions per chunk)
  auto load = [&]() __attribute__((always_inline)) {
    const int32_t shift = (tap_d * a.conv.hp + tap_h) * a.conv.wp + tap_w;
    const int32_t kcA = (a.conv.lead - shift) * (int32_t)a.ldg + lcin * 64;
    const int32_t kcB = (ltap * cg + lcin) * 64;
    char* sa = lds + st_load * kDxStage + wave * (32 * kDxRow);
    char* sb = lds + st_load * kDxStage + kDxLdsA + wave * (16 * kDxRow);
    char* sk = lds + st_load * kDxStage + kDxLdsA + kDxLdsB + ((ksel * 2 + kword) * 256 + (wave & 1) * 128) * 4;
#pragma unroll
    for (int j = 0; j < 4; ++j) load_to_lds16(rsA, sa + j * 8 * kDxRow, voA[j], kcA * 2);
#pragma unroll
    for (int j = 0; j < 2; ++j) load_to_lds16(rsB, sb + j * 8 * kDxRow, voB[j], kcB * 2);
    // output row q reads the gradient of output q - shift: its mask words lie at that row
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int64_t src = m0 + krow0 + 64 * j - shift;
      const bool ok = src >= 0 && src < a.P;
      const int64_t word = (int64_t)(2 * lcin + kword) * mask_rows + src;
      load_to_lds4(rsK, sk + j * 256, ok ? (int)(word * 4) : -1);
    }
    st_load = st_load == kDxStages - 1 ? 0 : st_load + 1;
    if (++lcin == cg) {
      lcin = 0; ++ltap;
      if (++tap_w == a.conv.kw) { tap_w = 0; if (++tap_h == a.conv.kh) { tap_h = 0; ++tap_d; } }
    }
  };

  load();
  if (nchunks > 1) load();
  if (nchunks > 2) load();
  if (nchunks > 2) lds_barrier<2 * kLoads>();
  else if (nchunks > 1) lds_barrier<kLoads>();
  else lds_barrier<0>();

  uint32_t rdA = (wm * 64 + r) * kDxRow + ((h ^ ((r >> 1) & 7)) << 4);
  uint32_t rdB = kDxLdsA + (wn * 64 + r) * kDxRow + ((h ^ ((r >> 1) & 7)) << 4);
  uint32_t rdK = kDxLdsA + kDxLdsB + (wn * 2 * 256 + wm * 64 + r) * 4;
  int st_read = 0;
  u32x4 fa[2][2], fb[2][2];   // fragments of two consecutive k-steps
  auto read_frags = [&](int s, int buf) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < 2; ++i) fa[buf][i] = *(const u32x4*)(lds + (rdA ^ (s << 5)) + i * 32 * kDxRow);
#pragma unroll
    for (int j = 0; j < 2; ++j) fb[buf][j] = *(const u32x4*)(lds + (rdB ^ (s << 5)) + j * 32 * kDxRow);
  };
  // one 64-wide chunk: the reads of k-step s + 1 are issued before the MFMAs of k-step s
  auto chunk = [&](auto first_c) __attribute__((always_inline)) {
    constexpr bool FIRST = decltype(first_c)::value;   // first chunk of a tap: the sums start from zero
    // the mask words of the two row halves (64 columns of the chunk: two words each)
    const uint32_t k00 = *(const uint32_t*)(lds + rdK), k01 = *(const uint32_t*)(lds + rdK + 1024);
    const uint32_t k10 = *(const uint32_t*)(lds + rdK + 128), k11 = *(const uint32_t*)(lds + rdK + 1024 + 128);
    read_frags(0, 0);
    const bool masked = __any((k00 | k01 | k10 | k11) != 0u);
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      if (s < 3) read_frags(s + 1, (s + 1) & 1);
      if (masked) {   // values s * 16 + h * 8 ... + 7 of the chunk: byte (2 s + h) of the row's 8
        const int sh = 8 * ((2 * s + h) & 3);
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          const uint32_t byte = (i == 0 ? (s < 2 ? k00 : k01) : (s < 2 ? k10 : k11)) >> sh;
          const uint2 lo2 = keep_lut[byte & 15u], hi2 = keep_lut[(byte >> 4) & 15u];
          fa[s & 1][i].x &= lo2.x; fa[s & 1][i].y &= lo2.y;
          fa[s & 1][i].z &= hi2.x; fa[s & 1][i].w &= hi2.y;
        }
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          if (FIRST && s == 0) Mma16<D>::run_zero(fa[0][i], fb[0][j], acc[i][j]);
          else Mma16<D>::run(fa[s & 1][i], fb[s & 1][j], acc[i][j]);
        }
    }
  };
  int ch = 0;
  for (int tap = 0; tap < a.kvol; ++tap) {
    for (int c = 0; c < cg; ++c, ++ch) {
      if (c == 0) chunk(std::true_type{}); else chunk(std::false_type{});
      // end of the chunk: the next one must have landed before anyone reads it, and the stage of
      // this one takes the chunk after next
      if (ch + 2 < nchunks) lds_barrier<kLoads>(); else lds_barrier<0>();
      if (ch + 3 < nchunks) load();
      const bool wrap = st_read == kDxStages - 1;
      st_read = wrap ? 0 : st_read + 1;
      const int step = wrap ? -(kDxStages - 1) * kDxStage : kDxStage;
      rdA += step; rdB += step; rdK += step;
    }
    // the tap is complete: its partial, rounded to the dtype, is the patch-gradient entry of the
    // reference; it joins the pixel's fp32 sum and, where the input is clipped, the range sums
    // (the masks are made opaque here: tests hoisted out of the loop would be 128 lane masks)
    asm volatile("" : "+v"(up[0]), "+v"(up[1]), "+v"(lo[0]), "+v"(lo[1]));
#pragma unroll
    for (int bi = 0; bi < 2; ++bi)
#pragma unroll
      for (int bj = 0; bj < 2; ++bj)
#pragma unroll
        for (int v = 0; v < 16; v += 2) {
          const uint32_t pr = D::pack2(acc[bi][bj][v], acc[bi][bj][v + 1]);
          const float d0 = D::lo(pr), d1 = D::hi(pr);
          tot[bi][bj][v] += d0;
          tot[bi][bj][v + 1] += d1;
          const int e = bj * 16 + v;
          if ((wave_bits[bi] >> e) & 3u) {   // wave-uniform
            if ((up[bi] >> e) & 1u) s_up += fminf(d0, 0.0f);
            if ((lo[bi] >> e) & 1u) s_lo += fmaxf(d0, 0.0f);
            if ((up[bi] >> (e + 1)) & 1u) s_up += fminf(d1, 0.0f);
            if ((lo[bi] >> (e + 1)) & 1u) s_lo += fmaxf(d1, 0.0f);
          }
        }
  }

  // ---- store: rounded once, through LDS, 16-byte row vectors ----
  {
    constexpr int kOutStride = 128 * 2 + 16;
    __syncthreads();
    char* obase = lds + (wm * 64 + 4 * h) * kOutStride + (wn * 64 + r) * 2;
#pragma unroll
    for (int bj = 0; bj < 2; ++bj)
#pragma unroll
      for (int bi = 0; bi < 2; ++bi)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int ro = bi * 32 + 8 * (v >> 2) + (v & 3);
          const bool zero = (zr[bi] >> (bj * 16 + v)) & 1u;
          *(uint16_t*)(obase + ro * kOutStride + bj * 64) = D::to_elem(zero ? 0.0f : tot[bi][bj][v]);
        }
    __syncthreads();
    const int vcol = tid & 15, vrow = tid >> 4;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int row = vrow + 32 * j;
      const int64_t m = m0 + row;
      if (m < a.P) st16(a.out + m * a.ldo + n0 + vcol * 8, *(const u32x4*)(lds + row * kOutStride + vcol * 16));
    }
  }
  if (do_ir) {
    s_up = wave_sum(s_up); s_lo = wave_sum(s_lo);
    if (lane == 0) { red[wave][0] = s_up; red[wave][1] = s_lo; }
    __syncthreads();
    if (tid < 2) {   // one pair of sums per 64-column half
      float* p = a.partial + (bm * (a.C / 64) + n0 / 64 + tid) * 2;
      p[0] = (red[tid][0] + red[2 + tid][0]) + (red[4 + tid][0] + red[6 + tid][0]);
      p[1] = (red[tid][1] + red[2 + tid][1]) + (red[4 + tid][1] + red[6 + tid][1]);
    }
  }
}

// ir_grad[t] from the blocks' partial sums and the clipped-entry counts (reference
// torch_utils/torch_linear.py:92-106; the roundings of k_ir_grad_finalize).
template <class D>
__global__ __launch_bounds__(1024) void k_conv_ir_finalize(const float* __restrict__ partial, int64_t row_blocks,
                                                          int32_t col_blocks, int32_t per_tile,
                                                          const uint32_t* __restrict__ count,
                                                          int64_t count_rows, int32_t count_cols,
                                                          int32_t count_per_tile,
                                                          double numel, const void* ir, void* ir_grad,
                                                          float decay, float min_pct) {
  __shared__ double part[16][2];
  __shared__ unsigned long long part_count[16];
  const int t = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  double s_up = 0.0, s_lo = 0.0;
  // clipped patch entries of the tile: the layout kernel's counts [count_rows][count_cols], this
  // tile's columns. A thread walks rows (every 1024th), so that the loop holds no division and the
  // loads of a pass are independent.
  unsigned long long clipped = 0;
  for (int64_t r = tid; r < count_rows; r += 1024) {
    const uint32_t* c = count + r * count_cols + (int64_t)t * count_per_tile;
    for (int32_t j = 0; j < count_per_tile; ++j) clipped += c[j];
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) clipped += __shfl_xor(clipped, o, 64);
  for (int64_t rb = tid; rb < row_blocks; rb += 1024) {
    const float* p = partial + (rb * col_blocks + (int64_t)t * per_tile) * 2;
    for (int32_t j = 0; j < per_tile; ++j) { s_up += (double)p[2 * j]; s_lo += (double)p[2 * j + 1]; }
  }
  s_up = wave_sum(s_up); s_lo = wave_sum(s_lo);
  if (lane == 0) { part[wave][0] = s_up; part[wave][1] = s_lo; part_count[wave] = clipped; }
  __syncthreads();
  if (tid == 0) {
    s_up = 0.0; s_lo = 0.0; clipped = 0;
    for (int w = 0; w < 16; ++w) { s_up += part[w][0]; s_lo += part[w][1]; clipped += part_count[w]; }
    const float irv = D::load(ir, t);
    float gr = D::rd(0.0f + D::rd((float)s_up));
    gr = D::rd(gr - D::rd((float)s_lo));
    gr = D::rd(gr * irv);
    if (decay > 0.0f) {
      const float pct = 1.0f - __fdiv_rn((float)clipped, (float)numel);
      const float add = pct > min_pct ? D::rd(decay * irv) : 0.0f;
      gr = D::rd(gr + add);
    }
    D::store(ir_grad, t, gr);
  }
}

static bool direct_dtype(int32_t dtype) { return dtype == AHL_BF16 || dtype == AHL_F16; }

// Channels per K-tile if the split holds whole channels in multiples of 64, else 0.
static int32_t channels_per_tile(const DirectGeom& g, const Tiling& tl) {
  if (tl.extra != 0 || tl.base % g.kvol != 0) return 0;
  const int32_t ct = tl.base / g.kvol;
  return (ct % 64 == 0 && g.C % ct == 0) ? ct : 0;
}

}  // namespace ahl

using namespace ahl;

extern "C" {

int ahl_conv_direct_rows(const AhlConvGeom* geom, int64_t* pixels, int64_t* lead, int64_t* rows) {
  DirectGeom g;
  if (!make_direct(geom, &g) || !pixels || !lead || !rows) return AHL_ERR_ARG;
  *pixels = g.P; *lead = g.lead; *rows = g.rows;
  return AHL_OK;
}

int ahl_conv_direct_supported(const AhlConvGeom* geom, int32_t dtype, int64_t N, const int32_t* tile_ends_host,
                              int32_t n_tiles) {
  DirectGeom g;
  Tiling tl;
  if (!direct_dtype(dtype) || !make_direct(geom, &g)) return 0;
  if (!make_tiling(tile_ends_host, n_tiles, (int64_t)g.C * g.kvol, &tl)) return 0;
  if (N <= 0 || N % 64 != 0 || N > 16384) return 0;
  return channels_per_tile(g, tl) > 0 ? 1 : 0;
}

int64_t ahl_conv_count_words(const AhlConvGeom* geom) {
  DirectGeom g;
  if (!make_direct(geom, &g)) return -1;
  return cdiv(g.rows, 64) * cdiv(g.C, 64);
}

int ahl_conv_image_rows(const void* x, const AhlConvGeom* geom, int32_t dtype, const void* ir,
                        const int32_t* tile_ends_host, int32_t n_tiles, const AhlLinearCfg* cfg, void* xq_rows,
                        uint8_t* flag_rows, uint32_t* counts, void* stream) {
  DirectGeom g;
  Tiling tl;
  if (!x || !xq_rows || !cfg || !direct_dtype(dtype) || !make_direct(geom, &g)) return AHL_ERR_ARG;
  if ((flag_rows == nullptr) != (counts == nullptr)) return AHL_ERR_ARG;
  if (!make_tiling(tile_ends_host, n_tiles, (int64_t)g.C * g.kvol, &tl)) return AHL_ERR_TILING;
  const int32_t ct = channels_per_tile(g, tl);
  if (ct == 0 || cfg->ir_mode == AHL_IR_DYNAMIC || (cfg->ir_mode == AHL_IR_STATIC && !ir)) return AHL_ERR_UNSUPPORTED;
  if (cfg->ir_mode == AHL_IR_NONE && (cfg->inp_res > 0.0f || flag_rows)) return AHL_ERR_ARG;
  const int32_t S = g.in[0] * g.in[1] * g.in[2];
  const RowMap map = {g.in[0], g.in[1], g.in[2], g.pad[0], g.pad[1], g.pad[2], g.pin[0], g.pin[1], g.pin[2]};
  const TapSpan taps = {g.ker[0], g.ker[1], g.ker[2], g.out[0], g.out[1], g.out[2]};
  const dim3 grid((unsigned)cdiv(g.rows, 64), (unsigned)cdiv(g.C, 64));
  hipStream_t s = (hipStream_t)stream;
#define AHL_SCATTER(DT, MODE)                                                                          \
  hipLaunchKernelGGL((k_conv_scatter<DT, MODE>), grid, dim3(256), 0, s, (const uint16_t*)x, g.C, S, map, \
                     g.lead, g.P, g.rows, (uint16_t*)xq_rows, flag_rows, counts, taps, ir, ct,           \
                     cfg->inp_res, cfg->skip_rounding)
  if (dtype == AHL_F16) { if (cfg->ir_mode == AHL_IR_STATIC) AHL_SCATTER(F16, 1); else AHL_SCATTER(F16, 0); }
  else { if (cfg->ir_mode == AHL_IR_STATIC) AHL_SCATTER(BF16, 1); else AHL_SCATTER(BF16, 0); }
#undef AHL_SCATTER
  return check_launch("ahl_conv_image_rows");
}

int ahl_conv_grad_rows(const void* g_out, const AhlConvGeom* geom, int32_t dtype, int64_t N, void* g_rows,
                       void* stream) {
  DirectGeom g;
  if (!g_out || !g_rows || N <= 0 || N % 8 != 0 || !direct_dtype(dtype) || !make_direct(geom, &g)) return AHL_ERR_ARG;
  const int32_t S = g.out[0] * g.out[1] * g.out[2];
  const RowMap map = {g.out[0], g.out[1], g.out[2], 0, 0, 0, g.pin[0], g.pin[1], g.pin[2]};
  const dim3 grid((unsigned)cdiv(g.rows, 64), (unsigned)cdiv(N, 64));
  hipStream_t s = (hipStream_t)stream;
  if (dtype == AHL_F16)
    hipLaunchKernelGGL((k_conv_scatter<F16, 0>), grid, dim3(256), 0, s, (const uint16_t*)g_out, (int32_t)N, S, map,
                       g.lead, g.P, g.rows, (uint16_t*)g_rows, (uint8_t*)nullptr, (uint32_t*)nullptr, TapSpan{1, 1, 1, 1, 1, 1},
                       (const void*)nullptr, 64, 0.0f, 0);
  else
    hipLaunchKernelGGL((k_conv_scatter<BF16, 0>), grid, dim3(256), 0, s, (const uint16_t*)g_out, (int32_t)N, S, map,
                       g.lead, g.P, g.rows, (uint16_t*)g_rows, (uint8_t*)nullptr, (uint32_t*)nullptr, TapSpan{1, 1, 1, 1, 1, 1},
                       (const void*)nullptr, 64, 0.0f, 0);
  return check_launch("ahl_conv_grad_rows");
}

int ahl_conv_output(const void* y_rows, const AhlConvGeom* geom, int32_t dtype, int64_t N, void* y, void* stream) {
  DirectGeom g;
  if (!y_rows || !y || N <= 0 || N % 8 != 0 || !direct_dtype(dtype) || !make_direct(geom, &g)) return AHL_ERR_ARG;
  const int32_t S = g.out[0] * g.out[1] * g.out[2];
  const RowMap map = {g.out[0], g.out[1], g.out[2], 0, 0, 0, g.pin[0], g.pin[1], g.pin[2]};
  const dim3 grid((unsigned)cdiv(S, 64), (unsigned)cdiv(N, 64), (unsigned)g.B);
  hipStream_t s = (hipStream_t)stream;
  // the output rows carry no lead: row p of y_rows is output p
  if (dtype == AHL_F16)
    hipLaunchKernelGGL((k_conv_gather<F16>), grid, dim3(256), 0, s, (const uint16_t*)y_rows, (int32_t)N, S, map, 0,
                       (uint16_t*)y);
  else
    hipLaunchKernelGGL((k_conv_gather<BF16>), grid, dim3(256), 0, s, (const uint16_t*)y_rows, (int32_t)N, S, map, 0,
                       (uint16_t*)y);
  return check_launch("ahl_conv_output");
}

int ahl_conv_weight_layout(const void* src, int64_t ld_src, int32_t dtype, int64_t N, const AhlConvGeom* geom,
                           const int32_t* tile_ends_host, int32_t n_tiles, int32_t mode, int64_t stride, void* dst,
                           int64_t ld_dst, void* stream) {
  DirectGeom g;
  Tiling tl;
  if (!src || !dst || N <= 0 || mode < 0 || mode > 2 || !direct_dtype(dtype) || !make_direct(geom, &g)) return AHL_ERR_ARG;
  if (!make_tiling(tile_ends_host, n_tiles, (int64_t)g.C * g.kvol, &tl)) return AHL_ERR_TILING;
  const int32_t ct = channels_per_tile(g, tl);
  if (ct == 0) return AHL_ERR_UNSUPPORTED;
  const int64_t total = N * g.C * g.kvol;
  const bool dx = mode == 2;
  hipLaunchKernelGGL((k_conv_weights<uint16_t>), dim3((unsigned)cdiv(total, 256)), dim3(256), 0, (hipStream_t)stream,
                     (const uint16_t*)src, ld_src, (int32_t)N, g.C, g.kvol, ct, (int32_t)stride, (int)mode,
                     dx ? nullptr : (uint16_t*)dst, dx ? 0 : ld_dst, dx ? (uint16_t*)dst : nullptr, dx ? ld_dst : 0);
  return check_launch("ahl_conv_weight_layout");
}

int ahl_conv_weight_layouts(const void* src, int64_t ld_src, int32_t dtype, int64_t N, const AhlConvGeom* geom,
                            const int32_t* tile_ends_host, int32_t n_tiles, void* w_taps, int64_t ld_taps, void* w_dx,
                            int64_t ld_dx, void* stream) {
  DirectGeom g;
  Tiling tl;
  if (!src || !w_taps || !w_dx || N <= 0 || !direct_dtype(dtype) || !make_direct(geom, &g)) return AHL_ERR_ARG;
  if (!make_tiling(tile_ends_host, n_tiles, (int64_t)g.C * g.kvol, &tl)) return AHL_ERR_TILING;
  const int32_t ct = channels_per_tile(g, tl);
  if (ct == 0) return AHL_ERR_UNSUPPORTED;
  const int64_t total = N * g.C * g.kvol;
  hipLaunchKernelGGL((k_conv_weights<uint16_t>), dim3((unsigned)cdiv(total, 256)), dim3(256), 0, (hipStream_t)stream,
                     (const uint16_t*)src, ld_src, (int32_t)N, g.C, g.kvol, ct, 0, 0, (uint16_t*)w_taps, ld_taps,
                     (uint16_t*)w_dx, ld_dx);
  return check_launch("ahl_conv_weight_layouts");
}

int ahl_conv_fwd(const void* xq_rows, const void* w_taps, const void* bias, void* y_rows, uint32_t* keep,
                 uint32_t* clamp_flag, const void* ir, const void* wmax, const float* tile_max,
                 const AhlConvGeom* geom, int64_t N, const int32_t* tile_ends_host, int32_t n_tiles,
                 const AhlLinearCfg* cfg, void* stream) {
  DirectGeom g;
  Tiling tl;
  if (!xq_rows || !w_taps || !y_rows || !cfg || !direct_dtype(cfg->dtype) || !make_direct(geom, &g)) return AHL_ERR_ARG;
  const int64_t K = (int64_t)g.C * g.kvol;
  if (!make_tiling(tile_ends_host, n_tiles, K, &tl)) return AHL_ERR_TILING;
  const int32_t ct = channels_per_tile(g, tl);
  if (ct == 0 || N <= 0 || N % 64 != 0 || cfg->ir_mode == AHL_IR_DYNAMIC || cfg->tile_stride != 0) return AHL_ERR_UNSUPPORTED;
  {
    const bool noise_on = cfg->training && cfg->out_noise > 0.0f;
    const bool bound_on = cfg->out_res > 0.0f || cfg->out_bound > 0.0f;
    if (cfg->ir_mode == AHL_IR_NONE && (bound_on || noise_on)) return AHL_ERR_ARG;
    if (cfg->ir_mode != AHL_IR_NONE && !ir) return AHL_ERR_ARG;
    if ((noise_on || bound_on) && (!wmax || !tile_max)) return AHL_ERR_ARG;
  }
  const ConvMap map = make_map(g, +1, ct / 64, ct, g.rows - g.lead);
  const uint16_t* base = (const uint16_t*)xq_rows + (int64_t)g.lead * g.C;
  return launch_fast_fwd(base, g.C, w_taps, K, bias, y_rows, N, keep, clamp_flag, ir, wmax, tile_max, g.P, K, N, tl,
                         cfg, nullptr, (hipStream_t)stream, &map);
}

int64_t ahl_conv_bwd_dw_ws_bytes(const AhlConvGeom* geom, int64_t N, const int32_t* tile_ends_host, int32_t n_tiles,
                                 int64_t* padded_cols) {
  DirectGeom g;
  Tiling tl;
  if (!make_direct(geom, &g) || !make_tiling(tile_ends_host, n_tiles, (int64_t)g.C * g.kvol, &tl)) return -1;
  const int bw = fast_dw_image_block(g.P, tl.base, n_tiles, N);
  const int64_t stride = cdiv(tl.base, bw) * bw, kp = stride * n_tiles;
  if (padded_cols) *padded_cols = kp;
  return fast_dw_ws_bytes(g.P, kp, N, bw);
}

int ahl_conv_bwd_dw(const void* g_rows, const uint32_t* keep, const uint32_t* clamp_flag, const void* xq_rows,
                    void* dw_tiled, void* dbias, const AhlConvGeom* geom, int64_t N, const int32_t* tile_ends_host,
                    int32_t n_tiles, const AhlLinearCfg* cfg, void* ws, void* stream) {
  DirectGeom g;
  Tiling tl;
  if (!g_rows || !xq_rows || !dw_tiled || !cfg || !ws || !direct_dtype(cfg->dtype) || !make_direct(geom, &g)) return AHL_ERR_ARG;
  if (!make_tiling(tile_ends_host, n_tiles, (int64_t)g.C * g.kvol, &tl)) return AHL_ERR_TILING;
  const int32_t ct = channels_per_tile(g, tl);
  if (ct == 0 || N <= 0 || N % 8 != 0) return AHL_ERR_UNSUPPORTED;
  // columns per block and per K-tile of dw_tiled: the tile itself when blocks of 192 or 256 columns
  // divide it, else the tile padded to whole blocks of 256
  const int bw = fast_dw_image_block(g.P, tl.base, n_tiles, N);
  const int32_t stride = (int32_t)(cdiv(tl.base, bw) * bw);
  const int64_t kp = (int64_t)stride * n_tiles;
  Tiling padded;
  padded.n_tiles = n_tiles; padded.base = stride; padded.extra = 0;
  const ConvMap map = make_map(g, +1, ct / 64, ct, g.rows - g.lead);
  const uint16_t* gb = (const uint16_t*)g_rows + (int64_t)g.lead * N;
  const uint16_t* xb = (const uint16_t*)xq_rows + (int64_t)g.lead * g.C;
  return launch_fast_dw(cfg->dtype, gb, N, keep, clamp_flag, cfg->flag_token, xb, g.C, dw_tiled, kp, dbias, ws, g.P, kp, N,
                        padded, (hipStream_t)stream, &map, g.kvol * ct, bw);
}

int64_t ahl_conv_bwd_dx_ws_bytes(const AhlConvGeom* geom, int32_t n_tiles) {
  DirectGeom g;
  if (!make_direct(geom, &g) || n_tiles <= 0) return -1;
  // the blocks' partial sums of the range gradient: [row blocks][C / 64][2] floats
  return (cdiv(g.P, 128) * (g.C / 64) * 2 * 4 + 255) / 256 * 256;
}

int ahl_conv_bwd_dx(const void* g_rows, const uint32_t* keep, const uint32_t* clamp_flag, const void* w_dx,
                    const uint8_t* flag_rows, const uint32_t* counts, const void* ir, void* dimg_rows, void* dx,
                    void* ir_grad, const AhlConvGeom* geom, int64_t N, const int32_t* tile_ends_host, int32_t n_tiles,
                    const AhlLinearCfg* cfg, void* ws, void* stream) {
  DirectGeom g;
  Tiling tl;
  if (!g_rows || !w_dx || !dimg_rows || !dx || !cfg || !direct_dtype(cfg->dtype) || !make_direct(geom, &g)) return AHL_ERR_ARG;
  if (!make_tiling(tile_ends_host, n_tiles, (int64_t)g.C * g.kvol, &tl)) return AHL_ERR_TILING;
  const int32_t ct = channels_per_tile(g, tl);
  if (ct == 0 || N <= 0 || N % 64 != 0) return AHL_ERR_UNSUPPORTED;
  const bool is_static = cfg->ir_mode == AHL_IR_STATIC;
  if (is_static && (!flag_rows || !counts || !ir || !ir_grad || !ws || cfg->ir_grad_rule != AHL_IR_GRAD_LEARNED))
    return AHL_ERR_ARG;
  hipStream_t s = (hipStream_t)stream;
  // blocks: 256 x 128 (channel counts that are multiples of 128), else 128 x 128 or 256 x 64
  const bool pipe = g.C % 128 == 0;
  const bool wide = ct % 128 == 0;
  const int bm_rows = pipe ? 256 : wide ? 128 : 256, bn_cols = pipe ? 128 : wide ? 128 : 64;
  const int64_t row_blocks = cdiv(g.P, bm_rows);
  const int32_t col_blocks = g.C / bn_cols;
  // partial sums per (row block, column block); the 256 x 128 blocks leave one pair per 64 columns
  const int32_t partial_cols = pipe ? g.C / 64 : col_blocks, partial_per_tile = pipe ? ct / 64 : ct / bn_cols;
  float* partial = (float*)ws;
  ConvDxArgs a;
  a.g = (const uint16_t*)g_rows; a.ldg = N; a.keep = keep; a.clamp_flag = clamp_flag; a.flag_token = cfg->flag_token;
  a.w = (const uint16_t*)w_dx; a.ldw = (int64_t)g.kvol * N;
  a.flags = is_static ? flag_rows : nullptr;
  a.out = (uint16_t*)dimg_rows; a.ldo = g.C; a.partial = partial;
  a.P = g.P; a.rows = g.rows; a.N = (int32_t)N; a.C = g.C; a.ct = ct; a.kvol = g.kvol;
  a.conv = make_map(g, -1, (int32_t)(N / 64), 0, g.rows);
  if (row_blocks * col_blocks > 0x7fffffff) return AHL_ERR_ARG;
  const dim3 grid((unsigned)(pipe ? cdiv(row_blocks * col_blocks, 8) * 8 : row_blocks * col_blocks));
  if (pipe) {
    if (cfg->dtype == AHL_F16) {
      (void)hipFuncSetAttribute((const void*)k_conv_dx_pipe<F16>, hipFuncAttributeMaxDynamicSharedMemorySize, kDxLdsBytes);
      hipLaunchKernelGGL((k_conv_dx_pipe<F16>), grid, dim3(512), kDxLdsBytes, s, a);
    } else {
      (void)hipFuncSetAttribute((const void*)k_conv_dx_pipe<BF16>, hipFuncAttributeMaxDynamicSharedMemorySize, kDxLdsBytes);
      hipLaunchKernelGGL((k_conv_dx_pipe<BF16>), grid, dim3(512), kDxLdsBytes, s, a);
    }
  } else {
    const int lds_bytes = (bm_rows + bn_cols) * 144;   // the output staging (rows x (2 cols + 16)) fits too
    if (cfg->dtype == AHL_F16) {
      if (wide) hipLaunchKernelGGL((k_conv_dx<F16, 2, 2>), grid, dim3(256), lds_bytes, s, a);
      else hipLaunchKernelGGL((k_conv_dx<F16, 4, 1>), grid, dim3(256), lds_bytes, s, a);
    } else {
      if (wide) hipLaunchKernelGGL((k_conv_dx<BF16, 2, 2>), grid, dim3(256), lds_bytes, s, a);
      else hipLaunchKernelGGL((k_conv_dx<BF16, 4, 1>), grid, dim3(256), lds_bytes, s, a);
    }
  }
  // pixel rows -> [B, C, *spatial] (the range mask is applied already)
  const int32_t S = g.in[0] * g.in[1] * g.in[2];
  const RowMap map = {g.in[0], g.in[1], g.in[2], g.pad[0], g.pad[1], g.pad[2], g.pin[0], g.pin[1], g.pin[2]};
  const dim3 ggrid((unsigned)cdiv(S, 64), (unsigned)cdiv(g.C, 64), (unsigned)g.B);
  if (cfg->dtype == AHL_F16)
    hipLaunchKernelGGL((k_conv_gather<F16>), ggrid, dim3(256), 0, s, (const uint16_t*)dimg_rows, g.C, S, map, 0, (uint16_t*)dx);
  else
    hipLaunchKernelGGL((k_conv_gather<BF16>), ggrid, dim3(256), 0, s, (const uint16_t*)dimg_rows, g.C, S, map, 0, (uint16_t*)dx);
  if (is_static) {
    const double numel = (double)g.B * g.out[0] * g.out[1] * g.out[2] * (double)tl.base;
    // the clipped-entry counts of k_conv_scatter: [blocks of 64 rows][C / 64]
    if (cfg->dtype == AHL_F16)
      hipLaunchKernelGGL((k_conv_ir_finalize<F16>), dim3(n_tiles), dim3(1024), 0, s, (const float*)partial, row_blocks,
                         partial_cols, partial_per_tile, counts, cdiv(g.rows, 64), g.C / 64, ct / 64,
                         numel, ir, ir_grad, cfg->ir_decay, cfg->ir_input_min_percentage);
    else
      hipLaunchKernelGGL((k_conv_ir_finalize<BF16>), dim3(n_tiles), dim3(1024), 0, s, (const float*)partial, row_blocks,
                         partial_cols, partial_per_tile, counts, cdiv(g.rows, 64), g.C / 64, ct / 64,
                         numel, ir, ir_grad, cfg->ir_decay, cfg->ir_input_min_percentage);
  }
  return check_launch("ahl_conv_bwd_dx");
}

}  // extern "C"
