// Data movement that turns a convolution into the tiled analog matrix product: patch extraction
// (im2col), its adjoint (col2im) and the batched transpose between the [tokens, channels] layout
// of the matrix product and the [channels, positions] layout of a convolution output.
//
// All three are pure HBM kernels. Patches are written as rows of a [B * L, C * kD * kH * kW]
// matrix (L output positions per image), channel-major then kernel offsets with the last spatial
// dimension fastest: the order of `weight.view(out_channels, -1)` of a torch convolution weight,
// so the K-tiles of the analog layer cut the same columns as in the reference
// (nn/modules/conv.py:310-325 for 1-d/2-d through torch's unfold, :40-103 for 3-d).
// 1-d and 2-d convolutions use the same code with leading sizes of one.
#include "ahl_host.h"

namespace ahl {

struct ConvGeom {
  int32_t B, C;
  int32_t in[3], out[3], ker[3], str[3], pad[3], dil[3];
  int32_t kvol;  // kernel offsets per channel
  int64_t L;     // output positions per image
  int64_t K;     // patch length C * kvol
};

// Output extent of one dimension (torch's convolution arithmetic); <= 0 means "does not fit".
static int64_t conv_extent(int64_t in, int64_t ker, int64_t str, int64_t pad, int64_t dil) {
  const int64_t span = in + 2 * pad - dil * (ker - 1) - 1;
  if (span < 0) return 0;
  return span / str + 1;
}

static bool make_geom(const AhlConvGeom* a, ConvGeom* g) {
  if (a == nullptr || a->batch <= 0 || a->channels <= 0) return false;
  g->B = a->batch;
  g->C = a->channels;
  int64_t kvol = 1, L = 1, vol = 1;
  for (int d = 0; d < 3; ++d) {
    if (a->in_size[d] <= 0 || a->kernel[d] <= 0 || a->stride[d] <= 0 || a->padding[d] < 0 ||
        a->dilation[d] <= 0)
      return false;
    g->in[d] = a->in_size[d];
    g->ker[d] = a->kernel[d];
    g->str[d] = a->stride[d];
    g->pad[d] = a->padding[d];
    g->dil[d] = a->dilation[d];
    const int64_t o = conv_extent(a->in_size[d], a->kernel[d], a->stride[d], a->padding[d],
                                  a->dilation[d]);
    if (o <= 0 || o > 0x7fffffff) return false;
    g->out[d] = (int32_t)o;
    kvol *= a->kernel[d];
    L *= o;
    vol *= a->in_size[d];
    if (kvol > 0x7fffffff || vol > 0x7fffffff || L > 0x7fffffff) return false;
  }
  if (kvol * a->channels > 0x7fffffff) return false;
  g->kvol = (int32_t)kvol;
  g->L = L;
  g->K = kvol * a->channels;
  return true;
}

// Quotient and remainder of a small non-negative int by a run-time divisor through the fp32
// reciprocal (exact for a < 2^22 after one correction step): a handful of instructions instead
// of the ~40 of an integer division, which otherwise dominate the address arithmetic of these kernels.
struct SmallDiv {
  int32_t d;
  float inv;
  AHL_DEV int32_t quot(int32_t a) const {
    int32_t q = (int32_t)((float)a * inv);
    const int32_t r = a - q * d;
    if (r >= d) ++q;
    if (r < 0) --q;
    return q;
  }
};
static SmallDiv make_small_div(int32_t d) { return SmallDiv{d, 1.0f / (float)d}; }

// One thread gathers VEC consecutive patch entries (consecutive kernel offsets, carrying into
// the next kernel row / plane / channel) and writes them with one store. Threads of a wave walk
// along the patch, so the writes are contiguous; the reads of neighbouring offsets touch
// neighbouring input elements and mostly hit L2, since every input element is reused by up to
// kvol patches.
template <class E, int VEC>
__global__ __launch_bounds__(256) void k_im2col(const E* __restrict__ x, E* __restrict__ cols,
                                                int64_t ldc, ConvGeom g, int64_t groups_per_row,
                                                int64_t total) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  const int64_t m = idx / groups_per_row;
  const int32_t k0 = (int32_t)(idx - m * groups_per_row) * VEC;
  const int64_t b = m / g.L;
  int32_t l = (int32_t)(m - b * g.L);
  const int32_t ow = l % g.out[2];
  l /= g.out[2];
  const int32_t oh = l % g.out[1];
  const int32_t od = l / g.out[1];
  int32_t c = k0 / g.kvol;
  int32_t r = k0 - c * g.kvol;
  int32_t kw = r % g.ker[2];
  r /= g.ker[2];
  int32_t kh = r % g.ker[1];
  int32_t kd = r / g.ker[1];
  const int32_t id0 = od * g.str[0] - g.pad[0];
  const int32_t ih0 = oh * g.str[1] - g.pad[1];
  const int32_t iw0 = ow * g.str[2] - g.pad[2];
  const int64_t plane = (int64_t)g.in[1] * g.in[2];
  E v[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    E val = (E)0;
    if (k0 + j < g.K) {
      const int32_t id = id0 + kd * g.dil[0], ih = ih0 + kh * g.dil[1], iw = iw0 + kw * g.dil[2];
      if (id >= 0 && id < g.in[0] && ih >= 0 && ih < g.in[1] && iw >= 0 && iw < g.in[2])
        val = x[((b * g.C + c) * g.in[0] + id) * plane + (int64_t)ih * g.in[2] + iw];
    }
    v[j] = val;
    if (++kw == g.ker[2]) {
      kw = 0;
      if (++kh == g.ker[1]) {
        kh = 0;
        if (++kd == g.ker[0]) {
          kd = 0;
          ++c;
        }
      }
    }
  }
  E* dst = cols + m * ldc + k0;
  if constexpr (VEC * sizeof(E) == 16) {
    u32x4 pk;
    __builtin_memcpy(&pk, v, 16);
    *(u32x4*)dst = pk;
  } else {
#pragma unroll
    for (int j = 0; j < VEC; ++j)
      if (k0 + j < g.K) dst[j] = v[j];
  }
}

// Tiled variant for rows that can be written in 16-byte vectors: a block produces 64 patches x
// one 128-byte span of the patch dimension. Gather phase: each wave takes one patch entry
// (c, kd, kh, kw) at a time -- uniform over the wave -- and its 64 lanes read it for 64 consecutive
// patches, i.e. (for stride 1) 64 consecutive input elements: coalesced reads. The tile is turned
// in LDS (row stride of 33 words: conflict-free writes) and written out as row-contiguous
// 16-byte vectors.
template <class E>
__global__ __launch_bounds__(256) void k_im2col_tiled(const E* __restrict__ x, E* __restrict__ cols,
                                                      int64_t ldc, ConvGeom g, int64_t M,
                                                      int32_t k_tiles, SmallDiv by_ow, SmallDiv by_oh) {
  constexpr int KT = 128 / (int)sizeof(E);  // patch entries per tile: 64 bf16 or 32 fp32
  constexpr int EPV = 16 / (int)sizeof(E);  // entries per 16-byte vector
  constexpr int VPR = KT / EPV;             // vectors per tile row: 8
  __shared__ uint32_t tile[64 * 33];
  __shared__ int64_t first[2];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t m0 = (int64_t)(blockIdx.x / k_tiles) * 64;
  const int32_t k0 = (int32_t)(blockIdx.x % k_tiles) * KT;
  // (image, position) of the block's first patch: one 64-bit division per block; the lanes step
  // on from there with 32-bit arithmetic (positions per image < 2^22: checked by the launcher)
  if (tid == 0) {
    const int64_t b0 = m0 / g.L;
    first[0] = b0;
    first[1] = m0 - b0 * g.L;
  }
  __syncthreads();
  const bool mvalid = m0 + lane < M;
  int64_t b = first[0];
  int32_t l = (int32_t)first[1] + (mvalid ? lane : 0);
  const int32_t per_image = (int32_t)g.L;
  while (l >= per_image) { l -= per_image; b += 1; }
  const int32_t row = by_ow.quot(l);          // od * out[1] + oh
  const int32_t ow = l - row * g.out[2];
  const int32_t od = by_oh.quot(row);
  const int32_t oh = row - od * g.out[1];
  const int32_t id0 = od * g.str[0] - g.pad[0];
  const int32_t ih0 = oh * g.str[1] - g.pad[1];
  const int32_t iw0 = ow * g.str[2] - g.pad[2];
  const int64_t plane = (int64_t)g.in[1] * g.in[2];
  const E* xb = x + b * g.C * g.in[0] * plane;
  // element offset of this lane's patch origin inside its image (negative inside the padding);
  // the launcher has checked that one image has fewer than 2^31 elements
  const int32_t lane_off = (id0 * g.in[1] + ih0) * g.in[2] + iw0;
  E* trow = (E*)tile;
  constexpr int RS = 33 * 4 / (int)sizeof(E);  // tile row stride in entries
  // Per patch entry of the tile: its element offset inside an image relative to the patch origin
  // and its (kd, kh, kw) * dilation, decomposed once per block instead of once per load (three
  // integer divisions each); offset < 0 marks entries beyond K. The entry is the same for all
  // lanes of a wave, so the loop below reads it into scalar registers and the per-lane work is
  // one 32-bit add for the address and three range checks.
  __shared__ int32_t entry[KT][4];
  if (tid < KT) {
    const int32_t k = k0 + tid;
    int32_t off = -1, kd = 0, kh = 0, kw = 0;
    if (k < g.K) {
      const int32_t c = k / g.kvol;
      int32_t r = k - c * g.kvol;
      kw = (r % g.ker[2]) * g.dil[2];
      r /= g.ker[2];
      kh = (r % g.ker[1]) * g.dil[1];
      kd = (r / g.ker[1]) * g.dil[0];
      off = ((c * g.in[0] + kd) * g.in[1] + kh) * g.in[2] + kw;
    }
    entry[tid][0] = off;
    entry[tid][1] = kd;
    entry[tid][2] = kh;
    entry[tid][3] = kw;
  }
  __syncthreads();
  const uint32_t in0 = (uint32_t)g.in[0], in1 = (uint32_t)g.in[1], in2 = (uint32_t)g.in[2];
  // All loads of a wave are issued before the first value is used: entries outside the image
  // (or beyond K) read the image's first element instead and are zeroed afterwards, so there is
  // no branch that would make every load wait for the one before it.
  E vals[KT / 4];
#pragma unroll
  for (int i = 0; i < KT / 4; ++i) {
    const int kk = wave + 4 * i;
    const int32_t off = __builtin_amdgcn_readfirstlane(entry[kk][0]);
    const int32_t kd = __builtin_amdgcn_readfirstlane(entry[kk][1]);
    const int32_t kh = __builtin_amdgcn_readfirstlane(entry[kk][2]);
    const int32_t kw = __builtin_amdgcn_readfirstlane(entry[kk][3]);
    // unsigned compares fold the two-sided range checks into one each
    const bool ok = off >= 0 && (uint32_t)(id0 + kd) < in0 && (uint32_t)(ih0 + kh) < in1 &&
                    (uint32_t)(iw0 + kw) < in2;
    const E v = xb[ok ? lane_off + off : 0];
    vals[i] = ok ? v : (E)0;
  }
#pragma unroll
  for (int i = 0; i < KT / 4; ++i) trow[lane * RS + wave + 4 * i] = vals[i];
  __syncthreads();
  const int vcol = tid % VPR, vrow = tid / VPR;  // 32 rows per pass
#pragma unroll
  for (int pass = 0; pass < 2; ++pass) {
    const int p = vrow + 32 * pass;
    const int32_t k = k0 + vcol * EPV;
    if (m0 + p < M && k < g.K) {  // K is a multiple of EPV on this path
      const uint32_t* src = tile + p * 33 + vcol * 4;
      u32x4 v = {src[0], src[1], src[2], src[3]};
      *(u32x4*)(cols + (m0 + p) * ldc + k) = v;
    }
  }
}

// Adjoint of k_im2col as a gather: one thread per input element sums, in fp32 and in a fixed
// order (ascending kernel offset), the patch entries that were copied from it, and rounds once.
// No atomics, so the result is reproducible.
template <class D>
__global__ __launch_bounds__(256) void k_col2im(const void* __restrict__ dcols, int64_t ldc,
                                                ConvGeom g, void* __restrict__ dx, int64_t total) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  int64_t r = idx;
  const int32_t w = (int32_t)(r % g.in[2]);
  r /= g.in[2];
  const int32_t h = (int32_t)(r % g.in[1]);
  r /= g.in[1];
  const int32_t d = (int32_t)(r % g.in[0]);
  r /= g.in[0];
  const int32_t c = (int32_t)(r % g.C);
  const int64_t b = r / g.C;
  float acc = 0.f;
  for (int32_t kd = 0; kd < g.ker[0]; ++kd) {
    const int32_t td = d + g.pad[0] - kd * g.dil[0];
    if (td < 0 || td % g.str[0] != 0) continue;
    const int32_t od = td / g.str[0];
    if (od >= g.out[0]) continue;
    for (int32_t kh = 0; kh < g.ker[1]; ++kh) {
      const int32_t th = h + g.pad[1] - kh * g.dil[1];
      if (th < 0 || th % g.str[1] != 0) continue;
      const int32_t oh = th / g.str[1];
      if (oh >= g.out[1]) continue;
      for (int32_t kw = 0; kw < g.ker[2]; ++kw) {
        const int32_t tw = w + g.pad[2] - kw * g.dil[2];
        if (tw < 0 || tw % g.str[2] != 0) continue;
        const int32_t ow = tw / g.str[2];
        if (ow >= g.out[2]) continue;
        const int64_t l = ((int64_t)od * g.out[1] + oh) * g.out[2] + ow;
        const int64_t k = (int64_t)c * g.kvol + ((int64_t)kd * g.ker[1] + kh) * g.ker[2] + kw;
        acc += D::load(dcols, (b * g.L + l) * ldc + k);
      }
    }
  }
  D::store(dx, idx, acc);
}

// Tiled variant: a block computes a patch of rpb rows x cpb columns (rpb * cpb = 64; cpb is the
// smallest power of two that covers the image width, at most 64, so narrow images still fill
// the lanes) of one image plane for 8 channels. Every patch row that can contribute lies in a
// small window of output rows and a contiguous range of output columns; the block stages that
// window's entries of its 8 channels (8 * kvol contiguous entries per patch row, loaded as
// 16-byte vectors) in LDS once and then sums from LDS, in the same ascending kernel-offset order
// as k_col2im, so both give the same bits.
struct FoldPlan {
  int32_t cpb, rpb;   // columns and rows of the image patch of a block
  int32_t ow_span;    // staged output columns
  int32_t oh_span;    // staged output rows
  int32_t row_vecs;   // 16-byte vectors per staged patch row (8 * kvol entries)
  int32_t w_tiles, h_tiles;
  SmallDiv by_row_vecs, by_ow_span, by_oh_span, by_cpb, by_str[3];
};

template <class D>
__global__ __launch_bounds__(512) void k_col2im_tiled(const void* __restrict__ dcols, int64_t ldc,
                                                      ConvGeom g, FoldPlan fp,
                                                      void* __restrict__ dx) {
  typedef typename D::elem E;
  constexpr int EPV = D::EPV;
  extern __shared__ __attribute__((aligned(16))) char fold_lds[];
  const int tid = threadIdx.x;
  // block -> (image b, channel group, d, row tile, column tile)
  int64_t r = blockIdx.x;
  const int32_t wt = (int32_t)(r % fp.w_tiles);
  r /= fp.w_tiles;
  const int32_t ht = (int32_t)(r % fp.h_tiles);
  r /= fp.h_tiles;
  const int32_t d = (int32_t)(r % g.in[0]);
  r /= g.in[0];
  const int32_t cg = (int32_t)(r % (g.C / 8));
  const int64_t b = r / (g.C / 8);
  const int32_t w0 = wt * fp.cpb, h0 = ht * fp.rpb;
  const int32_t w_last = (w0 + fp.cpb - 1 < g.in[2] ? w0 + fp.cpb - 1 : g.in[2] - 1);
  const int32_t h_last = (h0 + fp.rpb - 1 < g.in[1] ? h0 + fp.rpb - 1 : g.in[1] - 1);
  // output columns / rows that can touch the patch: o = (i + pad - k * dil) / str
  int32_t ow_min = w0 + g.pad[2] - (g.ker[2] - 1) * g.dil[2];
  ow_min = ow_min <= 0 ? 0 : (ow_min + g.str[2] - 1) / g.str[2];
  int32_t ow_max = (w_last + g.pad[2]) / g.str[2];
  if (ow_max > g.out[2] - 1) ow_max = g.out[2] - 1;
  int32_t oh_min = h0 + g.pad[1] - (g.ker[1] - 1) * g.dil[1];
  oh_min = oh_min <= 0 ? 0 : (oh_min + g.str[1] - 1) / g.str[1];
  int32_t oh_max = (h_last + g.pad[1]) / g.str[1];
  if (oh_max > g.out[1] - 1) oh_max = g.out[1] - 1;
  const int32_t wspan = ow_max - ow_min + 1, hspan = oh_max - oh_min + 1;  // <= the plan's spans
  const int32_t row_bytes = fp.row_vecs * 16;
  const int32_t kbase = cg * 8 * g.kvol;       // first patch entry of the channel group
  // ---- stage: for every kd with a valid output plane, hspan x wspan patch rows ----
  const int32_t vec_total = g.ker[0] * fp.oh_span * fp.ow_span * fp.row_vecs;
  for (int32_t v = tid; v < vec_total; v += 512) {
    int32_t q = fp.by_row_vecs.quot(v);
    const int32_t vc = v - q * fp.row_vecs;
    int32_t q2 = fp.by_ow_span.quot(q);
    const int32_t oi = q - q2 * fp.ow_span;
    const int32_t kd = fp.by_oh_span.quot(q2);
    const int32_t hi = q2 - kd * fp.oh_span;
    const int32_t td = d + g.pad[0] - kd * g.dil[0];
    const int32_t od = td >= 0 ? fp.by_str[0].quot(td) : -1;
    if (oi < wspan && hi < hspan && od >= 0 && od * g.str[0] == td && od < g.out[0]) {
      const int64_t l = ((int64_t)od * g.out[1] + oh_min + hi) * g.out[2] + ow_min + oi;
      *(u32x4*)(fold_lds + (((int64_t)kd * fp.oh_span + hi) * fp.ow_span + oi) * row_bytes + vc * 16) =
          ld16((const E*)dcols + (b * g.L + l) * ldc + kbase + vc * EPV);
    }
  }
  __syncthreads();
  // ---- sum: thread = (channel tid / 64 of the group, pixel tid % 64 of the patch) ----
  const int32_t pix = tid & 63, cl = tid >> 6;
  const int32_t prow = fp.by_cpb.quot(pix);
  const int32_t w = w0 + pix - prow * fp.cpb, h = h0 + prow;
  if (w >= g.in[2] || h >= g.in[1]) return;
  float acc = 0.f;
  for (int32_t kd = 0; kd < g.ker[0]; ++kd) {
    const int32_t td = d + g.pad[0] - kd * g.dil[0];
    if (td < 0) continue;
    const int32_t od = fp.by_str[0].quot(td);
    if (od * g.str[0] != td || od >= g.out[0]) continue;
    for (int32_t kh = 0; kh < g.ker[1]; ++kh) {
      const int32_t th = h + g.pad[1] - kh * g.dil[1];
      if (th < 0) continue;
      const int32_t oh = fp.by_str[1].quot(th);
      if (oh * g.str[1] != th || oh >= g.out[1]) continue;
      const char* rows = fold_lds +
          (((int64_t)kd * fp.oh_span + (oh - oh_min)) * fp.ow_span) * row_bytes;
      for (int32_t kw = 0; kw < g.ker[2]; ++kw) {
        const int32_t tw = w + g.pad[2] - kw * g.dil[2];
        if (tw < 0) continue;
        const int32_t ow = fp.by_str[2].quot(tw);
        if (ow * g.str[2] != tw || ow >= g.out[2]) continue;
        const int32_t k = cl * g.kvol + (kd * g.ker[1] + kh) * g.ker[2] + kw;
        acc += D::load(rows + (int64_t)(ow - ow_min) * row_bytes, k);
      }
    }
  }
  const int64_t plane = (int64_t)g.in[1] * g.in[2];
  D::store(dx, (((b * g.C + cg * 8 + cl) * g.in[0] + d) * plane) + (int64_t)h * g.in[2] + w, acc);
}

// Wide variant: the image patch of a block has 256 pixels (rpb * cpb = 256) and a thread owns one
// pixel for all 8 channels of the group, so the index arithmetic of a kernel offset (which output
// position, whether it exists, where its staged row lies) is done once for 8 sums, and the halo
// of staged output rows is shared by four times as many image rows. Same staging layout, same
// ascending kernel-offset order and fp32 sums as above: the same bits.
template <class D>
__global__ __launch_bounds__(256) void k_col2im_wide(const void* __restrict__ dcols, int64_t ldc,
                                                     ConvGeom g, FoldPlan fp,
                                                     void* __restrict__ dx) {
  typedef typename D::elem E;
  constexpr int EPV = D::EPV;
  extern __shared__ __attribute__((aligned(16))) char fold_lds[];
  const int tid = threadIdx.x;
  int64_t r = blockIdx.x;
  const int32_t wt = (int32_t)(r % fp.w_tiles);
  r /= fp.w_tiles;
  const int32_t ht = (int32_t)(r % fp.h_tiles);
  r /= fp.h_tiles;
  const int32_t d = (int32_t)(r % g.in[0]);
  r /= g.in[0];
  const int32_t cg = (int32_t)(r % (g.C / 8));
  const int64_t b = r / (g.C / 8);
  const int32_t w0 = wt * fp.cpb, h0 = ht * fp.rpb;
  const int32_t w_last = (w0 + fp.cpb - 1 < g.in[2] ? w0 + fp.cpb - 1 : g.in[2] - 1);
  const int32_t h_last = (h0 + fp.rpb - 1 < g.in[1] ? h0 + fp.rpb - 1 : g.in[1] - 1);
  int32_t ow_min = w0 + g.pad[2] - (g.ker[2] - 1) * g.dil[2];
  ow_min = ow_min <= 0 ? 0 : (ow_min + g.str[2] - 1) / g.str[2];
  int32_t ow_max = (w_last + g.pad[2]) / g.str[2];
  if (ow_max > g.out[2] - 1) ow_max = g.out[2] - 1;
  int32_t oh_min = h0 + g.pad[1] - (g.ker[1] - 1) * g.dil[1];
  oh_min = oh_min <= 0 ? 0 : (oh_min + g.str[1] - 1) / g.str[1];
  int32_t oh_max = (h_last + g.pad[1]) / g.str[1];
  if (oh_max > g.out[1] - 1) oh_max = g.out[1] - 1;
  const int32_t wspan = ow_max - ow_min + 1, hspan = oh_max - oh_min + 1;  // <= the plan's spans
  const int32_t row_bytes = fp.row_vecs * 16;
  const int32_t kbase = cg * 8 * g.kvol;
  // ---- stage. Four vectors per thread and round, all loaded before the first is stored: slots
  // without data load the image's first patch row instead and are dropped, so no load waits
  // behind a branch ----
  const int32_t vec_total = g.ker[0] * fp.oh_span * fp.ow_span * fp.row_vecs;
  constexpr int kStageUnroll = 4;
  const E* img = (const E*)dcols + b * g.L * ldc + kbase;
  for (int32_t v0 = tid; v0 < vec_total; v0 += 256 * kStageUnroll) {
    u32x4 val[kStageUnroll];
    int32_t dst[kStageUnroll];
#pragma unroll
    for (int u = 0; u < kStageUnroll; ++u) {
      const int32_t v = v0 + 256 * u;
      const int32_t q = fp.by_row_vecs.quot(v);
      const int32_t vc = v - q * fp.row_vecs;
      const int32_t q2 = fp.by_ow_span.quot(q);
      const int32_t oi = q - q2 * fp.ow_span;
      const int32_t kd = fp.by_oh_span.quot(q2);
      const int32_t hi = q2 - kd * fp.oh_span;
      const int32_t td = d + g.pad[0] - kd * g.dil[0];
      const int32_t od = td >= 0 ? fp.by_str[0].quot(td) : -1;
      const bool ok = v < vec_total && oi < wspan && hi < hspan && od >= 0 &&
                      od * g.str[0] == td && od < g.out[0];
      const int64_t l = ok ? ((int64_t)od * g.out[1] + oh_min + hi) * g.out[2] + ow_min + oi : 0;
      val[u] = ld16(img + l * ldc + (ok ? vc : 0) * EPV);
      dst[u] = ok ? (((kd * fp.oh_span + hi) * fp.ow_span + oi) * row_bytes + vc * 16) : -1;
    }
#pragma unroll
    for (int u = 0; u < kStageUnroll; ++u)
      if (dst[u] >= 0) *(u32x4*)(fold_lds + dst[u]) = val[u];
  }
  __syncthreads();
  // ---- sum: thread = pixel tid of the patch, 8 channels ----
  const int32_t prow = fp.by_cpb.quot(tid);
  const int32_t w = w0 + tid - prow * fp.cpb, h = h0 + prow;
  if (w >= g.in[2] || h >= g.in[1]) return;
  float acc[8];
#pragma unroll
  for (int c = 0; c < 8; ++c) acc[c] = 0.f;
  for (int32_t kd = 0; kd < g.ker[0]; ++kd) {
    const int32_t td = d + g.pad[0] - kd * g.dil[0];
    if (td < 0) continue;
    const int32_t od = fp.by_str[0].quot(td);
    if (od * g.str[0] != td || od >= g.out[0]) continue;
    for (int32_t kh = 0; kh < g.ker[1]; ++kh) {
      const int32_t th = h + g.pad[1] - kh * g.dil[1];
      if (th < 0) continue;
      const int32_t oh = fp.by_str[1].quot(th);
      if (oh * g.str[1] != th || oh >= g.out[1]) continue;
      const char* rows = fold_lds + ((kd * fp.oh_span + (oh - oh_min)) * fp.ow_span) * row_bytes;
      for (int32_t kw = 0; kw < g.ker[2]; ++kw) {
        const int32_t tw = w + g.pad[2] - kw * g.dil[2];
        if (tw < 0) continue;
        const int32_t ow = fp.by_str[2].quot(tw);
        if (ow * g.str[2] != tw || ow >= g.out[2]) continue;
        const char* row = rows + (ow - ow_min) * row_bytes;
        const int32_t k = (kd * g.ker[1] + kh) * g.ker[2] + kw;
#pragma unroll
        for (int c = 0; c < 8; ++c) acc[c] += D::load(row, c * g.kvol + k);
      }
    }
  }
  const int64_t plane = (int64_t)g.in[1] * g.in[2];
  const int64_t o = (((b * g.C + cg * 8) * g.in[0] + d) * plane) + (int64_t)h * g.in[2] + w;
#pragma unroll
  for (int c = 0; c < 8; ++c) D::store(dx, o + c * g.in[0] * plane, acc[c]);
}

// dst[b][c][r] = src[b][r][c]; 32 x 32 tiles through LDS (padded against bank conflicts) so that
// both the reads and the writes are contiguous.
template <class E>
__global__ __launch_bounds__(256) void k_transpose_batched(const E* __restrict__ src,
                                                           int64_t ld_src, int64_t rows,
                                                           int64_t cols, E* __restrict__ dst,
                                                           int64_t ld_dst, int64_t tiles_c,
                                                           int64_t tiles_per_mat) {
  __shared__ E tile[32][33];
  const int64_t bid = blockIdx.x;
  const int64_t b = bid / tiles_per_mat;
  const int64_t t = bid - b * tiles_per_mat;
  const int64_t r0 = (t / tiles_c) * 32, c0 = (t % tiles_c) * 32;
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
  const E* s = src + b * rows * ld_src;
  E* d = dst + b * cols * ld_dst;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int64_t rr = r0 + ty + 8 * i, cc = c0 + tx;
    if (rr < rows && cc < cols) tile[ty + 8 * i][tx] = s[rr * ld_src + cc];
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int64_t cc = c0 + ty + 8 * i, rr = r0 + tx;
    if (rr < rows && cc < cols) d[cc * ld_dst + rr] = tile[tx][ty + 8 * i];
  }
}

// Vector variant for matrices whose rows and columns come in whole 16-byte vectors: 64 x 64
// tiles, 16-byte loads along the source rows into LDS, and every thread gathers the V elements
// of one destination vector (V consecutive source rows of one column) from LDS, so that both
// sides of HBM see 16-byte accesses, 128 contiguous bytes per 8 (bf16) or 16 (fp32) lanes.
template <class E>
__global__ __launch_bounds__(256) void k_transpose_vec(const E* __restrict__ src, int64_t ld_src,
                                                       int64_t rows, int64_t cols,
                                                       E* __restrict__ dst, int64_t ld_dst,
                                                       int64_t tiles_c, int64_t tiles_per_mat) {
  constexpr int V = 16 / (int)sizeof(E);   // elements per vector
  constexpr int T = 64;                    // tile edge
  constexpr int VPR = T / V;               // vectors per tile row
  constexpr int RS = T + V;                // LDS row stride in elements (a multiple of 16 bytes)
  __shared__ __attribute__((aligned(16))) E tile[T * RS];
  const int64_t bid = blockIdx.x;
  const int64_t b = bid / tiles_per_mat;
  const int64_t t = bid - b * tiles_per_mat;
  const int64_t r0 = (t / tiles_c) * T, c0 = (t % tiles_c) * T;
  const E* s = src + b * rows * ld_src;
  E* d = dst + b * cols * ld_dst;
  const int tid = threadIdx.x;
  u32x4 raw[T * VPR / 256];
#pragma unroll
  for (int i = 0; i < T * VPR / 256; ++i) {
    const int v = tid + 256 * i;
    const int r = v / VPR, cv = v % VPR;
    raw[i] = u32x4{0u, 0u, 0u, 0u};
    if (r0 + r < rows && c0 + cv * V < cols) raw[i] = ld16(s + (r0 + r) * ld_src + c0 + cv * V);
  }
#pragma unroll
  for (int i = 0; i < T * VPR / 256; ++i) {
    const int v = tid + 256 * i;
    *(u32x4*)(tile + (v / VPR) * RS + (v % VPR) * V) = raw[i];
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < T * VPR / 256; ++i) {
    const int v = tid + 256 * i;
    const int c = v / VPR, rv = v % VPR;     // destination row c, vector rv of its 64 elements
    if (c0 + c >= cols || r0 + rv * V >= rows) continue;
    E out[V];
#pragma unroll
    for (int e = 0; e < V; ++e) out[e] = tile[(rv * V + e) * RS + c];
    st16(d + (c0 + c) * ld_dst + r0 + rv * V, *(const u32x4*)out);
  }
}

template <class E, int VEC>
static int launch_im2col(const void* x, void* cols, int64_t ldc, const ConvGeom& g,
                         hipStream_t st) {
  const int64_t M = (int64_t)g.B * g.L;
  const int64_t gpr = cdiv(g.K, VEC);
  const int64_t total = M * gpr;
  const int64_t blocks = cdiv(total, 256);
  if (blocks > 0x7fffffff) return AHL_ERR_UNSUPPORTED;
  hipLaunchKernelGGL((k_im2col<E, VEC>), dim3((unsigned)blocks), dim3(256), 0, st, (const E*)x,
                     (E*)cols, ldc, g, gpr, total);
  return check_launch("k_im2col");
}

}  // namespace ahl

using namespace ahl;

extern "C" int ahl_conv_out_size(const AhlConvGeom* geom, int32_t* out_size) {
  ConvGeom g;
  if (out_size == nullptr || !make_geom(geom, &g)) return AHL_ERR_ARG;
  for (int d = 0; d < 3; ++d) out_size[d] = g.out[d];
  return AHL_OK;
}

template <class E>
static int launch_im2col_tiled(const void* x, void* cols, int64_t ldc, const ConvGeom& g,
                               hipStream_t st) {
  constexpr int KT = 128 / (int)sizeof(E);
  const int64_t M = (int64_t)g.B * g.L;
  const int64_t k_tiles = cdiv(g.K, KT);
  const int64_t blocks = cdiv(M, 64) * k_tiles;
  if (blocks > 0x7fffffff) return AHL_ERR_UNSUPPORTED;
  hipLaunchKernelGGL((k_im2col_tiled<E>), dim3((unsigned)blocks), dim3(256), 0, st, (const E*)x,
                     (E*)cols, ldc, g, M, (int32_t)k_tiles, make_small_div(g.out[2]),
                     make_small_div(g.out[1]));
  return check_launch("k_im2col_tiled");
}

extern "C" int ahl_im2col(const void* x, const AhlConvGeom* geom, int32_t dtype, void* cols,
                          int64_t ldc, void* stream) {
  ConvGeom g;
  if (x == nullptr || cols == nullptr || !make_geom(geom, &g) || ldc < g.K) return AHL_ERR_ARG;
  hipStream_t st = (hipStream_t)stream;
  // the tiled kernel addresses the elements of one image with 32-bit offsets
  // and the positions of one image with the fp32-reciprocal division
  const bool small_image = (int64_t)g.C * g.in[0] * g.in[1] * g.in[2] <= 0x3fffffff && g.L < (1 << 22);
  if (dtype == AHL_F16) dtype = AHL_BF16;   // patch extraction moves 2-byte elements, whatever they hold
  if (dtype == AHL_F32) {
    if (g.K % 4 == 0 && ldc % 4 == 0 && aligned16(cols) && small_image)
      return launch_im2col_tiled<uint32_t>(x, cols, ldc, g, st);
    return launch_im2col<uint32_t, 1>(x, cols, ldc, g, st);
  }
  if (dtype == AHL_BF16) {
    if (g.K % 8 == 0 && ldc % 8 == 0 && aligned16(cols) && small_image)
      return launch_im2col_tiled<uint16_t>(x, cols, ldc, g, st);
    return launch_im2col<uint16_t, 1>(x, cols, ldc, g, st);
  }
  return AHL_ERR_ARG;
}

extern "C" int ahl_col2im(const void* dcols, int64_t ldc, const AhlConvGeom* geom, int32_t dtype,
                          void* dx, void* stream) {
  ConvGeom g;
  if (dcols == nullptr || dx == nullptr || !make_geom(geom, &g) || ldc < g.K) return AHL_ERR_ARG;
  const int64_t total = (int64_t)g.B * g.C * g.in[0] * g.in[1] * g.in[2];
  // tiled kernels: channel groups of 8 whose 8 * kvol patch entries are whole 16-byte vectors;
  // first the plan with 256 pixels per block, then (if its staging area does not fit) 64
  for (int pixels = 256; pixels >= 64; pixels /= 4) {
    const int epv = dtype == AHL_F32 ? 4 : 8;
    const int64_t row_entries = 8 * (int64_t)g.kvol;
    int32_t cpb = 64;
    while (cpb > 8 && cpb / 2 >= g.in[2]) cpb /= 2;
    const int32_t rpb = pixels / cpb;
    // widest window of output columns / rows that one block's image patch can reach
    int64_t ow_span = (cpb - 1 + (int64_t)(g.ker[2] - 1) * g.dil[2]) / g.str[2] + 2;
    int64_t oh_span = (rpb - 1 + (int64_t)(g.ker[1] - 1) * g.dil[1]) / g.str[1] + 2;
    if (ow_span > g.out[2]) ow_span = g.out[2];
    if (oh_span > g.out[1]) oh_span = g.out[1];
    const int64_t lds_limit = pixels == 256 ? 64 * 1024 : 96 * 1024;
    const int64_t lds_bytes = (int64_t)g.ker[0] * oh_span * ow_span * row_entries * dtype_bytes(dtype);
    const int64_t w_tiles = cdiv(g.in[2], cpb), h_tiles = cdiv(g.in[1], rpb);
    const int64_t tblocks = (int64_t)g.B * (g.C / 8) * g.in[0] * h_tiles * w_tiles;
    if (dtype_known(dtype) && g.C % 8 == 0 && row_entries % epv == 0 &&
        ldc % epv == 0 && aligned16(dcols) && lds_bytes <= lds_limit && tblocks <= 0x7fffffff &&
        g.in[0] + g.pad[0] < (1 << 22) && g.in[1] + g.pad[1] < (1 << 22) &&
        g.in[2] + g.pad[2] < (1 << 22)) {
      FoldPlan fp{cpb, rpb, (int32_t)ow_span, (int32_t)oh_span, (int32_t)(row_entries / epv),
                  (int32_t)w_tiles, (int32_t)h_tiles,
                  make_small_div((int32_t)(row_entries / epv)), make_small_div((int32_t)ow_span),
                  make_small_div((int32_t)oh_span), make_small_div(cpb),
                  {make_small_div(g.str[0]), make_small_div(g.str[1]), make_small_div(g.str[2])}};
      AHL_DISPATCH_DTYPE(dtype, {
        // a refusal of the LDS size shows at the launch that follows (check_launch)
        if (pixels == 256) {
          (void)hipFuncSetAttribute((const void*)k_col2im_wide<D>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
          hipLaunchKernelGGL((k_col2im_wide<D>), dim3((unsigned)tblocks), dim3(256), (size_t)lds_bytes,
                             (hipStream_t)stream, dcols, ldc, g, fp, dx);
        } else {
          (void)hipFuncSetAttribute((const void*)k_col2im_tiled<D>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
          hipLaunchKernelGGL((k_col2im_tiled<D>), dim3((unsigned)tblocks), dim3(512), (size_t)lds_bytes,
                             (hipStream_t)stream, dcols, ldc, g, fp, dx);
        }
      });
      return check_launch("k_col2im_tiled");
    }
  }
  const int64_t blocks = cdiv(total, 256);
  if (blocks > 0x7fffffff) return AHL_ERR_UNSUPPORTED;
  AHL_DISPATCH_DTYPE(dtype, {
    hipLaunchKernelGGL((k_col2im<D>), dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                       dcols, ldc, g, dx, total);
  });
  return check_launch("k_col2im");
}

extern "C" int ahl_transpose_batched(const void* src, int64_t ld_src, int32_t dtype, int64_t batch,
                                     int64_t rows, int64_t cols, void* dst, int64_t ld_dst,
                                     void* stream) {
  if (src == nullptr || dst == nullptr || batch <= 0 || rows <= 0 || cols <= 0 || ld_src < cols ||
      ld_dst < rows)
    return AHL_ERR_ARG;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == AHL_F16) dtype = AHL_BF16;   // a transposition moves 2-byte elements, whatever they hold
  if (dtype != AHL_F32 && dtype != AHL_BF16) return AHL_ERR_ARG;
  {
    // whole 16-byte vectors on both sides: the vector kernel
    const int64_t v = dtype == AHL_BF16 ? 8 : 4;
    const int64_t tiles_c = cdiv(cols, 64), per_mat = tiles_c * cdiv(rows, 64);
    if (rows % v == 0 && cols % v == 0 && ld_src % v == 0 && ld_dst % v == 0 && aligned16(src) &&
        aligned16(dst) && per_mat <= 0x7fffffff && batch <= 0x7fffffff / per_mat) {
      const dim3 vgrid((unsigned)(per_mat * batch));
      if (dtype == AHL_F32)
        hipLaunchKernelGGL((k_transpose_vec<uint32_t>), vgrid, dim3(256), 0, st,
                           (const uint32_t*)src, ld_src, rows, cols, (uint32_t*)dst, ld_dst,
                           tiles_c, per_mat);
      else
        hipLaunchKernelGGL((k_transpose_vec<uint16_t>), vgrid, dim3(256), 0, st,
                           (const uint16_t*)src, ld_src, rows, cols, (uint16_t*)dst, ld_dst,
                           tiles_c, per_mat);
      return check_launch("k_transpose_vec");
    }
  }
  const int64_t tiles_c = cdiv(cols, 32), tiles_r = cdiv(rows, 32);
  const int64_t per_mat = tiles_c * tiles_r;
  if (per_mat > 0x7fffffff || batch > 0x7fffffff / per_mat) return AHL_ERR_UNSUPPORTED;
  const dim3 grid((unsigned)(per_mat * batch));
  if (dtype == AHL_F32) {
    hipLaunchKernelGGL((k_transpose_batched<uint32_t>), grid, dim3(256), 0, st,
                       (const uint32_t*)src, ld_src, rows, cols, (uint32_t*)dst, ld_dst, tiles_c,
                       per_mat);
  } else if (dtype == AHL_BF16) {
    hipLaunchKernelGGL((k_transpose_batched<uint16_t>), grid, dim3(256), 0, st,
                       (const uint16_t*)src, ld_src, rows, cols, (uint16_t*)dst, ld_dst, tiles_c,
                       per_mat);
  } else {
    return AHL_ERR_ARG;
  }
  return check_launch("k_transpose_batched");
}
