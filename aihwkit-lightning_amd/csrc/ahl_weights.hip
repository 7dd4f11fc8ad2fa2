// Weight-side kernels: per-tile per-channel abs-max, on-the-fly quantisation and Gaussian weight
// noise into a scratch copy, and the in-place post-training quantisation.
#include "ahl_host.h"
#include "ahl_reduce_kernels.h"

namespace ahl {

// Quantiser of one (tile, channel) or one tile: the arithmetic of UniformQuantize called from
// clip_and_quantize (reference torch_utils/quant_utils.py:204-233 and :63-99) with bound = 1.0,
// res = scaling factors, max_quant_state = n_states / 2.
struct WQuant {
  float step;  // res after "alpha / res or alpha * res" and the zero fix
  float rc;    // max(step, tiny)
  float rcp;   // 1 / rc
};

template <class D>
AHL_DEV WQuant make_wquant(float wm, float n_states, bool all_gt1) {
  const float sc = D::rd(__fdiv_rn(wm, n_states));
  WQuant q;
  q.step = all_gt1 ? D::rd(__fdiv_rn(2.0f, sc)) : D::rd(2.0f * sc);
  if (q.step == 0.0f) q.step = 1.0f;
  q.rc = fmaxf(q.step, D::tiny());
  q.rcp = __fdiv_rn(1.0f, q.rc);
  return q;
}

template <class D>
AHL_DEV float wquant_apply(float w, const WQuant& q, float maxq, bool round = true) {
  float v = D::rd(D::div_exact_rcp(w, q.rc, q.rcp));
  v = fminf(fmaxf(v, -maxq), maxq);
  if (round) v = rintf(v);
  return D::rd(v * q.step);
}

// Step of the learnable clip without a quantiser (UniformQuantize with res = clip, bound 0.5):
// alpha = 1, so the step is the clip itself, or its inverse if every clip of the tile is > 1.
template <class D>
AHL_DEV WQuant make_wclip(float clip, bool all_gt1) {
  WQuant q;
  q.step = all_gt1 ? D::rd(__fdiv_rn(1.0f, clip)) : clip;
  if (q.step == 0.0f) q.step = 1.0f;
  q.rc = fmaxf(q.step, D::tiny());
  q.rcp = __fdiv_rn(1.0f, q.rc);
  return q;
}

struct ModArgs {
  const void* w;
  int64_t N, K, ld;
  Tiling tl;
  const void* wmax;       // dtype [T, N]
  const float* tile_max;  // [T]
  const float* tile_min;  // [T]
  void* w_eff;            // dtype [N, K] (may alias w for the in-place quantiser) or null
  int64_t ld_eff;
  int32_t quant_type, noise_type;
  float n_states, maxq, std_dev;
  uint64_t seed, offset;
  const uint64_t* seed_state;  // null, or device {key, call counter} that replaces seed / offset
};

// One thread per group of 8 consecutive inputs of one channel (one Philox call gives the 8
// normals of the group); consecutive threads walk along the row, so that with VEC every wave
// reads and writes contiguous 16-byte vectors. A group lies in at most two tiles when tiles are
// at least 7 inputs wide; NARROW (narrower tiles) looks the tile up element by element.
template <class D, bool VEC, bool NARROW = false>
__global__ __launch_bounds__(256) void k_weight_modify(ModArgs a, uint32_t blocks_per_row) {
  const int64_t n = blockIdx.x / blocks_per_row;
  const int32_t kb = (int32_t)((blockIdx.x % blocks_per_row) * 256 + threadIdx.x) * 8;
  if (kb >= a.K) return;
  const int32_t klast = kb + 7 < a.K ? kb + 7 : (int32_t)a.K - 1;
  const bool modify = a.quant_type != AHL_QUANT_NONE || a.noise_type != AHL_NOISE_NONE;

  float v[8];
  const typename D::elem* src = (const typename D::elem*)a.w + n * a.ld + kb;
  if (VEC) {
#pragma unroll
    for (int q = 0; q < 8 / D::EPV; ++q) D::unpack(ld16(src + q * D::EPV), v + q * D::EPV);
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = kb + e < a.K ? D::load(a.w, n * a.ld + kb + e) : 0.0f;
  }

  if (modify) {
    float xi[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (a.noise_type != AHL_NOISE_NONE) {
      const NoiseKey nk = noise_key(a.seed, a.offset, a.seed_state);
      normal8(nk.seed, nk.offset, 1u << 24, (uint32_t)(kb >> 3), (uint32_t)n, xi);
    }
    // constants of a tile for this channel
    struct TileConst { WQuant q; float nstd; };
    auto tile_const = [&](int t) {
      TileConst c;
      const float wm = D::load(a.wmax, (int64_t)t * a.N + n);
      const float tmax = a.tile_max[t];
      c.q.step = 1.0f; c.q.rc = 1.0f; c.q.rcp = 1.0f;
      if (a.quant_type == AHL_QUANT_DISCRETIZE_PER_CHANNEL) {
        const bool all_gt1 = D::rd(__fdiv_rn(a.tile_min[t], a.n_states)) > 1.0f;
        c.q = make_wquant<D>(wm, a.n_states, all_gt1);
      } else if (a.quant_type == AHL_QUANT_DISCRETIZE) {
        const bool all_gt1 = D::rd(__fdiv_rn(tmax, a.n_states)) > 1.0f;
        c.q = make_wquant<D>(tmax, a.n_states, all_gt1);
      } else if (a.quant_type == AHL_QUANT_CLIP_LEARNED) {
        c.q = make_wclip<D>(wm, a.tile_min[t] > 1.0f);
      }
      c.nstd = D::rd(a.std_dev * (a.noise_type == AHL_NOISE_ADD_NORMAL_PER_CHANNEL ? wm : tmax));
      return c;
    };
    const int t0 = a.tl.tile_of(kb), t1 = a.tl.tile_of(klast);
    TileConst c = tile_const(t0);
    const int32_t t1_start = t1 != t0 ? a.tl.start(t1) : 0x7fffffff;
    const TileConst c1 = !NARROW && t1 != t0 ? tile_const(t1) : c;
    int tn = t0;                              // NARROW: the tile of element e, walked along
    int32_t tn_end = a.tl.start(t0 + 1);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      if (NARROW && kb + e >= tn_end && kb + e <= klast) {
        ++tn;
        tn_end = a.tl.start(tn + 1);
        c = tile_const(tn);
      }
      const TileConst& ce = !NARROW && kb + e >= t1_start ? c1 : c;
      float x = v[e];
      if (a.quant_type != AHL_QUANT_NONE)
        x = wquant_apply<D>(x, ce.q, a.maxq, a.quant_type != AHL_QUANT_CLIP_LEARNED);
      if (a.noise_type != AHL_NOISE_NONE) x = D::rd(x + D::rd(ce.nstd * D::rd(xi[e])));
      v[e] = x;
    }
  }

  if (!a.w_eff) return;
  typename D::elem* dst = (typename D::elem*)a.w_eff + n * a.ld_eff + kb;
  if (VEC) {
#pragma unroll
    for (int q = 0; q < 8 / D::EPV; ++q) st16(dst + q * D::EPV, D::pack(v + q * D::EPV));
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e)
      if (kb + e < a.K) D::store(a.w_eff, n * a.ld_eff + kb + e, v[e]);
  }
}

// Abs-max and per-channel weight noise in one pass over W, for the common training
// configuration (no quantiser, noise scaled by the channel's own maximum): one wave per (channel,
// tile) reads its segment as 16-byte vectors, reduces the maximum, writes wmax[t, n] and then
// the noisy copy -- from registers for segments of up to 1024 inputs, else from a second
// (cache-resident) read. Same Philox counters and the same arithmetic as k_weight_modify.
template <class D>
__global__ __launch_bounds__(256) void k_weight_prep_rows(ModArgs a, void* __restrict__ wmax_out) {
  constexpr int E = D::EPV;       // elements per 16-byte vector
  constexpr int VPG = 8 / E;      // vectors per group of 8 inputs (one Philox call)
  const int lane = threadIdx.x & 63;
  const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int64_t n = wave / a.tl.n_tiles;
  const int32_t t = (int32_t)(wave % a.tl.n_tiles);
  if (n >= a.N) return;
  const int32_t g0 = a.tl.start(t) >> 3, g1 = a.tl.start(t + 1) >> 3;  // groups of 8 inputs
  const typename D::elem* row = (const typename D::elem*)a.w + n * a.ld;
  typename D::elem* dst = (typename D::elem*)a.w_eff + n * a.ld_eff;
  float keep[2][8];
  float mx = 0.0f;
  int it = 0;
  for (int32_t g = g0 + lane; g < g1; g += 64, ++it) {
    float v[8];
#pragma unroll
    for (int q = 0; q < VPG; ++q) D::unpack(ld16(row + (int64_t)g * 8 + q * E), v + q * E);
#pragma unroll
    for (int e = 0; e < 8; ++e) mx = fmaxf(mx, fabsf(v[e]));
    if (it < 2) {
#pragma unroll
      for (int e = 0; e < 8; ++e) keep[it][e] = v[e];
    }
  }
  mx = wave_max(mx);
  if (lane == 0) D::store(wmax_out, (int64_t)t * a.N + n, mx);
  const float nstd = D::rd(a.std_dev * D::rd(mx));
  const NoiseKey nk = noise_key(a.seed, a.offset, a.seed_state);
  it = 0;
  for (int32_t g = g0 + lane; g < g1; g += 64, ++it) {
    float v[8], xi[8];
    if (it < 2) {
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = keep[it][e];
    } else {
#pragma unroll
      for (int q = 0; q < VPG; ++q) D::unpack(ld16(row + (int64_t)g * 8 + q * E), v + q * E);
    }
    normal8(nk.seed, nk.offset, 1u << 24, (uint32_t)g, (uint32_t)n, xi);
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = D::rd(v[e] + D::rd(nstd * D::rd(xi[e])));
#pragma unroll
    for (int q = 0; q < VPG; ++q) st16(dst + (int64_t)g * 8 + q * E, D::pack(v + q * E));
  }
}

// Abs-max and the per-channel quantiser in one pass over W: one wave per (channel, tile) reduces
// the maximum of its segment, writes wmax[t, n] and quantises the segment with its own scale --
// from registers for segments of up to 1024 inputs, else from a second (cache-resident) read.
// The reference's resolution convention switches to "number of states" when EVERY scale of the
// tile exceeds one; a wave whose own scale does not knows the switch is off. The others (weights
// beyond the number of states: rare) leave their segment to k_quantize_finish, which runs after
// the tile minima are known. Same arithmetic as k_weight_modify; in place or not.
template <class D>
AHL_DEV bool quantize_deferred(float mx, float n_states) {
  return D::rd(__fdiv_rn(mx, n_states)) > 1.0f;
}

// Quantises segment (n, t) with the scale of its abs-max mx. `keep`: the first two vectors per
// lane if the caller still holds them, else null (they are read again).
template <class D>
AHL_DEV void quantize_segment(const ModArgs& a, int64_t n, int32_t t, float mx, bool all_gt1, int lane,
                              const float (*keep)[8]) {
  constexpr int E = D::EPV;
  constexpr int VPG = 8 / E;
  const int32_t g0 = a.tl.start(t) >> 3, g1 = a.tl.start(t + 1) >> 3;
  const typename D::elem* row = (const typename D::elem*)a.w + n * a.ld;
  typename D::elem* dst = (typename D::elem*)a.w_eff + n * a.ld_eff;
  const WQuant q = make_wquant<D>(D::rd(mx), a.n_states, all_gt1);
  int it = 0;
  for (int32_t g = g0 + lane; g < g1; g += 64, ++it) {
    float v[8];
    if (keep != nullptr && it < 2) {
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = keep[it][e];
    } else {
#pragma unroll
      for (int qv = 0; qv < VPG; ++qv) D::unpack(ld16(row + (int64_t)g * 8 + qv * E), v + qv * E);
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = wquant_apply<D>(v[e], q, a.maxq);
#pragma unroll
    for (int qv = 0; qv < VPG; ++qv) st16_stream(dst + (int64_t)g * 8 + qv * E, D::pack(v + qv * E));
  }
}

template <class D>
__global__ __launch_bounds__(256) void k_quantize_rows(ModArgs a, void* __restrict__ wmax_io) {
  constexpr int E = D::EPV;
  constexpr int VPG = 8 / E;
  const int lane = threadIdx.x & 63;
  const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int64_t n = wave / a.tl.n_tiles;
  const int32_t t = (int32_t)(wave % a.tl.n_tiles);
  if (n >= a.N) return;
  const int32_t g0 = a.tl.start(t) >> 3, g1 = a.tl.start(t + 1) >> 3;
  const typename D::elem* row = (const typename D::elem*)a.w + n * a.ld;
  float keep[2][8];
  float mx = 0.0f;
  int it = 0;
  for (int32_t g = g0 + lane; g < g1; g += 64, ++it) {
    float v[8];
#pragma unroll
    for (int q = 0; q < VPG; ++q) D::unpack(ld16_stream(row + (int64_t)g * 8 + q * E), v + q * E);
#pragma unroll
    for (int e = 0; e < 8; ++e) mx = fmaxf(mx, fabsf(v[e]));
    if (it < 2) {
#pragma unroll
      for (int e = 0; e < 8; ++e) keep[it][e] = v[e];
    }
  }
  mx = wave_max(mx);
  if (lane == 0) D::store(wmax_io, (int64_t)t * a.N + n, mx);
  if (quantize_deferred<D>(D::rd(mx), a.n_states)) return;  // needs the tile minimum
  quantize_segment<D>(a, n, t, mx, false, lane, keep);
}

// After k_quantize_rows, one block per tile: the tile's largest and smallest segment abs-max
// (what k_tile_minmax computes), and the segments that kernel deferred, if any: with no such
// segment (the usual case) the block is done after the reduction. With some, every wave walks a
// sixteenth of the channels, 64 at a time, and quantises the deferred ones among them. 1024
// threads: the kernel's duration is a thread's chain of dependent loads, one pass of eight for up
// to 8192 channels.
template <class D>
__global__ __launch_bounds__(1024) void k_quantize_finish(ModArgs a, const void* __restrict__ wmax,
                                                          float* __restrict__ tile_max,
                                                          float* __restrict__ tile_min) {
  __shared__ float smax[16], smin[16];
  __shared__ int s_any;
  const int32_t t = blockIdx.x;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  float mx = 0.0f, mn = __builtin_inff();
  bool mine = false;
  if (threadIdx.x == 0) s_any = 0;
  for (int64_t r0 = threadIdx.x; r0 < a.N; r0 += 1024 * 8) {
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int64_t r = r0 + 1024 * u;
      v[u] = D::load(wmax, (int64_t)t * a.N + (r < a.N ? r : r0));  // r0 again: no effect
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      mx = fmaxf(mx, v[u]);
      mn = fminf(mn, v[u]);
      mine = mine || quantize_deferred<D>(v[u], a.n_states);
    }
  }
  mx = wave_max(mx);
  mn = wave_min(mn);
  if (lane == 0) { smax[wv] = mx; smin[wv] = mn; }
  __syncthreads();
  if (mine) s_any = 1;
  __syncthreads();
  float tmax = smax[0], tmin = smin[0];
#pragma unroll
  for (int w = 1; w < 16; ++w) { tmax = fmaxf(tmax, smax[w]); tmin = fminf(tmin, smin[w]); }
  if (threadIdx.x == 0) { tile_max[t] = tmax; tile_min[t] = tmin; }
  if (s_any == 0) return;
  const bool all_gt1 = quantize_deferred<D>(tmin, a.n_states);
  for (int64_t base = (int64_t)wv * 64; base < a.N; base += 1024) {
    const int64_t nl = base + lane;
    const float m = nl < a.N ? D::load(wmax, (int64_t)t * a.N + nl) : 0.0f;
    uint64_t todo = __ballot(nl < a.N && quantize_deferred<D>(m, a.n_states));
    while (todo) {
      const int src = __builtin_ctzll(todo);
      todo &= todo - 1;
      quantize_segment<D>(a, base + src, t, __shfl(m, src), all_gt1, lane, nullptr);
    }
  }
}

// LSQ backward of the learnable clip: one wave per (channel, tile).
struct ClipBwdArgs {
  void* dw; int64_t lddw;
  const void* w; int64_t ldw;
  const void* clip;        // dtype [T, N]
  const float* tile_min;   // [T]
  void* dclip;             // dtype [T, N]
  int64_t N;
  Tiling tl;
  int32_t quant_type;
  float n_states, maxq, maxq_exact;
};

template <class D>
__global__ __launch_bounds__(256) void k_learned_clip_bwd(ClipBwdArgs a) {
  const int lane = threadIdx.x & 63;
  const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int64_t n = wave / a.tl.n_tiles;
  const int32_t t = (int32_t)(wave % a.tl.n_tiles);
  if (n >= a.N) return;
  const bool quant = a.quant_type == AHL_QUANT_DISCRETIZE_PER_CHANNEL;
  const float clip = D::load(a.clip, (int64_t)t * a.N + n);
  WQuant q;
  if (quant) q = make_wquant<D>(clip, a.n_states, D::rd(__fdiv_rn(a.tile_min[t], a.n_states)) > 1.0f);
  else q = make_wclip<D>(clip, a.tile_min[t] > 1.0f);
  // grad_scale in double like the Python expression, then the fp32 scalar of the tensor op
  const double numel = (double)a.N * (double)a.tl.size(t);
  const float gs = (float)(quant ? 2.0 * sqrt((double)a.maxq_exact / numel) : 1.0 / sqrt(numel));
  float acc = 0.0f;
  for (int32_t k = a.tl.start(t) + lane; k < a.tl.start(t + 1); k += 64) {
    const float w = D::load(a.w, n * a.ldw + k);
    const float g = D::load(a.dw, n * a.lddw + k);
    const float qw = D::rd(D::div_exact_rcp(w, q.rc, q.rcp));
    const bool small = qw < -a.maxq, big = qw > a.maxq;
    // (indicator terms) * grad * grad_scale, evaluated in fp32 as torch promotes them
    float term;
    if (small) term = -a.maxq_exact;
    else if (big) term = a.maxq_exact;
    else term = quant ? D::rd(-qw + rintf(qw)) : 0.0f;
    acc += (term * g) * gs;
    if (small || big) D::store(a.dw, n * a.lddw + k, 0.0f);
  }
  acc = wave_sum(acc);
  if (lane == 0) {
    float r = D::rd(acc);                                // cast to the parameter dtype
    if (quant) r = D::rd(__fdiv_rn(r, a.n_states));       // through clip / n_states
    D::store(a.dclip, (int64_t)t * a.N + n, r);
  }
}

}  // namespace ahl

using namespace ahl;

static int launch_prep(const void* w, int64_t N, int64_t K, int64_t ld, const Tiling& tl,
                       const AhlModifierCfg* cfg, bool with_noise, void* wmax, float* tile_max,
                       float* tile_min, void* w_eff, int64_t ld_eff, hipStream_t s) {
  const int32_t dtype = cfg->dtype;
  const int32_t noise = with_noise ? cfg->noise_type : AHL_NOISE_NONE;
  if (cfg->quant_type < 0 || cfg->quant_type > 3 || noise < 0 || noise > 2) return AHL_ERR_ARG;
  const bool clip_only = cfg->quant_type == AHL_QUANT_CLIP_LEARNED;
  if (clip_only && !cfg->wmax_given) return AHL_ERR_ARG;
  if (cfg->quant_type != AHL_QUANT_NONE && !clip_only && !(cfg->res > 0.0f)) return AHL_ERR_ARG;
  AHL_DISPATCH_DTYPE(dtype, {
    const bool vec = aligned16(w) && (ld % D::EPV == 0);
    if (cdiv(N * tl.n_tiles, 4) > 0x7fffffff) return AHL_ERR_ARG;
    const dim3 grid((unsigned)cdiv(N * tl.n_tiles, 4));
    // one pass for "abs-max + per-channel noise, no quantiser" on 16-byte aligned tiles
    if (!cfg->wmax_given && w_eff && cfg->quant_type == AHL_QUANT_NONE &&
        noise == AHL_NOISE_ADD_NORMAL_PER_CHANNEL && vec && tl.extra == 0 && tl.base % 8 == 0 &&
        aligned16(w_eff) && ld_eff % D::EPV == 0) {
      ModArgs a;
      a.w = w; a.N = N; a.K = K; a.ld = ld; a.tl = tl; a.wmax = nullptr; a.tile_max = nullptr;
      a.tile_min = nullptr; a.w_eff = w_eff; a.ld_eff = ld_eff; a.quant_type = AHL_QUANT_NONE;
      a.noise_type = noise; a.n_states = 1.0f; a.maxq = 1.0f; a.std_dev = cfg->std_dev;
      a.seed = cfg->seed; a.offset = cfg->offset; a.seed_state = cfg->seed_state;
      hipLaunchKernelGGL((k_weight_prep_rows<D>), grid, dim3(256), 0, s, a, wmax);
      if (!cfg->skip_tile_stats)
        hipLaunchKernelGGL((k_tile_minmax<D>), dim3(tl.n_tiles), dim3(256), 0, s, wmax, N, tile_max, tile_min);
      return check_launch("ahl_weight_prep(one pass)");
    }
    // one pass for "abs-max + per-channel quantiser, no noise" on 16-byte aligned tiles
    if (!cfg->wmax_given && w_eff && cfg->quant_type == AHL_QUANT_DISCRETIZE_PER_CHANNEL &&
        noise == AHL_NOISE_NONE && vec && tl.extra == 0 && tl.base % 8 == 0 && aligned16(w_eff) &&
        ld_eff % D::EPV == 0) {
      ModArgs a;
      a.w = w; a.N = N; a.K = K; a.ld = ld; a.tl = tl; a.wmax = nullptr; a.tile_max = tile_max;
      a.tile_min = tile_min; a.w_eff = w_eff; a.ld_eff = ld_eff; a.quant_type = cfg->quant_type;
      a.noise_type = noise; a.n_states = fmaxf(cfg->res, 1.0f / cfg->res);
      a.maxq = host_round_dtype(D::kId, a.n_states / 2.0f);
      a.std_dev = 0.0f; a.seed = 0; a.offset = 0; a.seed_state = nullptr;
      hipLaunchKernelGGL((k_quantize_rows<D>), grid, dim3(256), 0, s, a, wmax);
      hipLaunchKernelGGL((k_quantize_finish<D>), dim3(tl.n_tiles), dim3(1024), 0, s, a, (const void*)wmax, tile_max,
                         tile_min);
      return check_launch("ahl_weight_prep(one-pass quantiser)");
    }
    if (cfg->wmax_given) {
      // wmax holds the learnable clip: nothing to reduce
    } else if (vec) {
      hipLaunchKernelGGL((k_sliced_absmax<D, true>), grid, dim3(256), 0, s, w, N, ld, tl, wmax);
    } else {
      hipLaunchKernelGGL((k_sliced_absmax<D, false>), grid, dim3(256), 0, s, w, N, ld, tl, wmax);
    }
    hipLaunchKernelGGL((k_tile_minmax<D>), dim3(tl.n_tiles), dim3(256), 0, s, wmax, N, tile_max, tile_min);
    if (w_eff) {
      ModArgs a;
      a.w = w; a.N = N; a.K = K; a.ld = ld; a.tl = tl; a.wmax = wmax; a.tile_max = tile_max;
      a.tile_min = tile_min; a.w_eff = w_eff; a.ld_eff = ld_eff;
      a.quant_type = cfg->quant_type; a.noise_type = noise;
      const float res = cfg->res;
      a.n_states = (cfg->quant_type != AHL_QUANT_NONE && !clip_only) ? fmaxf(res, 1.0f / res) : 1.0f;
      // clamp(Tensor, Scalar, Scalar) converts its bounds to the tensor dtype first
      a.maxq = host_round_dtype(D::kId, a.n_states / 2.0f);
      if (clip_only) a.maxq = 1.0f;
      a.std_dev = cfg->std_dev; a.seed = cfg->seed; a.offset = cfg->offset; a.seed_state = cfg->seed_state;
      const int64_t bpr = cdiv(cdiv(K, 8), 256);
      if (bpr * N > 0x7fffffff) return AHL_ERR_ARG;
      const bool vec_mod = vec && K % 8 == 0 && aligned16(w_eff) && ld_eff % D::EPV == 0;
      if (tl.base < 7)
        hipLaunchKernelGGL((k_weight_modify<D, false, true>), dim3((unsigned)(bpr * N)), dim3(256), 0, s, a, (uint32_t)bpr);
      else if (vec_mod)
        hipLaunchKernelGGL((k_weight_modify<D, true>), dim3((unsigned)(bpr * N)), dim3(256), 0, s, a, (uint32_t)bpr);
      else
        hipLaunchKernelGGL((k_weight_modify<D, false>), dim3((unsigned)(bpr * N)), dim3(256), 0, s, a, (uint32_t)bpr);
    }
  });
  return check_launch("ahl_weight_prep");
}

extern "C" {

int ahl_weight_prep(const void* w, int64_t N, int64_t K, int64_t ld, const int32_t* tile_ends_host,
                    int32_t n_tiles, const AhlModifierCfg* cfg, void* wmax, float* tile_max,
                    float* tile_min, void* w_eff, int64_t ld_eff, void* stream) {
  if (!w || !cfg || !wmax || !tile_max || !tile_min || N <= 0 || K <= 0 || ld < K) return AHL_ERR_ARG;
  if (w_eff && ld_eff < K) return AHL_ERR_ARG;
  if (w_eff == w) return AHL_ERR_ARG;  // never modifies the parameter storage
  Tiling tl;
  if (!make_tiling(tile_ends_host, n_tiles, K, &tl)) return AHL_ERR_TILING;
  return launch_prep(w, N, K, ld, tl, cfg, true, wmax, tile_max, tile_min, w_eff, ld_eff,
                     (hipStream_t)stream);
}

int ahl_learned_clip_bwd(void* dw, int64_t lddw, const void* w, int64_t ldw, const void* clip,
                         const float* tile_min, void* dclip, int64_t N, int64_t K,
                         const int32_t* tile_ends_host, int32_t n_tiles, const AhlModifierCfg* cfg,
                         void* stream) {
  if (!dw || !w || !clip || !tile_min || !dclip || !cfg || N <= 0 || K <= 0 || lddw < K || ldw < K)
    return AHL_ERR_ARG;
  const bool quant = cfg->quant_type == AHL_QUANT_DISCRETIZE_PER_CHANNEL;
  if (!quant && cfg->quant_type != AHL_QUANT_CLIP_LEARNED) return AHL_ERR_ARG;
  if (quant && !(cfg->res > 0.0f)) return AHL_ERR_ARG;
  Tiling tl;
  if (!make_tiling(tile_ends_host, n_tiles, K, &tl)) return AHL_ERR_TILING;
  ClipBwdArgs a;
  a.dw = dw; a.lddw = lddw; a.w = w; a.ldw = ldw; a.clip = clip; a.tile_min = tile_min;
  a.dclip = dclip; a.N = N; a.tl = tl; a.quant_type = cfg->quant_type;
  a.n_states = quant ? fmaxf(cfg->res, 1.0f / cfg->res) : 1.0f;
  a.maxq_exact = quant ? a.n_states / 2.0f : 1.0f;
  a.maxq = host_round_dtype(cfg->dtype, a.maxq_exact);
  const int64_t nb = cdiv(N * n_tiles, 4);
  if (nb > 0x7fffffff) return AHL_ERR_ARG;
  AHL_DISPATCH_DTYPE(cfg->dtype, {
    hipLaunchKernelGGL((k_learned_clip_bwd<D>), dim3((unsigned)nb), dim3(256), 0, (hipStream_t)stream, a);
  });
  return check_launch("ahl_learned_clip_bwd");
}

int ahl_quantize_weights(void* w, int64_t N, int64_t K, int64_t ld, const int32_t* tile_ends_host,
                         int32_t n_tiles, const AhlModifierCfg* cfg, void* ws_wmax, float* ws_tile,
                         void* stream) {
  if (!w || !cfg || !ws_wmax || !ws_tile || N <= 0 || K <= 0 || ld < K) return AHL_ERR_ARG;
  if (cfg->quant_type == AHL_QUANT_NONE) return AHL_OK;
  Tiling tl;
  if (!make_tiling(tile_ends_host, n_tiles, K, &tl)) return AHL_ERR_TILING;
  return launch_prep(w, N, K, ld, tl, cfg, false, ws_wmax, ws_tile, ws_tile + n_tiles, w, ld,
                     (hipStream_t)stream);
}

}  // extern "C"
