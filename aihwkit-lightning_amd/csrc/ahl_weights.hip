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
  q.rc = fmaxf(q.step, kTinyF32);
  q.rcp = __fdiv_rn(1.0f, q.rc);
  return q;
}

template <class D>
AHL_DEV float wquant_apply(float w, const WQuant& q, float maxq) {
  float v = D::rd(D::div(w, q.rc, q.rcp));
  v = fminf(fmaxf(v, -maxq), maxq);
  v = rintf(v);
  return D::rd(v * q.step);
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
};

// One thread per group of 8 consecutive inputs of one channel (one Philox call gives the 8
// normals of the group); consecutive threads walk along the row, so that with VEC every wave
// reads and writes contiguous 16-byte vectors.
template <class D, bool VEC>
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
    if (a.noise_type != AHL_NOISE_NONE)
      normal8(a.seed, a.offset, 1u << 24, (uint32_t)(kb >> 3), (uint32_t)n, xi);
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
      }
      c.nstd = D::rd(a.std_dev * (a.noise_type == AHL_NOISE_ADD_NORMAL_PER_CHANNEL ? wm : tmax));
      return c;
    };
    const int t0 = a.tl.tile_of(kb), t1 = a.tl.tile_of(klast);
    TileConst c = tile_const(t0);
    const int32_t t1_start = t1 != t0 ? a.tl.start(t1) : 0x7fffffff;  // a group spans at most 2 tiles
    const TileConst c1 = t1 != t0 ? tile_const(t1) : c;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const TileConst& ce = kb + e >= t1_start ? c1 : c;
      float x = v[e];
      if (a.quant_type != AHL_QUANT_NONE) x = wquant_apply<D>(x, ce.q, a.maxq);
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

}  // namespace ahl

using namespace ahl;

static int launch_prep(const void* w, int64_t N, int64_t K, int64_t ld, const Tiling& tl,
                       const AhlModifierCfg* cfg, bool with_noise, void* wmax, float* tile_max,
                       float* tile_min, void* w_eff, int64_t ld_eff, hipStream_t s) {
  const int32_t dtype = cfg->dtype;
  const int32_t noise = with_noise ? cfg->noise_type : AHL_NOISE_NONE;
  if (cfg->quant_type < 0 || cfg->quant_type > 2 || noise < 0 || noise > 2) return AHL_ERR_ARG;
  if (cfg->quant_type != AHL_QUANT_NONE && !(cfg->res > 0.0f)) return AHL_ERR_ARG;
  AHL_DISPATCH_DTYPE(dtype, {
    const bool vec = aligned16(w) && (ld % D::EPV == 0);
    if (cdiv(N * tl.n_tiles, 4) > 0x7fffffff) return AHL_ERR_ARG;
    const dim3 grid((unsigned)cdiv(N * tl.n_tiles, 4));
    if (vec) hipLaunchKernelGGL((k_sliced_absmax<D, true>), grid, dim3(256), 0, s, w, N, ld, tl, wmax);
    else hipLaunchKernelGGL((k_sliced_absmax<D, false>), grid, dim3(256), 0, s, w, N, ld, tl, wmax);
    hipLaunchKernelGGL((k_tile_minmax<D>), dim3(tl.n_tiles), dim3(256), 0, s, wmax, N, tile_max, tile_min);
    if (w_eff) {
      ModArgs a;
      a.w = w; a.N = N; a.K = K; a.ld = ld; a.tl = tl; a.wmax = wmax; a.tile_max = tile_max;
      a.tile_min = tile_min; a.w_eff = w_eff; a.ld_eff = ld_eff;
      a.quant_type = cfg->quant_type; a.noise_type = noise;
      const float res = cfg->res;
      a.n_states = cfg->quant_type != AHL_QUANT_NONE ? fmaxf(res, 1.0f / res) : 1.0f;
      // clamp(Tensor, Scalar, Scalar) converts its bounds to the tensor dtype first
      a.maxq = D::kIsBf16 ? host_round_bf16(a.n_states / 2.0f) : a.n_states / 2.0f;
      a.std_dev = cfg->std_dev; a.seed = cfg->seed; a.offset = cfg->offset;
      const int64_t bpr = cdiv(cdiv(K, 8), 256);
      if (bpr * N > 0x7fffffff) return AHL_ERR_ARG;
      const bool vec_mod = vec && K % 8 == 0 && aligned16(w_eff) && ld_eff % D::EPV == 0;
      if (vec_mod)
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
