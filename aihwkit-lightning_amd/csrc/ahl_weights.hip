// Weight-side kernels: per-tile per-channel abs-max, on-the-fly quantisation and Gaussian weight
// noise into a scratch copy (plus its transpose for the input-gradient product), and the
// in-place post-training quantisation.
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
  void* w_eff_t;          // dtype [K, N] or null
  int32_t quant_type, noise_type;
  float n_states, maxq, std_dev;
  uint64_t seed, offset;
};

// 64 (channels) x 64 (inputs) tile per block; thread = 8 consecutive inputs x 2 channels.
template <class D>
__global__ __launch_bounds__(256) void k_weight_modify(ModArgs a) {
  __shared__ typename D::elem tileT[64][64 + 4];
  const int k0 = blockIdx.x * 64, n0 = blockIdx.y * 64;
  const int kq = threadIdx.x & 7, nr = threadIdx.x >> 3;
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int64_t n = n0 + nr + 32 * j;
    const int kb = k0 + 8 * kq;
    float xi[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (a.noise_type != AHL_NOISE_NONE && n < a.N && kb < a.K)
      normal8(a.seed, a.offset, 1u << 24, (uint32_t)(kb >> 3), (uint32_t)n, xi);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int k = kb + e;
      float v = 0.0f;
      if (n < a.N && k < a.K) {
        v = D::load(a.w, n * a.ld + k);
        if (a.quant_type != AHL_QUANT_NONE || a.noise_type != AHL_NOISE_NONE) {
          const int t = a.tl.tile_of(k);
          const float wm = D::load(a.wmax, (int64_t)t * a.N + n);
          const float tmax = a.tile_max[t];
          if (a.quant_type == AHL_QUANT_DISCRETIZE_PER_CHANNEL) {
            const bool all_gt1 = D::rd(__fdiv_rn(a.tile_min[t], a.n_states)) > 1.0f;
            v = wquant_apply<D>(v, make_wquant<D>(wm, a.n_states, all_gt1), a.maxq);
          } else if (a.quant_type == AHL_QUANT_DISCRETIZE) {
            const bool all_gt1 = D::rd(__fdiv_rn(tmax, a.n_states)) > 1.0f;
            v = wquant_apply<D>(v, make_wquant<D>(tmax, a.n_states, all_gt1), a.maxq);
          }
          if (a.noise_type != AHL_NOISE_NONE) {
            const float ref = a.noise_type == AHL_NOISE_ADD_NORMAL_PER_CHANNEL ? wm : tmax;
            const float nstd = D::rd(a.std_dev * ref);
            v = D::rd(v + D::rd(nstd * D::rd(xi[e])));
          }
        }
        if (a.w_eff) D::store(a.w_eff, n * a.ld_eff + k, v);
      }
      tileT[8 * kq + e][nr + 32 * j] = D::to_elem(v);
    }
  }
  if (!a.w_eff_t) return;
  __syncthreads();
  const int nq = threadIdx.x & 15, kr = threadIdx.x >> 4;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int64_t k = k0 + kr + 16 * j;
    if (k >= a.K) continue;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int64_t n = n0 + 4 * nq + e;
      if (n < a.N) ((typename D::elem*)a.w_eff_t)[k * a.N + n] = tileT[kr + 16 * j][4 * nq + e];
    }
  }
}

}  // namespace ahl

using namespace ahl;

static int launch_prep(const void* w, int64_t N, int64_t K, int64_t ld, const Tiling& tl,
                       const AhlModifierCfg* cfg, bool with_noise, void* wmax, float* tile_max,
                       float* tile_min, void* w_eff, int64_t ld_eff, void* w_eff_t, hipStream_t s) {
  const int32_t dtype = cfg->dtype;
  const int32_t noise = with_noise ? cfg->noise_type : AHL_NOISE_NONE;
  if (cfg->quant_type < 0 || cfg->quant_type > 2 || noise < 0 || noise > 2) return AHL_ERR_ARG;
  if (cfg->quant_type != AHL_QUANT_NONE && !(cfg->res > 0.0f)) return AHL_ERR_ARG;
  AHL_DISPATCH_DTYPE(dtype, {
    const bool vec = aligned16(w) && (ld % D::EPV == 0);
    const dim3 grid((unsigned)cdiv(N, 4));
    if (vec) hipLaunchKernelGGL((k_sliced_absmax<D, true>), grid, dim3(256), 0, s, w, N, ld, tl, wmax);
    else hipLaunchKernelGGL((k_sliced_absmax<D, false>), grid, dim3(256), 0, s, w, N, ld, tl, wmax);
    hipLaunchKernelGGL((k_tile_minmax<D>), dim3(tl.n_tiles), dim3(256), 0, s, wmax, N, tile_max, tile_min);
    if (w_eff || w_eff_t) {
      ModArgs a;
      a.w = w; a.N = N; a.K = K; a.ld = ld; a.tl = tl; a.wmax = wmax; a.tile_max = tile_max;
      a.tile_min = tile_min; a.w_eff = w_eff; a.ld_eff = ld_eff; a.w_eff_t = w_eff_t;
      a.quant_type = cfg->quant_type; a.noise_type = noise;
      const float res = cfg->res;
      a.n_states = cfg->quant_type != AHL_QUANT_NONE ? fmaxf(res, 1.0f / res) : 1.0f;
      // clamp(Tensor, Scalar, Scalar) converts its bounds to the tensor dtype first
      a.maxq = D::kIsBf16 ? host_round_bf16(a.n_states / 2.0f) : a.n_states / 2.0f;
      a.std_dev = cfg->std_dev; a.seed = cfg->seed; a.offset = cfg->offset;
      hipLaunchKernelGGL((k_weight_modify<D>), dim3((unsigned)cdiv(K, 64), (unsigned)cdiv(N, 64)), dim3(256), 0, s, a);
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
  return launch_prep(w, N, K, ld, tl, cfg, true, wmax, tile_max, tile_min, w_eff, ld_eff, nullptr,
                     (hipStream_t)stream);
}

int ahl_quantize_weights(void* w, int64_t N, int64_t K, int64_t ld, const int32_t* tile_ends_host,
                         int32_t n_tiles, const AhlModifierCfg* cfg, void* ws_wmax, float* ws_tile,
                         void* stream) {
  if (!w || !cfg || !ws_wmax || !ws_tile || N <= 0 || K <= 0 || ld < K) return AHL_ERR_ARG;
  if (cfg->quant_type == AHL_QUANT_NONE) return AHL_OK;
  Tiling tl;
  if (!make_tiling(tile_ends_host, n_tiles, K, &tl)) return AHL_ERR_TILING;
  return launch_prep(w, N, K, ld, tl, cfg, false, ws_wmax, ws_tile, ws_tile + n_tiles, w, ld, nullptr,
                     (hipStream_t)stream);
}

}  // extern "C"
