// Shared by the bf16 forward kernels (ahl_fast.hip): launch arguments and the
// small device helpers of the per-K-tile epilogue.
#pragma once
#include "ahl_host.h"
#include <math.h>

namespace ahl {

// round two fp32 values to bf16 precision, keeping them in fp32 registers (3 instructions)
AHL_DEV void rd2(float& a, float& b) {
  const uint32_t p = pack_bf16x2(a, b);
  a = unpack_lo(p);
  b = unpack_hi(p);
}

struct FastFwdArgs {
  const void* xq; int64_t ldx;   // pre-quantised input, bf16 [M, K]
  const void* w; int64_t ldw;    // effective weights, bf16 [N, K]
  const void* bias;
  void* y; int64_t ldy;
  uint32_t* keep;                // clamp mask [T, ceil(N/32), M] or null
  uint32_t* clamp_flag;          // receives flag_value if any tile output was clamped; may be null
  uint32_t flag_value;           // the caller's token, or 1 for a word the launcher cleared
  const void* ir;                // [T] static, [T, M] dynamic
  const void* wmax;              // [T, N]
  const float* tile_max;         // [T]
  int64_t M, N;
  int32_t tile;                  // columns of a tile that hold data, rounded up to 64
  int32_t tile_stride;           // columns from one tile start to the next (>= tile)
  int32_t n_tiles;
  float out_bound, out_res, step_factor;
  float noise_scale;
  int32_t noise_per_channel, bound_per_channel, skip_rounding, clamp_on, step_by_division;
  uint64_t seed, offset;
  const uint64_t* seed_state;    // null, or device {key, call counter} that replaces seed / offset
  uint16_t* part;                // null, or [T, M, N]: every block takes ONE K-tile and leaves its
                                 // result there; k_tile_sum adds the tiles in order (few rows)
  ConvMap conv;                  // conv.on: xq is a padded channels-last image (see ConvMap)
};

AHL_DEV void mma_bf16_zero(const u32x4& a, const u32x4& b, f32x16& c) {
  const f32x16 z = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                              __builtin_bit_cast(bf16x8, b), z, 0, 0, 0);
}

AHL_DEV void mma_bf16(const u32x4& a, const u32x4& b, f32x16& c) {
  c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                              __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

// step of an ADC with bound B (a value of the 16-bit dtype held in fp32): rd(rd(2B) / n) for n states, rd(2B * res)
// for a relative resolution. 2B is exact, so the second form is one product with the factor
// 2 * res; for n with <= 8 significant bits the product with fl(2 / n) rounds to the same bf16 as
// the quotient (see BF16::div). Only other n need the division; that case is a branch on a
// launch constant, so the common one carries no division code.
// float16: the same holds for n with <= 11 significant bits and steps that are normal float16 values
// (BOTH facts are checked exhaustively on the CPU; smaller steps are divided), but 2B itself can leave the type's range (B > 32752): it is rounded first, so that
// such a bound gives the infinite step the reference gets.
template <class D = BF16>
AHL_DEV float adc_step(float B, const FastFwdArgs& a) {
  if (__builtin_expect(a.step_by_division != 0, 0)) return D::rd(__fdiv_rn(D::rd(B + B), a.out_res));
  if (D::kDoubleCanOverflow) {
    const float s = D::rd(D::rd(B + B) * (0.5f * a.step_factor));
    // a step below the smallest normal float16 is rounded on the subnormal grid, where the product
    // with fl(1 / n) can fall on the other side of a tie than the quotient: divide there
    if (__builtin_expect(s < 6.2e-5f && a.out_res > 1.0f, 0)) return D::rd(__fdiv_rn(D::rd(B + B), a.out_res));
    return s;
  }
  return D::rd(B * a.step_factor);
}

// the same for four bounds at once, rounded in pairs (the product form only)
template <class D>
AHL_DEV void adc_step4(const float* B, float* r, const FastFwdArgs& a) {
  if (D::kDoubleCanOverflow) {
#pragma unroll
    for (int c = 0; c < 4; ++c) r[c] = B[c] + B[c];
    round2<D>(r[0], r[1]); round2<D>(r[2], r[3]);
    const float hf = 0.5f * a.step_factor;
    float twoB[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) { twoB[c] = r[c]; r[c] *= hf; }
    round2<D>(r[0], r[1]); round2<D>(r[2], r[3]);
    // subnormal steps: by division (see adc_step)
    if (__builtin_expect(fminf(fminf(r[0], r[1]), fminf(r[2], r[3])) < 6.2e-5f && a.out_res > 1.0f, 0)) {
#pragma unroll
      for (int c = 0; c < 4; ++c) r[c] = D::rd(__fdiv_rn(twoB[c], a.out_res));
    }
    return;
  } else {
#pragma unroll
    for (int c = 0; c < 4; ++c) r[c] = B[c] * a.step_factor;
  }
  round2<D>(r[0], r[1]); round2<D>(r[2], r[3]);
}

}  // namespace ahl
