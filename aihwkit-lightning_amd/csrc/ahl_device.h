// Device-side building blocks shared by every kernel of libanalog_hip.so (gfx950 only).
//
//  * dtype traits: F32 / BF16 with rd() = "round the fp32 result of one elementwise op to the
//    tensor dtype", which is where torch rounds when it evaluates an op on bf16 tensors.
//  * Tiling: the reference's K-tile split rule in closed form.
//  * Philox4x32-10 counter-based RNG + Box-Muller.
//  * wave64 reductions.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define AHL_DEV __device__ __forceinline__

namespace ahl {

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// ---------------------------------------------------------------------------------------------
// K-tile split (reference nn/modules/linear.py:155-170): n_tiles = ceil(K / max_input_size),
// base, extra = divmod(K, n_tiles); the first `extra` tiles have base+1 columns, the rest base.
struct Tiling {
  int32_t n_tiles;
  int32_t base;
  int32_t extra;
  AHL_DEV int32_t start(int32_t t) const { return t * base + (t < extra ? t : extra); }
  AHL_DEV int32_t size(int32_t t) const { return base + (t < extra ? 1 : 0); }
  AHL_DEV int32_t tile_of(int32_t k) const {
    const int32_t big = extra * (base + 1);
    return k < big ? k / (base + 1) : extra + (k - big) / base;
  }
};

// ---------------------------------------------------------------------------------------------
// Block index -> (row block, column block) of the output. Workgroups go to the 8 XCDs round
// robin (block b runs on XCD b % 8) and each XCD has its own L2, so (1) every XCD gets one
// contiguous range of the linear tile order, and (2) that order walks bands of G row blocks
// column by column: the blocks resident on an XCD at any time then form a compact patch of
// about G rows by (resident / G) columns and share their operand panels in L2, instead of a
// 1- or 2-row strip that streams the whole other operand.
AHL_DEV void block_to_tile(int64_t bid, int64_t nb, int64_t nbm, int64_t nbn, int G, int64_t& bm,
                           int64_t& bn) {
  int64_t lin = bid;
  if ((nb & 7) == 0) lin = (bid & 7) * (nb >> 3) + (bid >> 3);
  const int64_t per_band = (int64_t)G * nbn;
  const int64_t band = lin / per_band, in_band = lin % per_band;
  const int64_t first = band * G;
  const int64_t gsz = nbm - first < G ? nbm - first : G;
  bm = first + in_band % gsz;
  bn = in_band / gsz;
}

// ---------------------------------------------------------------------------------------------
// A convolution read straight off the image (stride 1, dilation 1), instead of off a patch matrix.
// The image is kept zero-padded and channels-last as a flat [pixels, C] matrix; the outputs are
// numbered on the same PADDED pixel grid (row p is the output whose receptive field has its
// first corner at padded pixel p; rows whose field would leave the image are computed and
// dropped). A kernel offset ("tap") is then ONE constant row offset for every output:
//   tap = (id * kh + ih) * kw + iw   ->   rows (id * hp + ih) * wp + iw.
// The contraction of a K-tile runs over (tap, channel) instead of the reference's (channel, tap)
// -- the same terms, so the tile's sum is the same up to the order of the fp32 additions -- and a
// 64-wide chunk of it is 64 consecutive channels of one tap: the same 128-byte row segment a
// matrix operand has, at a row offset that depends on the chunk only.
struct ConvMap {
  int32_t on;          // 0: a plain matrix operand
  int32_t sign;        // +1: output row m reads rows m + offset(tap); -1: rows m + lead - offset(tap)
  int32_t lead;        // sign -1: rows of zeros in front of the operand (= the largest offset)
  int32_t cg;          // 64-wide chunks per tap
  int32_t tile_base;   // columns between the starts of two tiles inside an operand row
  int32_t kh, kw;      // kernel extents of the two inner dimensions
  int32_t hp, wp;      // padded image extents of the two inner dimensions
  int64_t alloc_rows;  // rows the operand's allocation holds (all readable, zero beyond the data)
};
AHL_DEV int32_t conv_tap_rows(const ConvMap& c, int32_t tap) {
  const int32_t iw = tap % c.kw, r = tap / c.kw;
  const int32_t ih = r % c.kh, id = r / c.kh;
  return (id * c.hp + ih) * c.wp + iw;
}
// element offset inside the operand of chunk i of tile t, relative to the output row's own row
AHL_DEV int32_t conv_chunk_offset(const ConvMap& c, int32_t t, int32_t i, int32_t ld) {
  const int32_t tap = i / c.cg;
  const int32_t rows = c.sign > 0 ? conv_tap_rows(c, tap) : c.lead - conv_tap_rows(c, tap);
  return rows * ld + t * c.tile_base + (i - tap * c.cg) * 64;
}

// ---------------------------------------------------------------------------------------------
// Clamp-mask layout: one bit per (tile, row, column). Word [(t * ceil(N/32) + n / 32) * M + m]
// has bit (n % 32) set where the tile-t output of element (m, n) left the ADC range (and so
// passes no gradient). One 64-lane ballot over a 32x32 MFMA result register yields two such
// words (rows r and r + 4); the 64 rows of a wave's tile are 256 contiguous bytes.
// The row dimension of the mask is padded to a multiple of 64, so that the words of four
// consecutive rows are always one aligned 16-byte vector inside the plane, whatever M is.
AHL_DEV int64_t clamp_rows(int64_t M) { return (M + 63) & ~(int64_t)63; }
AHL_DEV int64_t clamp_plane_words(int64_t M, int64_t N) { return ((N + 31) >> 5) * clamp_rows(M); }
AHL_DEV int64_t clamp_word(int64_t m, int64_t n, int64_t M) { return (n >> 5) * clamp_rows(M) + m; }
// Whether the forward's one-word flag says that some output was clamped (no flag: assume so).
// token 0: the forward cleared the word and set it non-zero; otherwise it stored the token.
AHL_DEV bool clamp_flag_says_clamped(const uint32_t* flag, uint32_t token) {
  if (flag == nullptr) return true;
  const uint32_t v = *flag;
  return token ? v == token : v != 0u;
}

// ---------------------------------------------------------------------------------------------
// bf16 <-> f32
AHL_DEV float bf16_bits_to_f32(uint32_t bits16) { return __uint_as_float(bits16 << 16); }
AHL_DEV uint32_t f32_to_bf16_bits(float x) {
  return (uint32_t)__builtin_bit_cast(uint16_t, (__bf16)x);
}
AHL_DEV uint32_t pack_bf16x2(float lo, float hi) {
  f32x2 v = {lo, hi};
  bf16x2 b = __builtin_convertvector(v, bf16x2);  // one v_cvt_pk_bf16_f32 (RNE)
  return __builtin_bit_cast(uint32_t, b);
}
AHL_DEV float unpack_lo(uint32_t w) { return __uint_as_float(w << 16); }
AHL_DEV float unpack_hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }

// ---------------------------------------------------------------------------------------------
// dtype traits. `vec` is one 16-byte global/LDS transaction holding EPV elements.
struct F32 {
  typedef float elem;
  static constexpr int kId = 0;
  static constexpr int EPV = 4;
  static constexpr bool kIsBf16 = false;
  static AHL_DEV float tiny() { return 1.17549435e-38f; }   // torch.finfo(dtype).tiny
  static AHL_DEV float rd(float x) { return x; }
  static AHL_DEV elem to_elem(float x) { return x; }
  static AHL_DEV float load(const void* p, int64_t i) { return ((const float*)p)[i]; }
  static AHL_DEV void store(void* p, int64_t i, float v) { ((float*)p)[i] = v; }
  static AHL_DEV void unpack(const u32x4& v, float* f) {
    f[0] = __uint_as_float(v.x); f[1] = __uint_as_float(v.y);
    f[2] = __uint_as_float(v.z); f[3] = __uint_as_float(v.w);
  }
  static AHL_DEV u32x4 pack(const float* f) {
    u32x4 v = {__float_as_uint(f[0]), __float_as_uint(f[1]), __float_as_uint(f[2]),
               __float_as_uint(f[3])};
    return v;
  }
  // x / d, where rcp_d is 1/d: fp32 tensors use the IEEE quotient like torch on the CPU.
  static AHL_DEV float div(float x, float d, float /*rcp_d*/) { return __fdiv_rn(x, d); }
  static AHL_DEV float div_exact_rcp(float x, float d, float /*rcp_d*/) { return __fdiv_rn(x, d); }
  static AHL_DEV float div_to_round(float x, float d, float /*rcp_d*/) { return __fdiv_rn(x, d); }
};

struct BF16 {
  typedef uint16_t elem;
  static constexpr int kId = 1;
  static constexpr int EPV = 8;
  static constexpr bool kIsBf16 = true;
  static AHL_DEV float tiny() { return 1.17549435e-38f; }
  static AHL_DEV float rd(float x) { return bf16_bits_to_f32(f32_to_bf16_bits(x)); }
  static AHL_DEV elem to_elem(float x) { return (elem)f32_to_bf16_bits(x); }
  static AHL_DEV float load(const void* p, int64_t i) {
    return bf16_bits_to_f32(((const uint16_t*)p)[i]);
  }
  static AHL_DEV void store(void* p, int64_t i, float v) {
    ((uint16_t*)p)[i] = (uint16_t)f32_to_bf16_bits(v);
  }
  static AHL_DEV void unpack(const u32x4& v, float* f) {
    f[0] = unpack_lo(v.x); f[1] = unpack_hi(v.x); f[2] = unpack_lo(v.y); f[3] = unpack_hi(v.y);
    f[4] = unpack_lo(v.z); f[5] = unpack_hi(v.z); f[6] = unpack_lo(v.w); f[7] = unpack_hi(v.w);
  }
  static AHL_DEV u32x4 pack(const float* f) {
    u32x4 v = {pack_bf16x2(f[0], f[1]), pack_bf16x2(f[2], f[3]), pack_bf16x2(f[4], f[5]),
               pack_bf16x2(f[6], f[7])};
    return v;
  }
  // For bf16 operands x and d (8-bit significands) the exact quotient is never closer than
  // 2^-17 (relative) to a bf16 rounding boundary unless it is representable, so rounding
  // x * fl32(1/d) to bf16 gives bit-identical results to rounding fl32(x / d). The caller
  // rounds the returned value with rd().
  static AHL_DEV float div(float x, float /*d*/, float rcp_d) { return x * rcp_d; }
  static AHL_DEV float div_exact_rcp(float x, float /*d*/, float rcp_d) { return x * rcp_d; }
  static AHL_DEV float div_to_round(float x, float /*d*/, float rcp_d) { return x * rcp_d; }
  // two values as one register of 16-bit halves (rounded to nearest even), and back
  static AHL_DEV uint32_t pack2(float lo, float hi) { return pack_bf16x2(lo, hi); }
  static AHL_DEV float lo(uint32_t w) { return unpack_lo(w); }
  static AHL_DEV float hi(uint32_t w) { return unpack_hi(w); }
  // state counts of a quantiser with <= 8 significant bits give the same step whether it is
  // computed as 2 B / n or as B * fl(2 / n) (see div)
  static constexpr int kExactStepBits = 8;
  static constexpr bool kDoubleCanOverflow = false;   // 2 x a finite value overflows only near 3e38
};

// float16: like bfloat16, every elementwise result is rounded to the tensor dtype (round to
// nearest even; v_cvt_f16_f32 / v_cvt_f32_f16), 8 elements per 16-byte vector.
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
AHL_DEV uint32_t pack_f16x2(float lo, float hi) {
  f32x2 v = {lo, hi};
  f16x2 h = __builtin_convertvector(v, f16x2);
  return __builtin_bit_cast(uint32_t, h);
}
AHL_DEV float f16_lo(uint32_t w) { return (float)__builtin_bit_cast(f16x2, w)[0]; }
AHL_DEV float f16_hi(uint32_t w) { return (float)__builtin_bit_cast(f16x2, w)[1]; }

struct F16 {
  typedef uint16_t elem;
  static constexpr int kId = 2;
  static constexpr int EPV = 8;
  static constexpr bool kIsBf16 = false;
  static AHL_DEV float tiny() { return 6.103515625e-05f; }
  // The two conversions are written as instructions: left to the compiler, "round the fp32
  // result of an operation to float16" is merged with the operation into mixed-precision
  // instructions in some kernels and not in others, and the two forms do not always round alike.
  static AHL_DEV float rd(float x) {
    uint32_t h;
    float r;
    asm("v_cvt_f16_f32 %0, %1" : "=v"(h) : "v"(x));
    asm("v_cvt_f32_f16 %0, %1" : "=v"(r) : "v"(h));
    return r;
  }
  static AHL_DEV elem to_elem(float x) {
    uint32_t h;
    asm("v_cvt_f16_f32 %0, %1" : "=v"(h) : "v"(x));
    return (elem)h;
  }
  static AHL_DEV float load(const void* p, int64_t i) { return (float)((const _Float16*)p)[i]; }
  static AHL_DEV void store(void* p, int64_t i, float v) { ((elem*)p)[i] = to_elem(v); }
  static AHL_DEV void unpack(const u32x4& v, float* f) {
    f[0] = f16_lo(v.x); f[1] = f16_hi(v.x); f[2] = f16_lo(v.y); f[3] = f16_hi(v.y);
    f[4] = f16_lo(v.z); f[5] = f16_hi(v.z); f[6] = f16_lo(v.w); f[7] = f16_hi(v.w);
  }
  static AHL_DEV u32x4 pack(const float* f) {
    u32x4 v = {pack_f16x2(f[0], f[1]), pack_f16x2(f[2], f[3]), pack_f16x2(f[4], f[5]),
               pack_f16x2(f[6], f[7])};
    return v;
  }
  // 11-bit significands. With the CORRECTLY ROUNDED fp32 reciprocal, rounding x * rcp_d to
  // float16 equals rounding x / d for every pair of float16 values whose quotient is a NORMAL
  // float16 (exhaustive over the significands), as for bfloat16. A quotient below 2^-14 is rounded
  // on the subnormal grid, where the exact quotient can be a tie that fl32(1 / d) tips (x = 5.424e-6,
  // d = 14 is one of them): there the corrected quotient of div() is taken, which is the IEEE fp32
  // quotient for subnormal x as well. The caller rounds the returned value with rd().
  static AHL_DEV float div_exact_rcp(float x, float d, float rcp_d) {
    const float q0 = x * rcp_d;
    return fabsf(q0) < 6.2e-5f ? div(x, d, rcp_d) : q0;
  }
  // The same for a quotient that is rounded to an integer next: below 2^-14 that is zero (with the
  // quotient's sign) whichever neighbour on the subnormal grid the float16 rounding picked.
  static AHL_DEV float div_to_round(float x, float /*d*/, float rcp_d) { return x * rcp_d; }
  // With a reciprocal that is one fp32 step off (v_rcp_f32) a few products land on the other
  // side of a float16 rounding boundary, so the fp32 IEEE quotient is needed. For float16-valued
  // x and d it takes one correction step instead of the full division
  // sequence: q0 = x * rcp_d (rcp_d within one fp32 step of 1 / d), r = x - d * q0 (exact in an
  // fma: x is a multiple of the product's last place and the difference has < 14 bits),
  // q1 = q0 + r * rcp_d = (x / d) (1 + e), |e| < 2^-45. x / d cannot lie within 2^-36 (relative) of
  // a midpoint between two fp32 values (d times a 25-bit odd number has more bits than x), so q1
  // IS the correctly rounded fp32 quotient. Zero and non-finite x keep q0 (sign of zero, inf).
  static AHL_DEV float div(float x, float d, float rcp_d) {
    const float q0 = x * rcp_d;
    const float r = __builtin_fmaf(-d, q0, x);
    const float q1 = __builtin_fmaf(r, rcp_d, q0);
    // class bits 3, 4, 7, 8: normal or subnormal of either sign (not zero, infinite or NaN)
    return __builtin_amdgcn_classf(q0, 0x198) ? q1 : q0;
  }
  // the packing conversion as an instruction, for the reason given at rd()
  static AHL_DEV uint32_t pack2(float lo, float hi) {
    uint32_t w;
    asm("v_cvt_pk_f16_f32 %0, %1, %2" : "=v"(w) : "v"(lo), "v"(hi));
    return w;
  }
  static AHL_DEV float lo(uint32_t w) { return f16_lo(w); }
  static AHL_DEV float hi(uint32_t w) { return f16_hi(w); }
  // state counts with <= 11 significant bits: rd(2B / n) == rd(rd(2B) * fl(1 / n)), as for div
  static constexpr int kExactStepBits = 11;
  static constexpr bool kDoubleCanOverflow = true;    // 2B is inf for B > 32752
};

// round two fp32 values to the 16-bit dtype D, keeping them in fp32 registers (3 instructions)
template <class D>
AHL_DEV void round2(float& a, float& b) {
  const uint32_t p = D::pack2(a, b);
  a = D::lo(p);
  b = D::hi(p);
}

// ---- MFMA wrappers: one 32 x 32 x 16 product of 16-bit operands (8 per lane) ----
typedef _Float16 f16x8m __attribute__((ext_vector_type(8)));
template <class D>
struct Mma16;
template <>
struct Mma16<BF16> {
  static AHL_DEV void run(const u32x4& a, const u32x4& b, f32x16& c) {
    c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
  static AHL_DEV void run_zero(const u32x4& a, const u32x4& b, f32x16& c) {   // c = a x b
    const f32x16 z = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                __builtin_bit_cast(bf16x8, b), z, 0, 0, 0);
  }
};
template <>
struct Mma16<F16> {
  static AHL_DEV void run(const u32x4& a, const u32x4& b, f32x16& c) {
    c = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8m, a),
                                               __builtin_bit_cast(f16x8m, b), c, 0, 0, 0);
  }
  static AHL_DEV void run_zero(const u32x4& a, const u32x4& b, f32x16& c) {
    const f32x16 z = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    c = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8m, a),
                                               __builtin_bit_cast(f16x8m, b), z, 0, 0, 0);
  }
};

static constexpr float kTinyF32 = 1.17549435e-38f;  // finfo(float32).tiny == finfo(bfloat16).tiny

// ---------------------------------------------------------------------------------------------
// Resolution convention of the reference's UniformQuantize (torch_utils/quant_utils.py:63-76):
// res > 1 is a number of states (step = 2*bound / res), otherwise the step is 2*bound * res.
template <class D>
AHL_DEV float quant_step(float bound, float res) {
  const float alpha = D::rd(2.0f * bound);
  return res > 1.0f ? D::rd(__fdiv_rn(alpha, res)) : D::rd(alpha * res);
}

// ---------------------------------------------------------------------------------------------
// a ^ b ^ c in one instruction (v_bitop3_b32 with truth table 0x96)
AHL_DEV uint32_t xor3(uint32_t a, uint32_t b, uint32_t c) {
  return __builtin_amdgcn_bitop3_b32(a, b, c, 0x96);
}

// Philox4x32-10 (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3", SC'11).
// one round: the counter is replaced, the key moves on
AHL_DEV void philox_round(u32x4& c, uint32_t& k0, uint32_t& k1) {
  const uint64_t p0 = (uint64_t)0xD2511F53u * c.x;
  const uint64_t p1 = (uint64_t)0xCD9E8D57u * c.z;
  u32x4 n;
  n.x = xor3((uint32_t)(p1 >> 32), c.y, k0);
  n.y = (uint32_t)p1;
  n.z = xor3((uint32_t)(p0 >> 32), c.w, k1);
  n.w = (uint32_t)p0;
  c = n;
  k0 += 0x9E3779B9u;
  k1 += 0xBB67AE85u;
}
AHL_DEV u32x4 philox4x32_10(u32x4 c, uint32_t k0, uint32_t k1) {
#pragma unroll
  for (int r = 0; r < 10; ++r) philox_round(c, k0, k1);
  return c;
}

// Two standard normals from one 32-bit word (Box-Muller with two 16-bit uniforms):
//   u1 = (lo16 + 0.5) / 65536, u2 = (hi16 + 0.5) / 65536,
//   r = sqrt(-2 ln u1), (n0, n1) = r * (cos 2 pi u2, sin 2 pi u2).
// The radius is limited to 4.85 sigma (u1 >= 2^-17); the variance deficit is < 1e-4.
// v_log_f32 is log2, v_sin_f32 / v_cos_f32 take their argument in revolutions.
AHL_DEV void box_muller16(uint32_t w, float& n0, float& n1) {
  const float a = (float)(w & 0xffffu) + 0.5f;
  // radius^2 = -2 ln(a / 65536) = (16 - log2 a) * 2 ln 2
  const float r2 = __builtin_fmaf(__builtin_amdgcn_logf(a), -1.3862943611198906f, 22.180709777918250f);
  const float r = __builtin_amdgcn_sqrtf(r2);
  // angle in revolutions: the high half as the mantissa of a float in [1, 2); v_sin/v_cos are
  // periodic in whole revolutions, so the leading 1 needs no subtraction
  const float rev = __uint_as_float(0x3f800000u | ((w >> 9) & 0x007fff80u));
  n0 = r * __builtin_amdgcn_cosf(rev);
  n1 = r * __builtin_amdgcn_sinf(rev);
}

// Philox key and counter offset of a call. They come by value, or -- for launches that are
// replayed from a HIP graph, where a value baked into the launch would repeat the same noise on
// every replay -- from device memory: state[0] = key, state[1] = a running call counter that
// ahl_seed_advance moves; the by-value offset is added to it.
struct NoiseKey { uint64_t seed, offset; };
AHL_DEV NoiseKey noise_key(uint64_t seed, uint64_t offset, const uint64_t* state) {
  NoiseKey k = {seed, offset};
  if (state != nullptr) { k.seed = state[0]; k.offset = state[1] + offset; }
  return k;
}

AHL_DEV void normal8(uint64_t seed, uint64_t offset, uint32_t stream_and_tile, uint32_t c0,
                     uint32_t c1, float* out8) {
  u32x4 c = {c0, c1, stream_and_tile, (uint32_t)offset};
  const u32x4 r = philox4x32_10(c, (uint32_t)seed, (uint32_t)(seed >> 32));
  box_muller16(r.x, out8[0], out8[1]);
  box_muller16(r.y, out8[2], out8[3]);
  box_muller16(r.z, out8[4], out8[5]);
  box_muller16(r.w, out8[6], out8[7]);
}

// ---------------------------------------------------------------------------------------------
// wave64 reductions (all lanes end up with the result)
// Records the clamp bits of one register of a 32x32 MFMA result (lane l holds column l % 32 of
// row `row` for l < 32 and of row `row + 4` for l >= 32, rows counted within the wave's tile)
// in `words`, where lane L keeps the mask word of row L. Must be called by the whole wave.
// v_writelane_b32 through the compiler (this clang declares no builtin for it): it then places the
// wait states after the compare that produced the value itself, and a lane number that is a
// constant after unrolling becomes an immediate operand.
extern "C" __device__ int ahl_writelane(int value, int lane, int old) __asm("llvm.amdgcn.writelane.i32");

AHL_DEV void clamp_record_bits(uint64_t b, int row, uint32_t& words) {
  // the ballot is wave-uniform: its halves go into lanes `row` and `row + 4` directly (a select
  // per lane would cost two compares that write scalar registers)
  words = (uint32_t)ahl_writelane((int)(uint32_t)b, row, (int)words);
  words = (uint32_t)ahl_writelane((int)(uint32_t)(b >> 32), row + 4, (int)words);
}
AHL_DEV void clamp_record(bool clamped, int row, uint32_t& words) {
  clamp_record_bits(__builtin_amdgcn_ballot_w64(clamped), row, words);
}

// Zeroes the elements of a vector of 8 bf16 whose bit in the low byte of `bits` is set.
AHL_DEV u32x4 clamp_apply8(const u32x4& v, uint32_t bits) {
  // per pair of elements: 0x0000ffff for the even bit, 0xffff0000 for the odd one
  auto pair = [&](uint32_t x, int i) -> uint32_t {
    const uint32_t lo = ((bits >> (2 * i)) & 1u) * 0xffffu;
    const uint32_t hi = (uint32_t)(((int32_t)(bits << (30 - 2 * i))) >> 31) << 16;
    return x & ~(lo | hi);
  };
  u32x4 o = {pair(v.x, 0), pair(v.y, 1), pair(v.z, 2), pair(v.w, 3)};
  return o;
}

AHL_DEV float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}
AHL_DEV float wave_min(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fminf(v, __shfl_xor(v, o, 64));
  return v;
}
AHL_DEV float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
AHL_DEV double wave_sum(double v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

AHL_DEV int64_t cdiv_dev(int64_t a, int64_t b) { return (a + b - 1) / b; }

// 16-byte global load / store of one `vec`
AHL_DEV u32x4 ld16(const void* p) { return *(const u32x4*)p; }
AHL_DEV void st16(void* p, const u32x4& v) { *(u32x4*)p = v; }
// The same for data that is touched once (streaming passes over a whole matrix): non-temporal, so
// that the lines do not displace what other kernels keep in the caches.
AHL_DEV u32x4 ld16_stream(const void* p) { return __builtin_nontemporal_load((const u32x4*)p); }
AHL_DEV void st16_stream(void* p, const u32x4& v) { __builtin_nontemporal_store(v, (u32x4*)p); }

}  // namespace ahl

namespace ahl {

// ---------------------------------------------------------------------------------------------
// DAC: clamp to the input range and quantise (Appendix of the torch-mode arithmetic):
//   r = step(ir, inp_res); q = rd(xc / max(r, tiny)); q = rne(q); xq = rd(q * r)
// (reference torch_utils/quant_utils.py:63-99 called from torch_utils/torch_linear.py:182-192).
struct Dac {
  float ir;    // clamp bound (ignored when clamp is off)
  float r;     // quantisation step (unclamped; the product uses this one)
  float rc;    // max(r, tiny): the divisor
  float rcp;   // 1 / rc
};

template <class D>
AHL_DEV Dac make_dac(float ir, float inp_res) {
  Dac d;
  d.ir = ir;
  d.r = inp_res > 0.0f ? quant_step<D>(ir, inp_res) : 1.0f;
  d.rc = fmaxf(d.r, D::tiny());
  d.rcp = __fdiv_rn(1.0f, d.rc);
  return d;
}

template <class D, bool CLAMP, bool QUANT>
AHL_DEV float dac_apply(float x, const Dac& d, bool skip_rounding) {
  float v = x;
  if (CLAMP) v = fminf(fmaxf(v, -d.ir), d.ir);
  if (QUANT) {
    float q = D::rd(D::div_exact_rcp(v, d.rc, d.rcp));
    if (!skip_rounding) q = rintf(q);  // v_rndne_f32: round half to even like torch.round
    v = D::rd(q * d.r);
  }
  return v;
}

// Iterates one wave over the columns [c0, c1) of a row; f(value) is called once per element.
// VEC: the row base (p + row*ld) is 16-byte aligned, so whole `vec`s can be loaded for the
// aligned middle part; head and tail are done element-wise.
// U 16-byte loads are in flight per lane before the first value is used (a lane's elements still
// arrive in ascending column order, so sums do not depend on U): the compiler does not move a
// load across per-element work such as LDS atomics, and a wave that walks its row with one load
// in flight is bound by that load's latency.
template <class D, bool VEC, int U, class F>
AHL_DEV void wave_row_foreach_n(const void* row, int32_t c0, int32_t c1, int lane, F f) {
  if (VEC) {
    constexpr int E = D::EPV;
    int32_t a0 = (c0 + E - 1) / E * E;
    int32_t a1 = c1 / E * E;
    if (a0 > a1) { a0 = c1; a1 = c1; }
    for (int32_t c = c0 + lane; c < a0; c += 64) f(D::load(row, c));
    const typename D::elem* base = (const typename D::elem*)row;
    const int32_t v1 = a1 / E;
    for (int32_t v = a0 / E + lane; v < v1; v += 64 * U) {
      u32x4 x[U];
#pragma unroll
      for (int u = 0; u < U; ++u) x[u] = ld16(base + (int64_t)(v + 64 * u < v1 ? v + 64 * u : v) * E);
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (v + 64 * u < v1) {
          float e[E];
          D::unpack(x[u], e);
#pragma unroll
          for (int i = 0; i < E; ++i) f(e[i]);
        }
      }
    }
    for (int32_t c = a1 + lane; c < c1; c += 64) f(D::load(row, c));
  } else {
    for (int32_t c = c0 + lane; c < c1; c += 64) f(D::load(row, c));
  }
}

template <class D, bool VEC, class F>
AHL_DEV void wave_row_foreach(const void* row, int32_t c0, int32_t c1, int lane, F f) {
  wave_row_foreach_n<D, VEC, 2>(row, c0, c1, lane, f);
}

}  // namespace ahl
