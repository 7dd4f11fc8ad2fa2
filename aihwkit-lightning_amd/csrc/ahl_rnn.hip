// Gate arithmetic of the recurrent cells as one kernel per direction of differentiation.
//
// A recurrent step of the reference (nn/modules/rnn/cells.py:176-186 LSTM, :321-343 GRU) is two
// analog products followed by about ten element-wise torch operations, and about twenty more in
// the backward pass: at the sizes of a step (batch x hidden elements) every one of them is a
// launch that moves a few hundred kilobytes. These kernels do the same arithmetic in one pass
// each. They round where the chain of torch operations rounds (after every operation in the
// layer's dtype; an activation and its derivative are evaluated in fp32 and rounded once, as
// torch's GPU kernels do), so results are those of the unfused chain.
//
// Layout: all matrices row-major and dense; gates [rows, G * hidden] with the gate blocks in the
// reference's order (LSTM: input, forget, cell, output; GRU: reset, update, new). A thread owns
// one 16-byte vector of consecutive hidden units of one row: hidden must be a multiple of 8
// (bf16) or 4 (fp32).
#include "ahl_host.h"

namespace ahl {

AHL_DEV float sigmoid_f(float x) { return __fdiv_rn(1.0f, 1.0f + expf(-x)); }

template <class D>
struct Vec {
  float v[D::EPV];
  AHL_DEV void load(const void* base, int64_t idx) {
    D::unpack(ld16((const typename D::elem*)base + idx), v);
  }
  AHL_DEV void store(void* base, int64_t idx) const {
    st16((typename D::elem*)base + idx, D::pack(v));
  }
};

// act [rows, 4H] receives the activated gates (i, f, g, o) when not null.
template <class D>
__global__ __launch_bounds__(256) void k_lstm_gates_fwd(const void* __restrict__ ig,
                                                        const void* __restrict__ hg,
                                                        const void* __restrict__ cx, int64_t rows,
                                                        int64_t hidden, void* __restrict__ hy,
                                                        void* __restrict__ cy,
                                                        void* __restrict__ act) {
  constexpr int E = D::EPV;
  const int64_t vpr = hidden / E;
  const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (t >= rows * vpr) return;
  const int64_t r = t / vpr, h0 = (t - r * vpr) * E;
  const int64_t g0 = r * 4 * hidden + h0, s0 = r * hidden + h0;
  Vec<D> gate[4], c, add;
#pragma unroll
  for (int k = 0; k < 4; ++k) gate[k].load(ig, g0 + k * hidden);
  if (hg != nullptr) {
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      add.load(hg, g0 + k * hidden);
#pragma unroll
      for (int e = 0; e < E; ++e) gate[k].v[e] = D::rd(gate[k].v[e] + add.v[e]);
    }
  }
  c.load(cx, s0);
  Vec<D> out_h, out_c;
#pragma unroll
  for (int e = 0; e < E; ++e) {
    const float i = D::rd(sigmoid_f(gate[0].v[e]));
    const float f = D::rd(sigmoid_f(gate[1].v[e]));
    const float g = D::rd(tanhf(gate[2].v[e]));
    const float o = D::rd(sigmoid_f(gate[3].v[e]));
    const float cn = D::rd(D::rd(f * c.v[e]) + D::rd(i * g));
    out_c.v[e] = cn;
    out_h.v[e] = D::rd(o * D::rd(tanhf(cn)));
    gate[0].v[e] = i; gate[1].v[e] = f; gate[2].v[e] = g; gate[3].v[e] = o;
  }
  out_h.store(hy, s0);
  out_c.store(cy, s0);
  if (act != nullptr) {
#pragma unroll
    for (int k = 0; k < 4; ++k) gate[k].store(act, g0 + k * hidden);
  }
}

// dgates [rows, 4H]: gradient of the summed pre-activations (the same for the input and the
// hidden projection); dcx [rows, H]. dcy may be null (the cell state is not used downstream).
template <class D>
__global__ __launch_bounds__(256) void k_lstm_gates_bwd(const void* __restrict__ dhy,
                                                        const void* __restrict__ dcy,
                                                        const void* __restrict__ act,
                                                        const void* __restrict__ cx,
                                                        const void* __restrict__ cy, int64_t rows,
                                                        int64_t hidden, void* __restrict__ dgates,
                                                        void* __restrict__ dcx) {
  constexpr int E = D::EPV;
  const int64_t vpr = hidden / E;
  const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (t >= rows * vpr) return;
  const int64_t r = t / vpr, h0 = (t - r * vpr) * E;
  const int64_t g0 = r * 4 * hidden + h0, s0 = r * hidden + h0;
  Vec<D> a[4], c_old, c_new, dh, dc;
#pragma unroll
  for (int k = 0; k < 4; ++k) a[k].load(act, g0 + k * hidden);
  c_old.load(cx, s0);
  c_new.load(cy, s0);
  dh.load(dhy, s0);
  if (dcy != nullptr) dc.load(dcy, s0);
  Vec<D> out_dc;
#pragma unroll
  for (int e = 0; e < E; ++e) {
    const float i = a[0].v[e], f = a[1].v[e], g = a[2].v[e], o = a[3].v[e];
    const float tc = D::rd(tanhf(c_new.v[e]));
    const float d_o = D::rd(dh.v[e] * tc);
    const float d_tc = D::rd(dh.v[e] * o);
    float d_c = D::rd(d_tc * (1.0f - tc * tc));
    if (dcy != nullptr) d_c = D::rd(dc.v[e] + d_c);
    const float d_f = D::rd(d_c * c_old.v[e]);
    out_dc.v[e] = D::rd(d_c * f);
    const float d_i = D::rd(d_c * g);
    const float d_g = D::rd(d_c * i);
    a[0].v[e] = D::rd(d_i * (1.0f - i) * i);
    a[1].v[e] = D::rd(d_f * (1.0f - f) * f);
    a[2].v[e] = D::rd(d_g * (1.0f - g * g));
    a[3].v[e] = D::rd(d_o * (1.0f - o) * o);
  }
#pragma unroll
  for (int k = 0; k < 4; ++k) a[k].store(dgates, g0 + k * hidden);
  out_dc.store(dcx, s0);
}

// act [rows, 3H] receives (reset, update, new) when not null.
template <class D>
__global__ __launch_bounds__(256) void k_gru_gates_fwd(const void* __restrict__ ig,
                                                       const void* __restrict__ hg,
                                                       const void* __restrict__ hx, int64_t rows,
                                                       int64_t hidden, void* __restrict__ hy,
                                                       void* __restrict__ act) {
  constexpr int E = D::EPV;
  const int64_t vpr = hidden / E;
  const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (t >= rows * vpr) return;
  const int64_t r = t / vpr, h0 = (t - r * vpr) * E;
  const int64_t g0 = r * 3 * hidden + h0, s0 = r * hidden + h0;
  Vec<D> gi[3], gh[3], h, out;
#pragma unroll
  for (int k = 0; k < 3; ++k) { gi[k].load(ig, g0 + k * hidden); gh[k].load(hg, g0 + k * hidden); }
  h.load(hx, s0);
#pragma unroll
  for (int e = 0; e < E; ++e) {
    const float rg = D::rd(sigmoid_f(D::rd(gi[0].v[e] + gh[0].v[e])));
    const float z = D::rd(sigmoid_f(D::rd(gi[1].v[e] + gh[1].v[e])));
    const float n = D::rd(tanhf(D::rd(gi[2].v[e] + D::rd(rg * gh[2].v[e]))));
    out.v[e] = D::rd(n + D::rd(z * D::rd(h.v[e] - n)));
    gi[0].v[e] = rg; gi[1].v[e] = z; gi[2].v[e] = n;
  }
  out.store(hy, s0);
  if (act != nullptr) {
#pragma unroll
    for (int k = 0; k < 3; ++k) gi[k].store(act, g0 + k * hidden);
  }
}

// digates / dhgates [rows, 3H]: gradients of the input and the hidden projection's outputs (they
// differ in the "new" block: the reset gate scales the hidden part only); dhx [rows, H]: the
// direct path h -> h' (the path through the hidden projection is the projection's own backward).
template <class D>
__global__ __launch_bounds__(256) void k_gru_gates_bwd(const void* __restrict__ dhy,
                                                       const void* __restrict__ act,
                                                       const void* __restrict__ hg,
                                                       const void* __restrict__ hx, int64_t rows,
                                                       int64_t hidden, void* __restrict__ digates,
                                                       void* __restrict__ dhgates,
                                                       void* __restrict__ dhx) {
  constexpr int E = D::EPV;
  const int64_t vpr = hidden / E;
  const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (t >= rows * vpr) return;
  const int64_t r = t / vpr, h0 = (t - r * vpr) * E;
  const int64_t g0 = r * 3 * hidden + h0, s0 = r * hidden + h0;
  Vec<D> a[3], hn, h, dh, d_in[3], d_hn, d_h;
#pragma unroll
  for (int k = 0; k < 3; ++k) a[k].load(act, g0 + k * hidden);
  hn.load(hg, g0 + 2 * hidden);
  h.load(hx, s0);
  dh.load(dhy, s0);
#pragma unroll
  for (int e = 0; e < E; ++e) {
    const float rg = a[0].v[e], z = a[1].v[e], n = a[2].v[e];
    const float diff = D::rd(h.v[e] - n);
    const float d_z = D::rd(dh.v[e] * diff);
    const float d_diff = D::rd(dh.v[e] * z);
    const float d_n = D::rd(dh.v[e] - d_diff);          // dh + (-d_diff)
    const float d_pre = D::rd(d_n * (1.0f - n * n));
    const float d_r = D::rd(d_pre * hn.v[e]);
    d_hn.v[e] = D::rd(d_pre * rg);
    d_in[0].v[e] = D::rd(d_r * (1.0f - rg) * rg);
    d_in[1].v[e] = D::rd(d_z * (1.0f - z) * z);
    d_in[2].v[e] = d_pre;
    d_h.v[e] = d_diff;
  }
#pragma unroll
  for (int k = 0; k < 3; ++k) d_in[k].store(digates, g0 + k * hidden);
  d_in[0].store(dhgates, g0);
  d_in[1].store(dhgates, g0 + hidden);
  d_hn.store(dhgates, g0 + 2 * hidden);
  d_h.store(dhx, s0);
}

static bool gate_args_ok(int32_t dtype, int64_t rows, int64_t hidden, int64_t* blocks) {
  if (rows <= 0 || hidden <= 0 || !dtype_known(dtype)) return false;
  const int epv = dtype == AHL_F32 ? 4 : 8;
  if (hidden % epv != 0) return false;
  *blocks = cdiv(rows * (hidden / epv), 256);
  return *blocks <= 0x7fffffff;
}

}  // namespace ahl

using namespace ahl;

#define AHL_ALIGNED_ALL(...)                              \
  do {                                                    \
    const void* ptrs[] = {__VA_ARGS__};                   \
    for (const void* p : ptrs)                            \
      if (p != nullptr && !aligned16(p)) return AHL_ERR_ARG; \
  } while (0)

extern "C" int ahl_lstm_gates_fwd(const void* igates, const void* hgates, const void* cx,
                                  int32_t dtype, int64_t rows, int64_t hidden, void* hy, void* cy,
                                  void* act, void* stream) {
  int64_t blocks;
  if (!igates || !cx || !hy || !cy || !gate_args_ok(dtype, rows, hidden, &blocks)) return AHL_ERR_ARG;
  AHL_ALIGNED_ALL(igates, hgates, cx, hy, cy, act);
  AHL_DISPATCH_DTYPE(dtype, {
    hipLaunchKernelGGL((k_lstm_gates_fwd<D>), dim3((unsigned)blocks), dim3(256), 0,
                       (hipStream_t)stream, igates, hgates, cx, rows, hidden, hy, cy, act);
  });
  return check_launch("ahl_lstm_gates_fwd");
}

extern "C" int ahl_lstm_gates_bwd(const void* dhy, const void* dcy, const void* act, const void* cx,
                                  const void* cy, int32_t dtype, int64_t rows, int64_t hidden,
                                  void* dgates, void* dcx, void* stream) {
  int64_t blocks;
  if (!dhy || !act || !cx || !cy || !dgates || !dcx || !gate_args_ok(dtype, rows, hidden, &blocks))
    return AHL_ERR_ARG;
  AHL_ALIGNED_ALL(dhy, dcy, act, cx, cy, dgates, dcx);
  AHL_DISPATCH_DTYPE(dtype, {
    hipLaunchKernelGGL((k_lstm_gates_bwd<D>), dim3((unsigned)blocks), dim3(256), 0,
                       (hipStream_t)stream, dhy, dcy, act, cx, cy, rows, hidden, dgates, dcx);
  });
  return check_launch("ahl_lstm_gates_bwd");
}

extern "C" int ahl_gru_gates_fwd(const void* igates, const void* hgates, const void* hx,
                                 int32_t dtype, int64_t rows, int64_t hidden, void* hy, void* act,
                                 void* stream) {
  int64_t blocks;
  if (!igates || !hgates || !hx || !hy || !gate_args_ok(dtype, rows, hidden, &blocks))
    return AHL_ERR_ARG;
  AHL_ALIGNED_ALL(igates, hgates, hx, hy, act);
  AHL_DISPATCH_DTYPE(dtype, {
    hipLaunchKernelGGL((k_gru_gates_fwd<D>), dim3((unsigned)blocks), dim3(256), 0,
                       (hipStream_t)stream, igates, hgates, hx, rows, hidden, hy, act);
  });
  return check_launch("ahl_gru_gates_fwd");
}

extern "C" int ahl_gru_gates_bwd(const void* dhy, const void* act, const void* hgates,
                                 const void* hx, int32_t dtype, int64_t rows, int64_t hidden,
                                 void* digates, void* dhgates, void* dhx, void* stream) {
  int64_t blocks;
  if (!dhy || !act || !hgates || !hx || !digates || !dhgates || !dhx ||
      !gate_args_ok(dtype, rows, hidden, &blocks))
    return AHL_ERR_ARG;
  AHL_ALIGNED_ALL(dhy, act, hgates, hx, digates, dhgates, dhx);
  AHL_DISPATCH_DTYPE(dtype, {
    hipLaunchKernelGGL((k_gru_gates_bwd<D>), dim3((unsigned)blocks), dim3(256), 0,
                       (hipStream_t)stream, dhy, act, hgates, hx, rows, hidden, digates, dhgates,
                       dhx);
  });
  return check_launch("ahl_gru_gates_bwd");
}
