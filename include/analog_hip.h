/*
 * analog_hip.h -- C ABI of libanalog_hip.so: the AnalogLinear hot path on MI355X (gfx950).
 *
 * Conventions
 *   - Every entry point returns an int status (AHL_OK == 0). Nothing throws, nothing allocates,
 *     nothing synchronises: work is enqueued on the hipStream_t passed as `stream` (a void*;
 *     NULL is the default stream). All data pointers are DEVICE pointers unless a parameter is
 *     named *_host. The caller owns every buffer, including scratch ("ws_*" parameters).
 *   - Matrices are row-major with an explicit leading dimension in ELEMENTS.
 *   - dtype is AHL_F32, AHL_BF16 or AHL_F16 and applies to every pointer documented as "dtype".
 *     In AHL_BF16 / AHL_F16 every elementwise result is rounded to the 16-bit type
 *     (round-to-nearest-even) exactly where the reference's torch-mode rounds when it runs on
 *     tensors of that type. Both 16-bit types have the MFMA kernels for large shapes (the
 *     reference's accelerated slot takes float32 and float16, triton_utils/triton_linear.py:630);
 *     AHL_F32 runs on general kernels.
 *   - K-tiles ("analog tiles" along the input dimension) are described by `tile_ends_host`,
 *     the reference's `upper_end_of_slices` (nn/modules/linear.py:76-80) as a HOST int32 array
 *     of n_tiles cumulative end offsets. It must follow the reference's split rule
 *     (nn/modules/linear.py:155-170); anything else returns AHL_ERR_TILING.
 *
 * Each entry point cites the reference code it replaces (paths relative to the reference's
 * src/aihwkit_lightning/).
 */
#ifndef ANALOG_HIP_H_
#define ANALOG_HIP_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- status codes ------------------------------------------------------------------------- */
#define AHL_OK 0
#define AHL_ERR_ARG 1          /* null pointer, negative size, bad enum                          */
#define AHL_ERR_TILING 2       /* tile_ends_host does not follow the reference split rule        */
#define AHL_ERR_UNSUPPORTED 3  /* valid in the reference but not implemented here                 */
#define AHL_ERR_LAUNCH 4       /* hipLaunchKernel reported an error (see ahl_last_hip_error)      */
#define AHL_ERR_WORKSPACE 5    /* a ws_* buffer is too small                                      */

/* ---- enums -------------------------------------------------------------------------------- */
#define AHL_F32 0
#define AHL_BF16 1
#define AHL_F16 2

#define AHL_IR_NONE 0     /* input range disabled: no clamp, no DAC                               */
#define AHL_IR_STATIC 1   /* one scalar per tile, ir[n_tiles] (learned or calibrated)             */
#define AHL_IR_DYNAMIC 2  /* per token and tile abs-max, ir[n_tiles, M]                           */

#define AHL_NOISE_NONE 0
#define AHL_NOISE_ADD_NORMAL 1              /* std = std_dev * max|W_tile|          */
#define AHL_NOISE_ADD_NORMAL_PER_CHANNEL 2  /* std = std_dev * max|W_tile[n, :]|    */

/* Backward of the clamp to a static input range (AhlLinearCfg.ir_grad_rule):
 * AHL_IR_GRAD_LEARNED: StraightThroughClamp + InputRangeForward (torch_utils/torch_linear.py:29-108)
 *   ir_grad[t] = (sum_{x >= ir} min(d, 0) - sum_{x <= -ir} max(d, 0)) * ir[t] + decay switch
 * AHL_IR_GRAD_CLAMP: autograd of torch.clamp(x, -ir, ir) with tensor bounds, the fast_mode path
 *   (torch_utils/torch_linear.py:361-422): ir_grad[t] = sum_{x > ir} d - sum_{x < -ir} d
 * Both zero dx where |x| > ir[t].                                                         */
#define AHL_IR_GRAD_LEARNED 0
#define AHL_IR_GRAD_CLAMP 1

#define AHL_QUANT_NONE 0
#define AHL_QUANT_DISCRETIZE 1              /* scale from max|W_tile|               */
#define AHL_QUANT_DISCRETIZE_PER_CHANNEL 2  /* scale from max|W_tile[n, :]|         */
#define AHL_QUANT_CLIP_LEARNED 3            /* no quantiser, clamp(w / c, -1, 1) * c with the
                                               learnable clip c (needs wmax_given)   */

#define AHL_CLIP_LAYER 0        /* one std over the whole matrix   */
#define AHL_CLIP_PER_CHANNEL 1  /* one std per output channel (row) */

/* Forward/backward behaviour of one AnalogLinear call; a flattened
 * TorchInferenceRPUConfig (simulator/configs/configs.py:27-88) plus call state.          */
typedef struct AhlLinearCfg {
  int32_t dtype;                 /* AHL_F32 | AHL_BF16 | AHL_F16                                */
  int32_t ir_mode;               /* AHL_IR_*                                                    */
  float inp_res;                 /* forward.inp_res; <= 0 switches the DAC off                  */
  float out_res;                 /* forward.out_res; <= 0 switches ADC quantisation off         */
  float out_bound;               /* forward.out_bound; <= 0 switches the output clamp off       */
  float out_noise;               /* forward.out_noise; used only when training != 0             */
  int32_t out_noise_per_channel; /* forward.out_noise_per_channel                               */
  int32_t bound_per_channel;     /* clip.type is one of the *_PER_CHANNEL kinds                 */
  int32_t training;              /* module.training                                             */
  int32_t skip_rounding;         /* the reference's test switch _AIHWKIT_NO_ROUNDING            */
  float ir_decay;                /* pre_post.input_range.decay                                  */
  float ir_input_min_percentage; /* pre_post.input_range.input_min_percentage                   */
  int32_t ir_grad_rule;          /* AHL_IR_GRAD_*: which backward the static range clamp has     */
  int32_t tile_stride;           /* 0: xq and w_eff are dense [rows, K]. > 0: they are in the
                                    padded tile layout with this stride (see ahl_tile_stride)    */
  uint32_t flag_token;           /* what "something was clamped" looks like in the one-word
                                    clamp_flag. 0: ahl_linear_fwd clears the word (one small
                                    launch) and sets it non-zero; the backward entry points read
                                    "non-zero". != 0: the forward stores this value and clears
                                    nothing, the backward reads "equal to this value" -- pass the
                                    same cfg to both, and a value that differs from call to call:
                                    a stale or accidental match only makes the backward apply a
                                    mask that clamps nothing. Launches recorded into a HIP graph
                                    repeat their by-value arguments on every replay: record them
                                    with 0 (the clearing launch is a kernel and is recorded too)  */
  uint64_t seed;                 /* Philox key for this call                                    */
  uint64_t offset;               /* Philox counter offset for this call                         */
  const uint64_t* seed_state;    /* NULL, or a DEVICE uint64[2] = {key, call counter}: the kernels
                                    then take the key from [0] and add [1] to `offset`. For
                                    launches recorded into a HIP graph, whose by-value arguments
                                    would repeat the same noise on every replay: record an
                                    ahl_seed_advance on the state in front of them               */
} AhlLinearCfg;

/* Weight modifier of the training forward / post-training quantisation; a flattened
 * WeightModifierParameter (simulator/parameters/inference.py:29-71).                     */
typedef struct AhlModifierCfg {
  int32_t dtype;
  int32_t quant_type; /* AHL_QUANT_*                                                            */
  int32_t noise_type; /* AHL_NOISE_* (ignored by ahl_quantize_weights)                          */
  float res;          /* modifier.res (number of states, or its inverse). The number of states
                         is max(res, 1 / res) in float: callers that hold the inverse in double
                         should pass the number of states (1 / (1 / 30) is not 30 in float)   */
  float std_dev;      /* modifier.std_dev                                                       */
  int32_t wmax_given; /* != 0: wmax[T, N] is an input (clip.type LEARNABLE_PER_CHANNEL: the
                         learnable_weight_clip takes the place of the per-tile abs-max,
                         torch_utils/torch_linear.py:222-244) instead of being computed            */
  int32_t skip_tile_stats; /* != 0: the caller does not need tile_max / tile_min (every consumer
                              scales per channel); ahl_weight_prep may then leave them unwritten  */
  uint64_t seed;
  uint64_t offset;
  const uint64_t* seed_state; /* as in AhlLinearCfg                                             */
} AhlModifierCfg;

/* ---- padded tile layout ------------------------------------------------------------------
 * The MFMA kernels of the 16-bit dtypes want every K-tile to start on a 256-column boundary. The
 * reference's split rule (nn/modules/linear.py:155-170) gives that only for some shapes
 * (4096 inputs in tiles of 512 do, 11008 in tiles of 512 or 2304 in tiles of 576 do not). For
 * the others the two operands the library produces itself -- the quantised input xq (ahl_dac)
 * and the effective weights w_eff -- can be kept in a padded layout: tile t starts at column
 * t * tile_stride, holds its size(t) columns and is zero up to the next tile; a row has
 * n_tiles * tile_stride columns. Zeros add nothing to any product, so results do not change.
 * Tensors the caller owns (x, y, dx, dw) stay dense.                                          */

/* The stride the fast kernels want for this split: 0 if the dense layout already suits them or
 * the dtype has no fast kernels, else ceil(K / n_tiles) rounded up to a multiple of 256.       */
int64_t ahl_tile_stride(int64_t K, int32_t n_tiles, int32_t dtype);

/* dst[r, t * tile_stride + j] = src[r, start(t) + j] for j < size(t), 0 for the rest of the
 * stride; src dtype [rows, K] (row stride ld_src), dst dtype [rows, n_tiles * tile_stride].    */
int ahl_pad_tiles(const void* src, int64_t ld_src, int32_t dtype, int64_t rows, int64_t K,
                  const int32_t* tile_ends_host, int32_t n_tiles, int64_t tile_stride, void* dst,
                  int64_t ld_dst, void* stream);

/* The inverse copy: dst[r, start(t) + j] = src[r, t * tile_stride + j].                        */
int ahl_unpad_tiles(const void* src, int64_t ld_src, int32_t dtype, int64_t rows, int64_t K,
                    const int32_t* tile_ends_host, int32_t n_tiles, int64_t tile_stride, void* dst,
                    int64_t ld_dst, void* stream);

/* ---- library ------------------------------------------------------------------------------ */

/* ABI version of this header; bumped when a signature changes. */
int ahl_abi_version(void);
/* Text of the last HIP error seen by a launcher on this thread ("" if none). */
const char* ahl_last_hip_error(void);

/* state[1] += delta for a device-resident noise state uint64[2] = {Philox key, call counter}
 * (AhlLinearCfg.seed_state): one small launch, so that every replay of a recorded graph draws
 * new noise. The reference draws one seed per call on the host (triton_utils/
 * triton_linear.py:541,617); this is that draw for callers whose launches are replayed.        */
int ahl_seed_advance(uint64_t* state, uint64_t delta, void* stream);

/* ---- reductions (memory-bound) ------------------------------------------------------------ */

/* Per-tile, per-row abs-max of x[rows, cols]: out[t, r] = max_{c in tile t} |x[r, c]|.
 * out is dtype [n_tiles, rows]. Optionally also tile_max[t] = max_r out[t, r] and
 * tile_min[t] = min_r out[t, r] as float (pass NULL to skip both).
 * Replaces nn/modules/torch_utils/torch_abs_max.py:17-39 (weights [N,K] -> [T,N]),
 * the per-forward amax at torch_utils/torch_linear.py:220, and the dynamic input range
 * at torch_linear.py:155-157 (x [M,K] -> [T,M]); Triton counterpart
 * triton_utils/triton_abs_max.py:232-327.                                                */
int ahl_sliced_absmax(const void* x, int32_t dtype, int64_t rows, int64_t cols, int64_t ld,
                      const int32_t* tile_ends_host, int32_t n_tiles, void* out, float* tile_max,
                      float* tile_min, void* stream);

/* Per-tile unbiased standard deviation over ALL rows: out[t] = std(x[:, tile t]) as float.
 * ws_partials needs ahl_sliced_std_ws_bytes(rows, n_tiles) bytes.
 * Replaces `values.std()` at torch_utils/torch_linear.py:342; Triton counterpart
 * triton_utils/triton_std.py:184-245.                                                    */
int ahl_sliced_std(const void* x, int32_t dtype, int64_t rows, int64_t cols, int64_t ld,
                   const int32_t* tile_ends_host, int32_t n_tiles, float* out, void* ws_partials,
                   void* stream);
int64_t ahl_sliced_std_ws_bytes(int64_t rows, int32_t n_tiles);

/* ---- calibration statistics (inference/calibration/calibration.py:57-152) -------------------
 * The reference drops the rows of a batch that are entirely zero before it takes a statistic
 * (`x_input[~(x_input == 0.0).all(-1)]`, calibration.py:95); "kept rows" below are the others. */

/* kept[r] = 1 unless x[r, :] == 0 everywhere (uint8 [rows]); *n_kept = number of kept rows.     */
int ahl_row_nonzero(const void* x, int32_t dtype, int64_t rows, int64_t cols, int64_t ld,
                    uint8_t* kept, uint32_t* n_kept, void* stream);

/* out[t] = unbiased std of x[kept rows, tile t] as float (MOVING_STD, calibration.py:140-142).
 * ws needs ahl_sliced_std_kept_ws_bytes(rows, n_tiles) bytes.                                  */
int ahl_sliced_std_kept(const void* x, int32_t dtype, int64_t rows, int64_t cols, int64_t ld,
                        const int32_t* tile_ends_host, int32_t n_tiles, float* out, void* ws,
                        void* stream);
int64_t ahl_sliced_std_kept_ws_bytes(int64_t rows, int32_t n_tiles);

/* out[t] = torch.quantile(x[kept rows, tile t].float().flatten(), q) (linear interpolation;
 * NaN if the tile holds a NaN or no row is kept), exact, by radix selection on the device
 * (MOVING_QUANTILE and CACHE_QUANTILE, calibration.py:133-138, :305-313).
 * ws needs ahl_sliced_quantile_ws_bytes(rows, n_tiles) bytes.                                  */
int ahl_sliced_quantile(const void* x, int32_t dtype, int64_t rows, int64_t cols, int64_t ld,
                        const int32_t* tile_ends_host, int32_t n_tiles, float q, float* out,
                        void* ws, void* stream);
int64_t ahl_sliced_quantile_ws_bytes(int64_t rows, int32_t n_tiles);

/* Moving average of the calibrated range (calibration.py:144-147), on the device:
 *   ir[t] = dtype((float(ir[t]) * idx[t] + float(alpha * val[t])) / (idx[t] + 1)); idx[t] += 1
 * ir dtype [T], idx int32 [T], val float [T]; val_in_dtype != 0 rounds val to dtype first (a std
 * that torch returns in the tensor dtype). A tile whose val is NaN (no kept row in the batch) is
 * left as it is, idx included.                                                                 */
int ahl_ir_moving_update(void* ir, int32_t* idx, const float* val, int32_t dtype, int32_t n_tiles,
                         double alpha, int32_t val_in_dtype, void* stream);

/* Gate arithmetic of the recurrent cells in one pass per direction: everything between the two
 * analog products of a step and the new state. Replaces the element-wise torch operations of
 * nn/modules/rnn/cells.py:176-186 (LSTM: gates = igates + hgates; i, f, g, o = sigmoid / tanh of
 * the four blocks; c' = f c + i g; h' = o tanh(c')) and :321-343 (GRU: r = sigmoid(i_r + h_r);
 * z = sigmoid(i_z + h_z); n = tanh(i_n + r h_n); h' = n + z (h - n)) and what autograd derives
 * from them, with the dtype rounding after every operation that the torch chain has.
 * All matrices dense row-major, 16-byte aligned; gates [rows, 4 hidden] / [rows, 3 hidden], states
 * [rows, hidden]; hidden a multiple of 8 (bf16, fp16) or 4 (fp32).
 * lstm fwd: hgates may be null (one product over [x, h], cells.py:244-267); act [rows, 4 hidden]
 *   receives the activated gates for the backward pass (null: not wanted).
 * lstm bwd: dcy may be null (c' unused downstream); dgates is the gradient of both products'
 *   outputs; dcx that of the previous cell state.
 * gru fwd: act [rows, 3 hidden] receives r, z, n (null: not wanted).
 * gru bwd: digates / dhgates are the gradients of the input / hidden product's outputs, dhx the
 *   direct path from the previous hidden state.                                              */
int ahl_lstm_gates_fwd(const void* igates, const void* hgates, const void* cx, int32_t dtype,
                       int64_t rows, int64_t hidden, void* hy, void* cy, void* act, void* stream);
int ahl_lstm_gates_bwd(const void* dhy, const void* dcy, const void* act, const void* cx,
                       const void* cy, int32_t dtype, int64_t rows, int64_t hidden, void* dgates,
                       void* dcx, void* stream);
int ahl_gru_gates_fwd(const void* igates, const void* hgates, const void* hx, int32_t dtype,
                      int64_t rows, int64_t hidden, void* hy, void* act, void* stream);
int ahl_gru_gates_bwd(const void* dhy, const void* act, const void* hgates, const void* hx,
                      int32_t dtype, int64_t rows, int64_t hidden, void* digates, void* dhgates,
                      void* dhx, void* stream);

/* Input-range initialisation from data, all tiles, no host sync:
 *   if idx[t] < init_from_data: if std[t] > 0 { ir[t] = (ir[t]*idx[t] + alpha*std[t])/(idx[t]+1);
 *   idx[t] += 1 }  ir[t] = |ir[t]|.   ir and idx are dtype [n_tiles], updated in place.
 * Replaces torch_utils/torch_linear.py:338-352.                                          */
int ahl_ir_init_update(void* ir, void* idx, const float* std, int32_t dtype, int32_t n_tiles,
                       float init_from_data, float init_std_alpha, void* stream);

/* Running per-tile abs-max for input-range calibration:
 *   cache[t] = max(cache[t], max_{r, c in tile t} |x[r, c]|), cache is float [n_tiles]
 *   (initialise to -inf). Replaces inference/calibration/calibration.py:110-124.         */
int ahl_running_absmax(const void* x, int32_t dtype, int64_t rows, int64_t cols, int64_t ld,
                       const int32_t* tile_ends_host, int32_t n_tiles, float* cache, void* stream);

/* fast_mode input range (TorchLinear.apply_input_range_fast, torch_utils/torch_linear.py:361-419),
 * the update only: for every tile with idx[t] < init_from_data, the signed min / max of
 * x[:, tile t] moves x_min[t] / x_max[t] (first batch: added to the initial +-1e-5; momentum -1:
 * running extrema; else exponential average), idx[t] += 1, ir[t] = max(|x_min[t]|, |x_max[t]|).
 * ir, idx, x_min, x_max: dtype [T], updated in place on the device, no host sync. The clamp
 * itself is the AHL_IR_STATIC forward; its backward is AHL_IR_GRAD_CLAMP.
 * ws needs ahl_ir_fast_update_ws_bytes(rows, n_tiles) bytes.                               */
int ahl_ir_fast_update(const void* x, int32_t dtype, int64_t rows, int64_t cols, int64_t ld,
                       const int32_t* tile_ends_host, int32_t n_tiles, void* ir, void* idx,
                       void* x_min, void* x_max, float init_from_data, double momentum, void* ws,
                       void* stream);
int64_t ahl_ir_fast_update_ws_bytes(int64_t rows, int32_t n_tiles);

/* Weight clipping after an optimizer step, in place on w[rows, cols]:
 *   bound = sigma * std_unbiased(w[r, :]) (AHL_CLIP_PER_CHANNEL) or sigma * std_unbiased(w);
 *   w = clamp(w, -bound, bound).  ws needs ahl_clip_weights_ws_bytes(rows) bytes.
 * Replaces AnalogLinear.clip_weights, nn/modules/linear.py:269-283.                      */
int ahl_clip_weights(void* w, int32_t dtype, int64_t rows, int64_t cols, int64_t ld, float sigma,
                     int32_t clip_kind, void* ws, void* stream);
int64_t ahl_clip_weights_ws_bytes(int64_t rows);

/* Column sums: out[c] = sum_r x[r, c] (float accumulate, rounded once to dtype).
 * ws needs ahl_col_sum_ws_bytes(cols) bytes.
 * The bias gradient of `out + bias`, torch_utils/torch_linear.py:314.                    */
int ahl_col_sum(const void* x, int32_t dtype, int64_t rows, int64_t cols, int64_t ld, void* out,
                void* ws, void* stream);
int64_t ahl_col_sum_ws_bytes(int64_t cols);

/* ---- weights ------------------------------------------------------------------------------ */

/* Everything the forward needs from the weights:
 *   wmax[t, n]  = max_{k in tile t} |w[n, k]|                       (dtype [T, N])
 *   tile_max[t] = max_n wmax[t, n], tile_min[t] = min_n wmax[t, n]  (float [T])
 *   w_eff       = noise(quantize(w))  (dtype [N, K], ld_eff)   -- only if w_eff != NULL
 * With quant_type/noise_type NONE, w_eff receives a plain copy of w.
 * Never writes to w (the Triton path's in-place store, triton_utils/triton_linear.py:152-156,
 * is deliberately not reproduced).
 * Replaces torch_utils/torch_linear.py:217-251 (amax, clip_and_quantize without learnable
 * clipping, modify_weight) and torch_utils/quant_utils.py:204-233.                       */
int ahl_weight_prep(const void* w, int64_t N, int64_t K, int64_t ld, const int32_t* tile_ends_host,
                    int32_t n_tiles, const AhlModifierCfg* cfg, void* wmax, float* tile_max,
                    float* tile_min, void* w_eff, int64_t ld_eff, void* stream);

/* Post-training quantisation in place, per tile, scale from the slice's own abs-max:
 * Replaces AnalogLinear.quantize_weights, nn/modules/linear.py:285-303.
 * ws_wmax: dtype [T, N]; ws_tile: float [2*T].                                            */
int ahl_quantize_weights(void* w, int64_t N, int64_t K, int64_t ld, const int32_t* tile_ends_host,
                         int32_t n_tiles, const AhlModifierCfg* cfg, void* ws_wmax, float* ws_tile,
                         void* stream);

/* ---- the analog matrix product ------------------------------------------------------------ */

/* Input-range clamp + DAC quantisation as one memory-bound pass over x[M, K]:
 *   AHL_IR_STATIC : xq = DAC(clamp(x, -ir_in[t], ir_in[t]))            ir_in dtype [T]
 *   AHL_IR_DYNAMIC: ir_out[t, m] = max_k |x[m, tile t]| (dtype [T, M]), xq = DAC(x) with it
 *   AHL_IR_NONE   : xq = x
 * Replaces torch_utils/torch_linear.py:155-192 (apply_input_range forward, dynamic abs-max,
 * UniformQuantize of the input). ahl_linear_fwd accepts the result as `xq`.
 * With cfg->tile_stride > 0 xq is written in the padded tile layout (ldxq >= n_tiles *
 * tile_stride), padding zeroed.                                                            */
int ahl_dac(const void* x, int64_t ldx, void* xq, int64_t ldxq, const void* ir_in, void* ir_out,
            int64_t M, int64_t K, const int32_t* tile_ends_host, int32_t n_tiles,
            const AhlLinearCfg* cfg, void* stream);

/* Forward of TorchLinear.linear (torch_utils/torch_linear.py:116-314) for x[M, K]:
 *   for every K-tile: clamp to the input range + DAC quantise, MFMA product with w_eff[N, K],
 *   output noise, ADC quantise, clamp to the output bound; per-tile results summed in dtype;
 *   bias added last.
 *   x        dtype [M, K] raw input; the clamp + DAC then run fused in the A-tile staging.
 *   xq       dtype [M, K] from ahl_dac, or NULL. 16-bit calls whose tiles are equal multiples of
 *            64 take a faster kernel when xq is given (x may then be NULL); with
 *            cfg->tile_stride > 0, xq and w_eff are in the padded tile layout and every split
 *            takes that kernel (16-bit dtypes only; AHL_ERR_UNSUPPORTED otherwise).
 *   ir       dtype [T] (AHL_IR_STATIC) or [T, M] (AHL_IR_DYNAMIC) or NULL (AHL_IR_NONE)
 *   wmax     dtype [T, N] from ahl_weight_prep, or NULL when neither noise nor bound is on
 *   tile_max float [T]    from ahl_weight_prep, or NULL likewise
 *   bias     dtype [N] or NULL
 *   y        dtype [M, N]
 *   clamp_mask  uint32 [T, ceil(N/32), Mr] or NULL, Mr = M rounded up to a multiple of 64 (rows
 *            beyond M are never written): bit (n % 32) of word [t][n / 32][m] is set
 *            where the tile-t output of element (m, n) left [-bound, bound] and was clamped
 *            (it passes no gradient). Written only when out_bound > 0 and clamp_mask != NULL;
 *            consumed by the two backward entry points.
 *   clamp_flag  uint32 [1] or NULL: receives non-zero if any tile output was clamped (or if the
 *            kernel does not track it); the backward entry points skip the mask when it is zero.
 *   ws       NULL, or ahl_linear_fwd_ws_bytes(...) bytes, 16-byte aligned. With it, calls of few
 *            rows (a recurrent or decoding step) give every K-tile of an output block to a block
 *            of its own and add the per-tile results in tile order afterwards: the same
 *            arithmetic and the same result bit for bit, on more of the chip. The size function
 *            returns 0 where that does not apply.
 * Slot of TritonLinear.forward, triton_utils/triton_linear.py:446-690.                   */
int64_t ahl_linear_fwd_ws_bytes(int64_t M, int64_t K, int64_t N, int32_t n_tiles, int32_t dtype);
int ahl_linear_fwd(const void* x, int64_t ldx, const void* xq, int64_t ldxq, const void* w_eff,
                   int64_t ldw, const void* bias, void* y, int64_t ldy, uint32_t* clamp_mask,
                   uint32_t* clamp_flag, const void* ir, const void* wmax, const float* tile_max,
                   int64_t M, int64_t K, int64_t N, const int32_t* tile_ends_host, int32_t n_tiles,
                   const AhlLinearCfg* cfg, void* ws, void* stream);

/* Input gradient and input-range gradient (torch_utils/torch_linear.py:29-108 backward):
 *   d[:, tile t] = (g * !clamped_t) @ w_eff[:, tile t]      w_eff [N, K] as used by the forward
 *   AHL_IR_STATIC: ir_grad[t] per reference InputRangeForward.backward (incl. decay switch),
 *                  dx zeroed where |x| > ir[t]; x[M, K] is the forward input.
 *   otherwise dx = d, ir_grad untouched.
 *   clamp_flag: NULL, or the flag written by ahl_linear_fwd (the mask is ignored when it reads 0).
 *   ws needs ahl_linear_bwd_dx_ws_bytes(M, K, N, n_tiles, dtype, cfg->tile_stride) bytes.
 *   With cfg->tile_stride > 0, w_eff is in the padded tile layout (x and dx stay dense: the
 *   kernel maps its columns back in the epilogue); needs a 16-bit dtype and N a multiple of 8.
 * Slot of TritonLinear.backward, triton_utils/triton_linear.py:695-764.                  */
int ahl_linear_bwd_dx(const void* g, int64_t ldg, const uint32_t* clamp_mask, const uint32_t* clamp_flag,
                      const void* w_eff, int64_t ldw, const void* x, int64_t ldx, const void* ir,
                      void* dx, int64_t lddx, void* ir_grad, int64_t M, int64_t K, int64_t N,
                      const int32_t* tile_ends_host, int32_t n_tiles, const AhlLinearCfg* cfg,
                      void* ws, void* stream);
int64_t ahl_linear_bwd_dx_ws_bytes(int64_t M, int64_t K, int64_t N, int32_t n_tiles, int32_t dtype,
                                   int64_t tile_stride);

/* ahl_linear_bwd_dx without a workspace argument, for callers that cannot allocate device memory
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc). It has no
 * counterpart in the reference. Same arguments, kernels and results as ahl_linear_bwd_dx; the
 * workspace is a static device array of AHL_STATIC_DX_SCRATCH_BYTES that every GPU the library
 * runs on holds until the process ends. Shapes whose ahl_linear_bwd_dx_ws_bytes(...) exceeds that
 * size return AHL_ERR_WORKSPACE (nothing is launched). The call itself allocates and frees
 * nothing. All calls on one GPU share that GPU's array: calls that overlap on one GPU (different
 * streams or threads) race; calls on one stream, or ordered by events, are safe. Nothing in the
 * array has to be cleared between calls (every slot is written before it is read).
 * The first call on each device looks up the array's device address (hipGetSymbolAddress, which
 * may load the library's code object on that device): make one call per device OUTSIDE any
 * stream capture before the calls that are recorded into a graph.                             */
#define AHL_STATIC_DX_SCRATCH_BYTES (16 * 1024 * 1024)
int ahl_linear_bwd_dx_static(const void* g, int64_t ldg, const uint32_t* clamp_mask,
                             const uint32_t* clamp_flag, const void* w_eff, int64_t ldw,
                             const void* x, int64_t ldx, const void* ir, void* dx, int64_t lddx,
                             void* ir_grad, int64_t M, int64_t K, int64_t N,
                             const int32_t* tile_ends_host, int32_t n_tiles,
                             const AhlLinearCfg* cfg, void* stream);

/* Backward of the learnable weight clip (UniformQuantize.backward with learn_res,
 * torch_utils/quant_utils.py:123-153, as called from clip_and_quantize :184-233).
 *   dw    dtype [N, K], in/out: on entry the gradient w.r.t. the clipped (and quantised) weights,
 *         on exit the gradient w.r.t. the weights (zero where a weight was clipped)
 *   w     dtype [N, K]  the weights of the forward;  clip dtype [T, N]  learnable_weight_clip
 *   tile_min float [T]  as returned by ahl_weight_prep for that clip
 *   dclip dtype [T, N]  gradient of the clip (LSQ rule, scaled by 1/sqrt(numel) without and
 *         2 sqrt(max_state / numel) with a quantiser, numel = N * tile width)
 *   cfg->quant_type: AHL_QUANT_CLIP_LEARNED or AHL_QUANT_DISCRETIZE_PER_CHANNEL.            */
int ahl_learned_clip_bwd(void* dw, int64_t lddw, const void* w, int64_t ldw, const void* clip,
                         const float* tile_min, void* dclip, int64_t N, int64_t K,
                         const int32_t* tile_ends_host, int32_t n_tiles, const AhlModifierCfg* cfg,
                         void* stream);

/* Weight gradient: dw[:, tile t] = (g * !clamped_t)^T @ DAC(clamp(x[:, tile t])).
 *   xq: the quantised input saved from the forward (ahl_dac), or NULL to re-quantise x here.
 *   dbias: dtype [N] or NULL; receives the bias gradient sum_m g[m, :] (the autograd of the
 *   bias addition in AnalogLinear.forward, nn/modules/linear.py:120-135), which the kernel
 *   gets for free while it streams g.
 *   With cfg->tile_stride > 0, xq is in the padded tile layout (dw stays dense).
 *   ws needs ahl_linear_bwd_dw_ws_bytes(M, K, N, n_tiles, dtype, clamp_mask != NULL,
 *   cfg->tile_stride) bytes
 *   (transposed staging copies of g and the quantised input).
 * Same reference slot as ahl_linear_bwd_dx.                                               */
int ahl_linear_bwd_dw(const void* g, int64_t ldg, const uint32_t* clamp_mask, const uint32_t* clamp_flag,
                      const void* x, int64_t ldx, const void* xq, int64_t ldxq, const void* ir,
                      void* dw, int64_t lddw, void* dbias, int64_t M, int64_t K, int64_t N,
                      const int32_t* tile_ends_host, int32_t n_tiles, const AhlLinearCfg* cfg,
                      void* ws, void* stream);
int64_t ahl_linear_bwd_dw_ws_bytes(int64_t M, int64_t K, int64_t N, int32_t n_tiles, int32_t dtype,
                                   int32_t has_mask, int64_t tile_stride);

/* ---- convolution as the same matrix product (nn/modules/conv.py:121-367) -------------------
 * A convolution layer of the reference unfolds its input into patches, runs the AnalogLinear
 * operator on them with weight.view(out_channels, -1), and transposes the result back. The three
 * entry points below are the data movement of that wrapper; the operator itself is
 * ahl_linear_fwd / ahl_linear_bwd_*. 1-d and 2-d layers use leading sizes of one.              */
typedef struct AhlConvGeom {
  int32_t batch, channels;
  int32_t in_size[3];  /* D, H, W of the input                                                  */
  int32_t kernel[3], stride[3], padding[3], dilation[3];
} AhlConvGeom;

/* Host only: out_size[d] = (in + 2 pad - dil (ker - 1) - 1) / stride + 1, the output extent
 * computed in _AnalogConvNd.forward (nn/modules/conv.py:357-362, :826-846). AHL_ERR_ARG if the
 * kernel does not fit.                                                                         */
int ahl_conv_out_size(const AhlConvGeom* geom, int32_t* out_size);

/* cols[(b * L + l), c * kvol + (kd * kH + kh) * kW + kw] = x[b, c, od*sD - pD + kd*dD, ...] or 0
 * outside the input; x dtype [B, C, D, H, W] contiguous, cols dtype [B * L, K] with row stride
 * ldc, L = product of the output extents, K = C * kD * kH * kW. Replaces
 * unfold(inp, ...).transpose(-1, -2).contiguous() (nn/modules/conv.py:310-322) and
 * unfold3d(...).transpose(-1, -2).contiguous() (:40-103, :777-792).                            */
int ahl_im2col(const void* x, const AhlConvGeom* geom, int32_t dtype, void* cols, int64_t ldc,
               void* stream);

/* Adjoint of ahl_im2col (the autograd of the unfold above): dx[b, c, d, h, w] = sum of the
 * dcols entries that ahl_im2col copied from that element, accumulated in fp32 in ascending
 * kernel-offset order and rounded once.                                                        */
int ahl_col2im(const void* dcols, int64_t ldc, const AhlConvGeom* geom, int32_t dtype, void* dx,
               void* stream);

/* dst[b][c][r] = src[b][r][c] for `batch` row-major matrices of rows x cols (row strides ld_src
 * and ld_dst, matrices back to back). Replaces out.transpose(-1, -2).contiguous()
 * (nn/modules/conv.py:356) and its autograd.                                                   */
int ahl_transpose_batched(const void* src, int64_t ld_src, int32_t dtype, int64_t batch,
                          int64_t rows, int64_t cols, void* dst, int64_t ld_dst, void* stream);

/* ---- convolution read off the image, without the patch matrix --------------------------------
 * For 16-bit dtypes, stride 1, dilation 1, a static (or no) input range, out_channels a multiple
 * of 64 and K-tiles that hold whole channels in multiples of 64 (ahl_conv_direct_supported), the
 * three products of _AnalogConvNd.forward / its autograd (nn/modules/conv.py:310-360) read a
 * zero-padded, channels-last copy of the image instead of the [B * L, C * kvol] patch matrix that
 * unfold writes: outputs are numbered on the PADDED pixel grid (P = B * prod(in + 2 pad) rows; a
 * row whose receptive field would leave the padded image is computed and dropped), and a kernel
 * offset is one constant row offset. A K-tile's contraction runs over (tap, channel) instead of
 * (channel, tap): the same terms in another order. Results equal the patch path's up to the order
 * of the fp32 additions inside a tile.
 * Pixel-row buffers ("rows" below) are dtype [rows, width] matrices, rows from
 * ahl_conv_direct_rows: `lead` rows of zeros, the P pixels, zeros to the end.
 * ahl_conv_image_rows and ahl_conv_grad_rows write EVERY row of their buffers (the zeros of the
 * lead, of the padding pixels and of the tail included): the caller need not clear them.      */
int ahl_conv_direct_rows(const AhlConvGeom* geom, int64_t* pixels, int64_t* lead, int64_t* rows);
int ahl_conv_direct_supported(const AhlConvGeom* geom, int32_t dtype, int64_t N, const int32_t* tile_ends_host,
                              int32_t n_tiles);

/* xq_rows[lead + p, c] = DAC(x[b, c, d, h, w]) at the padded pixel p of (b, d, h, w): clamp to the
 * range of channel c's K-tile and quantise (cfg->ir_mode AHL_IR_STATIC; AHL_IR_NONE copies).
 * flag_rows / counts (both or neither; static range, when a backward pass will follow): what
 * the input gradient needs to know about x -- flag_rows uint8 [rows, C] in the layout of xq_rows,
 * bit 0: x >= range, bit 1: x <= -range (entries whose gradient goes to the range), bit 2:
 * |x| > range (zeroed by the straight-through rule); counts uint32 [ahl_conv_count_words(geom)]:
 * per block of the kernel, the number of patch entries with bit 0 or 1 (the decay switch).
 * Replaces unfold + the per-tile clamp/DAC of torch_utils/torch_linear.py:134-192 and the
 * bookkeeping of :44-54, :92-106.                                                           */
int64_t ahl_conv_count_words(const AhlConvGeom* geom);
int ahl_conv_image_rows(const void* x, const AhlConvGeom* geom, int32_t dtype, const void* ir,
                        const int32_t* tile_ends_host, int32_t n_tiles, const AhlLinearCfg* cfg, void* xq_rows,
                        uint8_t* flag_rows, uint32_t* counts, void* stream);

/* Weight layouts for the three products, from / to the layer's [N, C * kvol] matrix
 * (weight.view(out_channels, -1)): mode 0 reorders every tile's columns to (tap, channel) -- the
 * forward's operand; mode 1 is its inverse from a matrix whose tiles start every `stride` columns
 * (what ahl_conv_bwd_dw leaves) ; mode 2 writes [C, kvol * N] for the input gradient. The
 * layer's matrix is nn/modules/conv.py:324 (modified_weights.view(out_channels, -1)), whose column
 * order (channel, tap) is that of unfold's patch entries (:325-352).                            */
int ahl_conv_weight_layout(const void* src, int64_t ld_src, int32_t dtype, int64_t N, const AhlConvGeom* geom,
                           const int32_t* tile_ends_host, int32_t n_tiles, int32_t mode, int64_t stride, void* dst,
                           int64_t ld_dst, void* stream);
/* Modes 0 and 2 of ahl_conv_weight_layout in one launch: a training step's forward leaves the
 * input gradient's operand beside its own (same source matrix, nn/modules/conv.py:324).         */
int ahl_conv_weight_layouts(const void* src, int64_t ld_src, int32_t dtype, int64_t N, const AhlConvGeom* geom,
                            const int32_t* tile_ends_host, int32_t n_tiles, void* w_taps, int64_t ld_taps, void* w_dx,
                            int64_t ld_dx, void* stream);

/* The analog forward on the padded pixel grid: y_rows [P, N] (no lead rows), clamp mask
 * [T, ceil(N/32), rows64(P)] and flag as ahl_linear_fwd writes them; w_taps from
 * ahl_conv_weight_layout mode 0; ir, wmax, tile_max, bias, cfg as for ahl_linear_fwd.
 * Slot of TorchLinear.linear as called from nn/modules/conv.py:325-352.                       */
int ahl_conv_fwd(const void* xq_rows, const void* w_taps, const void* bias, void* y_rows, uint32_t* clamp_mask,
                 uint32_t* clamp_flag, const void* ir, const void* wmax, const float* tile_max,
                 const AhlConvGeom* geom, int64_t N, const int32_t* tile_ends_host, int32_t n_tiles,
                 const AhlLinearCfg* cfg, void* stream);

/* y[b, n, *out] = y_rows[row of that output, n] (replaces out.transpose(-1, -2).contiguous() and
 * the view of nn/modules/conv.py:356-366), and its adjoint g_rows[lead + row, n] = g[b, n, *out].   */
int ahl_conv_output(const void* y_rows, const AhlConvGeom* geom, int32_t dtype, int64_t N, void* y, void* stream);
int ahl_conv_grad_rows(const void* g_out, const AhlConvGeom* geom, int32_t dtype, int64_t N, void* g_rows,
                       void* stream);

/* Weight gradient (and bias gradient if dbias != NULL) from the gradient rows and the quantised
 * image rows; dw_tiled is [N, padded_cols] with tile t at column t * (padded_cols / n_tiles), its
 * columns in (tap, channel) order (ahl_conv_weight_layout mode 1 turns it into the layer's order). */
int64_t ahl_conv_bwd_dw_ws_bytes(const AhlConvGeom* geom, int64_t N, const int32_t* tile_ends_host, int32_t n_tiles,
                                 int64_t* padded_cols);
int ahl_conv_bwd_dw(const void* g_rows, const uint32_t* clamp_mask, const uint32_t* clamp_flag, const void* xq_rows,
                    void* dw_tiled, void* dbias, const AhlConvGeom* geom, int64_t N, const int32_t* tile_ends_host,
                    int32_t n_tiles, const AhlLinearCfg* cfg, void* ws, void* stream);

/* Input gradient dx [B, C, *in] and, with a static range, ir_grad [T] (the autograd of unfold,
 * the product and the range clamp: torch_utils/torch_linear.py:29-108): w_dx from
 * ahl_conv_weight_layout mode 2; flag_rows and counts as ahl_conv_image_rows left them (only
 * with a static range); dimg_rows [P, C] is scratch the caller provides.                       */
int64_t ahl_conv_bwd_dx_ws_bytes(const AhlConvGeom* geom, int32_t n_tiles);
int ahl_conv_bwd_dx(const void* g_rows, const uint32_t* clamp_mask, const uint32_t* clamp_flag, const void* w_dx,
                    const uint8_t* flag_rows, const uint32_t* counts, const void* ir, void* dimg_rows, void* dx,
                    void* ir_grad, const AhlConvGeom* geom, int64_t N, const int32_t* tile_ends_host, int32_t n_tiles,
                    const AhlLinearCfg* cfg, void* ws, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* ANALOG_HIP_H_ */
