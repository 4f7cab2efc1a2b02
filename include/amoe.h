/* amoe.h -- C ABI of the MI355X-native CVMM path of Analog-MoE (libamoe.so).
 *
 * Every entry point is asynchronous on the HIP stream it is given, never synchronises the
 * host, never allocates or frees device memory and keeps no pointer after it returns: the
 * caller owns every buffer, including the workspace.  Return value: 0 on success, a negative
 * AMOE_E* code when the arguments are rejected on the host (nothing was launched), or a
 * positive hipError_t when a launch failed.  All device pointers must be 4-byte aligned;
 * 16-byte aligned rows make the kernels take their vector paths.
 *
 * The functions replace, one for one, the Triton launchers and the eager glue of the
 * reference's analog_moe/triton_src/cvmm.py (cited per function, file:line).  A nullable
 * pointer set to NULL switches the feature off; that replaces the reference's
 * `torch.tensor(-1)` sentinels (cvmm.py:585-598, 676-681).
 */
#ifndef AMOE_H
#define AMOE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define AMOE_VERSION 100
#define AMOE_MAX_TILES 16   /* K-tiles per projection (max_input_size splitting) */

enum { AMOE_F32 = 0, AMOE_BF16 = 1, AMOE_F16 = 2 };

enum {
  AMOE_OK = 0,
  AMOE_EINVAL = -1,       /* a size, stride or scalar is out of range */
  AMOE_ENULL = -2,        /* a required pointer is NULL */
  AMOE_ESHAPE = -3,       /* sizes are inconsistent with each other */
  AMOE_EALIGN = -4,       /* a pointer is not 4-byte aligned */
  AMOE_EWORKSPACE = -5,   /* workspace too small */
  AMOE_EUNSUPPORTED = -6  /* valid request this build does not implement */
};

int amoe_version(void);
const char* amoe_strerror(int rc);

/* ---------------------------------------------------------------------------------------
 * Selection: stable sort of expert ids, index and offset build.
 * Replaces cvmm_prepare_sel (cvmm.py:31-34: `ssel, perm = sel.flatten().sort()`) and the
 * second argsort of the backward (cvmm.py:850).  Tie order is fixed: ascending flat index.
 *   sel        [M] expert id of flat (token, head) position, int32 or int64 (sel_is_i64)
 *   sel_sorted [M] ascending ids;  perm [M] flat index of each sorted position (the
 *   up-projection's out_index);  in_index [M] = perm / k (its sel_index);
 *   offsets [E+1] first sorted position of each expert (new: the kernels use it to cut
 *   row tiles at expert boundaries).  Ids outside [0, E) make the call set *bad_flag != 0
 *   (device int32, may be NULL) and are sorted as expert E-1. */
size_t amoe_prepare_sel_workspace(int64_t M, int32_t E);
int amoe_prepare_sel(const void* sel, int32_t sel_is_i64, int64_t M, int32_t E, int32_t k,
                     int32_t* sel_sorted, int32_t* perm, int32_t* in_index, int32_t* offsets,
                     int32_t* bad_flag, void* workspace, size_t workspace_bytes, void* stream);

/* amoe_prepare_sel for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc): the same selection, bit for bit, without a workspace
 * argument.  No counterpart in the reference.  The unit histograms live in a device array inside the library
 * (AMOE_NOALLOC_SCRATCH_BYTES, one copy per GPU the library is used on, held until the process ends); the call
 * allocates and frees nothing.  A call whose amoe_prepare_sel_workspace(M, E) exceeds that size is rejected with
 * AMOE_EWORKSPACE (nothing launched).  All calls on one GPU share the array: calls that overlap on one GPU
 * (different streams, different threads) race; calls on one stream are ordered and safe. */
#define AMOE_NOALLOC_SCRATCH_BYTES (2u << 20)
size_t amoe_noalloc_scratch_bytes(void);
int amoe_prepare_sel_noalloc(const void* sel, int32_t sel_is_i64, int64_t M, int32_t E, int32_t k,
                             int32_t* sel_sorted, int32_t* perm, int32_t* in_index, int32_t* offsets,
                             int32_t* bad_flag, void* stream);

/* offsets[E+1] from an already sorted id vector, for callers that arrive with the
 * reference's own CVMMSel (cvmm.py:19-28), which carries no offsets. */
int amoe_offsets_from_sorted(const int32_t* sel_sorted, int64_t M, int32_t E, int32_t* offsets,
                             void* stream);

/* ---------------------------------------------------------------------------------------
 * Forward: out[out_index[i], :] = analog(x[in_index[i], :]) @ w[sel_sorted[i]]  for every
 * sorted position i.  Replaces the launcher cvmm_triton_quantized (cvmm.py:531-631) and
 * cvmm_kernel (cvmm.py:53-231).  Per K-tile t (one tile = the reference's behaviour):
 *   a = clamp(x, +-ir[i,t]) / ir[i,t] / abs_max[row]; a = rint(a / inp_res) * inp_res
 *   c = a @ w[e][tile rows, :]  (fp32 accumulate);  c += noise;  c = ADC(c)
 *   c *= abs_max[row];  c *= ir[i,t];  out += c
 * The K-tile split, the ADC and the in-kernel noise generator are this library's own
 * extensions (the reference asserts them off: moe_layer_aihwkit_lightning.py:152-160).
 */
typedef struct amoe_fwd_args {
  int32_t dtype;                 /* AMOE_F32 / AMOE_BF16 / AMOE_F16: type of x, w, out */
  int32_t M, N, K, E;            /* sorted rows, output features, input features, experts */
  int32_t n_in_rows, n_out_rows; /* rows of x / of out (indices are checked against nothing
                                    on the device; the caller guarantees the ranges).
                                    n_in_rows == 0 = unknown: 64-bit addressing of x, as
                                    n_x_rows == 0 in amoe_bwd_w_args */
  const void* x;   int64_t ldx;                       /* [n_in_rows, K], row stride ldx */
  const void* w;   int64_t w_stride_e, w_stride_k, w_stride_n; /* [E, K, N] view; one of
                                    w_stride_n / w_stride_k must be 1 (cvmm.py:839 passes a
                                    transposed view) */
  void* out;       int64_t ldo;                       /* [n_out_rows, N] */
  const int32_t* sel_sorted;     /* [M] */
  const int32_t* offsets;        /* [E+1] */
  const int32_t* in_index;       /* [M] */
  const int32_t* out_index;      /* [M] or NULL -> in_index (cvmm.py:196-205) */
  const float* ir;               /* [M, n_tiles] input range per sorted position, or NULL */
  int32_t ir_by_expert;          /* != 0: ir is the [E, n_tiles] table itself (what the caller
                                    would otherwise gather with input_range[sel],
                                    moe_layer_aihwkit_lightning.py:447-448) */
  const float* abs_max;          /* [n_in_rows] or NULL (cvmm.py:124-128, 156-158) */
  float inp_res;                 /* quantisation step; <= 0: no quantisation */
  int32_t n_tiles;               /* >= 1 */
  int32_t tile_bounds[AMOE_MAX_TILES + 1]; /* tile t covers input features [b[t], b[t+1]) */
  const float* noise;            /* [n_tiles, n_out_rows, N] fp32, already scaled, or NULL */
  int64_t noise_tile_stride, ldnoise;
  float noise_std;               /* used when noise == NULL and > 0: generate in the kernel
                                    noise_std * wmax[e, n] * N(0,1) */
  uint64_t noise_seed;
  const uint64_t* noise_seed_dev;/* optional device word added to noise_seed when the kernel starts:
                                    a captured graph draws new noise on each replay if the caller
                                    bumps the word between replays */
  const float* wmax;             /* [E, wmax_cols] max |w| per expert (cols 1) or channel (N) */
  int32_t wmax_cols;
  float out_bound, out_res;      /* ADC: clamp to +-out_bound*wmax, max(res,1/res) states;
                                    out_bound <= 0: off; out_res <= 0: clamp only */
  int32_t relu;                  /* fuse max(., 0) into the store */
  int32_t* range_flag;           /* device int32 or NULL: set to 1 if |a| > 1 is met before
                                    quantising (cvmm.py:162 asserts this) */
  /* Chaining two projections (no counterpart in the reference, which re-runs the input stage of
     the second projection for every block of its output columns): */
  void* xq_out;                  /* optional second output [n_out_rows, N], dtype: the input stage
                                    (clamp to +-xq_ir[e], / xq_ir[e], round to xq_inp_res) of the
                                    projection that consumes `out`, applied to `out` as stored.
                                    bf16 holds the integer codes, fp32 codes * xq_inp_res */
  int64_t ldxq;
  const float* xq_ir;            /* [E] input range of that projection (it must have one K-tile) */
  float xq_inp_res;              /* its quantisation step, > 0 */
  int32_t x_is_quantized;        /* != 0: x is such an image made with this call's ir / inp_res:
                                    the input stage is skipped, the rescale is not */
  /* The result as ADC codes (no counterpart in the reference): with an output quantiser, one K-tile and one
     max |W| per expert, every result is (code * step[e]) * ir[e] with an integer code in [-half, half],
     half = max(out_res, 1 / out_res) / 2 <= 127.  A caller that only streams the result once more (the gate
     reduction, the gate gradient) can take it at a quarter of fp32 / half of bf16: */
  uint8_t* code_out;             /* optional [n_out_rows, N]: code + 128; `out` is then not written and may be NULL */
  int64_t ldcode;
  float* code_scale_out;         /* with code_out: [E, 2] = (step[e], ir[e]); written for experts that have rows */
} amoe_fwd_args;

int amoe_cvmm_fwd(const amoe_fwd_args* args, void* stream);

/* Whether amoe_cvmm_fwd has a kernel that leaves the result as ADC codes (args->code_out) for a call of these
 * shapes, strides and settings: 1 or 0.  The one place where that is decided: amoe_cvmm_fwd asks this function
 * itself, and callers that must know the result's type before the call (operator shape functions under a tracer;
 * the reference's counterpart is the abstract implementation at cvmm.py:634-642) ask it instead of restating its
 * rules.  Only sizes, strides and scalars are read; pointer fields count as flags (NULL = feature off) and are
 * never dereferenced, so placeholders will do.  What remains for the call itself is the 16-byte alignment of x, w
 * and code_out. */
int amoe_fwd_codes_supported(const amoe_fwd_args* args);

/* ---------------------------------------------------------------------------------------
 * Weight gradient: grad_w[e] = sum_{i in expert e} clamp(x[in_index[i]], +-ir[i,t])^T
 *                                                   g[g_index[i]]          -> [E, K, N]
 * Replaces cvmm_triton_backward + cvmm_backward_kernel3 (cvmm.py:645-696, 254-397).
 * One workgroup owns one output tile of one expert: no atomics, no pre-zeroing, fixed
 * summation order.  Experts without rows get zeros (cvmm.py:671). */
typedef struct amoe_bwd_w_args {
  int32_t dtype;
  int32_t M, N, K, E;
  const void* x;  int64_t ldx;           /* forward input  [*, K] */
  const void* g;  int64_t ldg;           /* output gradient [*, N] */
  void* grad_w;                          /* [E, K, N] contiguous, dtype */
  const int32_t* offsets;                /* [E+1] */
  const int32_t* in_index;               /* [M] row of x per sorted position */
  const int32_t* g_index;                /* [M] row of g per sorted position, NULL -> in_index
                                            (cvmm.py:346-351) */
  const float* ir;                       /* [M, n_tiles] or NULL */
  int32_t ir_by_expert;                  /* != 0: ir is [E, n_tiles] */
  const void* g_scale;                   /* dtype, [M], one value per sorted position, or NULL: the
                                            clipped x row is multiplied by it and rounded to dtype, which
                                            gives the gate (x) dy outer product of cvmm.py:785-789
                                            without materialising it */
  int64_t n_x_rows, n_g_rows;            /* rows of x and of g (bounds the 32-bit addressing of the
                                            interior path; 0 = unknown: 64-bit addressing) */
  int32_t n_tiles;
  int32_t tile_bounds[AMOE_MAX_TILES + 1];
  void* workspace;                       /* optional, amoe_bwd_w_workspace(args) bytes: lets several
                                            workgroups share the rows of one expert (few or heavily
                                            loaded experts); the sum order stays fixed.  NULL: one
                                            workgroup per expert and 128x128 tile */
  size_t workspace_bytes;
  int32_t rows_per_chunk;                /* 0: the library sizes the row chunks; > 0: rows per chunk
                                            (rounded up to a multiple of 64) */
} amoe_bwd_w_args;

/* Bytes of workspace for this call (reads the sizes and tile bounds only). */
size_t amoe_bwd_w_workspace(const amoe_bwd_w_args* args);
int amoe_cvmm_bwd_w(const amoe_bwd_w_args* args, void* stream);

/* ---------------------------------------------------------------------------------------
 * Input gradient with the clip mask, the input-range gradient and the gate scaling fused
 * into the store.  Replaces the second cvmm_triton_quantized call of CVMM.backward and the
 * eager glue after it (cvmm.py:828-881, 884-888):
 *   G = g[g_index[i], :] @ w[e]^T                          (cvmm.py:835-846)
 *   ir_grad[i,t] = sum_n min([x>=ir] G gate, 0) - sum_n max([x<=-ir] G gate, 0)   (:863-865)
 *   ir_grad *= ir * gradient_scale (if gradient_relative)                         (:868-870)
 *   ir_grad += decay * ir * [mean(|x|<ir) > input_min_percentage]                 (:872-878)
 *   grad_x_full[out_index[i], :] = G * [|x|<ir] * gate [* (x>0) if relu_mask]     (:881, 888)
 * x is the forward input of the same call, read at row xf_index[i].
 * workspace: amoe_bwd_x_workspace(M, K, n_tiles) bytes. */
typedef struct amoe_bwd_x_args {
  int32_t dtype;
  int32_t M, N, K, E;            /* as in the forward call: w is [E, K, N]; output has K columns */
  const void* g;   int64_t ldg;  /* [n_g_rows, N] */
  int32_t n_g_rows;
  const void* w;   int64_t w_stride_e, w_stride_k; /* [E, K, N], N contiguous */
  void* grad_x_full; int64_t ldo;   /* [n_out_rows, K] */
  const void* x;   int64_t ldx;  /* forward input [*, K]; may be NULL when ir == NULL and
                                    relu_mask == 0 */
  const int32_t* offsets;        /* [E+1] */
  const int32_t* g_index;        /* [M] row of g */
  const int32_t* out_index;      /* [M] row of grad_x_full */
  const int32_t* xf_index;       /* [M] row of x */
  const void* gate;              /* [n_out_rows] dtype, indexed by output row, or NULL */
  const float* ir;               /* [M, n_tiles] or NULL */
  int32_t ir_by_expert;          /* != 0: ir is [E, n_tiles]; ir_grad stays per sorted position */
  float* ir_grad;                /* [M, n_tiles] out (required when ir != NULL) */
  int32_t n_tiles;
  int32_t tile_bounds[AMOE_MAX_TILES + 1];
  int32_t gradient_relative;  float gradient_scale;
  float decay;  float input_min_percentage;
  int32_t relu_mask;
  void* workspace;  size_t workspace_bytes;
  void* xc_out;                          /* optional [rows of x, K], dtype: gate * clamp(x, +-ir) at row
                                            xf_index[i] -- the x operand of the weight gradient of
                                            the same projection (amoe_cvmm_bwd_w then runs without
                                            ir and g_scale).  No counterpart in the reference, which
                                            clips inside its weight-gradient kernel for every block
                                            of output columns.  Needs x */
  int64_t ldxc;
} amoe_bwd_x_args;

size_t amoe_bwd_x_workspace(int64_t M, int32_t K, int32_t n_tiles);
int amoe_cvmm_bwd_x(const amoe_bwd_x_args* args, void* stream);

/* ---------------------------------------------------------------------------------------
 * Small row-wise companions of CVMM.forward / CVMM.backward.
 */
/* y[t, :] = sum_j gate[t, j] * z[t*k + j, :]   (cvmm.py:757-759).
 * counter (may be NULL): an int64 word in device memory to which the launch adds counter_add.  The layer passes the
 * step counter of the generated noise (amoe_fwd_args.noise_seed_dev): this is the launch that follows the last
 * kernel drawing from it, so the next forward, or the next replay of a captured graph, draws anew without a launch
 * of its own for the addition (the reference draws fresh torch.randn tensors per call, cvmm.py:712-716). */
int amoe_gate_reduce(int32_t dtype, const void* z, const void* gate, void* y,
                     int64_t T, int32_t k, int32_t D, int64_t* counter, int64_t counter_add, void* stream);
/* out[t, :] = sum_j full[t*k + j, :]           (cvmm.py:890-891) */
int amoe_ksum(int32_t dtype, const void* full, void* out, int64_t T, int32_t k, int32_t D,
              void* stream);
/* amoe_ksum with the input-range clip of the up-projection applied on the way (cvmm.py:848-881 and 890-891,
 * regrouped).  The clip mask of row r = t*k + j is |x[t, :]| < ir[sel[r], tile]: it depends on the token's input
 * row, shared by its k heads, so the GEMM that makes `full` (amoe_cvmm_bwd_x without x and ir) keeps no mask tile
 * and the input row is read once per token:
 *   grad_x[t, :]  = sum_j [|x[t]| < ir] full[t*k + j, :]                                   (:853, 881, 890-891)
 *   ir_grad[i, t] = sum_n min([x >= ir] full, 0) - sum_n max([x <= -ir] full, 0), row perm[i]  (:863-865)
 *   then the scaling and decay rules of amoe_cvmm_bwd_x                                      (:868-878)
 * full [T*k, D] and grad_x [T, D] are dense; x is [T, D] with row stride ldx; sel [T*k] holds the expert of
 * every row (the unsorted ids, int32 or int64); perm [T*k] and offsets [E+1] are amoe_prepare_sel's; ir is
 * [E, n_tiles].  ir_grad [T*k, n_tiles] is indexed by sorted position like amoe_cvmm_bwd_x's.
 * k <= 8, tile bounds multiples of 16 bytes of elements; otherwise AMOE_EUNSUPPORTED (use amoe_cvmm_bwd_x with
 * x and ir, then amoe_ksum).  workspace: amoe_ksum_clip_workspace(T, k, n_tiles) bytes. */
typedef struct amoe_ksum_clip_args {
  int32_t dtype;
  int64_t T;  int32_t k, D, E;
  const void* full;
  const void* x;  int64_t ldx;
  const void* sel;  int32_t sel_is_i64;
  const int32_t* perm;  const int32_t* offsets;
  const float* ir;
  int32_t n_tiles;
  int32_t tile_bounds[AMOE_MAX_TILES + 1];
  void* grad_x;
  float* ir_grad;
  int32_t gradient_relative;  float gradient_scale;
  float decay;  float input_min_percentage;
  void* workspace;  size_t workspace_bytes;
} amoe_ksum_clip_args;

size_t amoe_ksum_clip_workspace(int64_t T, int32_t k, int32_t n_tiles);
int amoe_ksum_clip(const amoe_ksum_clip_args* args, void* stream);
/* grad_gate[t*k + j] = <z[t*k + j, :], dy[t, :]>   (cvmm.py:889) */
int amoe_gate_grad(int32_t dtype, const void* z, const void* dy, void* grad_gate,
                   int64_t T, int32_t k, int32_t D, void* stream);
/* amoe_gate_reduce / amoe_gate_grad on a result stored as ADC codes (amoe_fwd_args.code_out): row r = t*k + j
 * belongs to expert sel[r] (the unsorted ids, int32 or int64), z[r, :] = ((code[r, :] - 128) * scale[e][0]) * scale[e][1]. */
int amoe_gate_reduce_codes(int32_t dtype, const uint8_t* codes, const float* scale, const void* sel,
                           int32_t sel_is_i64, const void* gate, void* y, int64_t T, int32_t k, int32_t D,
                           int64_t* counter, int64_t counter_add, void* stream);
int amoe_gate_grad_codes(int32_t dtype, const uint8_t* codes, const float* scale, const void* sel,
                         int32_t sel_is_i64, const void* dy, void* grad_gate, int64_t T, int32_t k, int32_t D,
                         void* stream);
/* abs_max[r] = max_n |x[r, n]|                 (cvmm.py:733, 737) */
int amoe_row_abs_max(int32_t dtype, const void* x, int64_t ldx, int64_t rows, int32_t K,
                     float* abs_max, void* stream);
/* wmax[e, c] = max |w[e, :, c]| (cols == N) or max |w[e]| (cols == 1)
 * (moe_layer_aihwkit_lightning.py:480-487) */
int amoe_weight_abs_max(int32_t dtype, const void* w, int32_t E, int32_t K, int32_t N,
                        int32_t cols, float* wmax, void* stream);
/* Both per-expert tables of a layer, wmax_a[e] = max |w_a[e]| and wmax_b[e] = max |w_b[e]| (the cols == 1 case of
 * amoe_weight_abs_max for keys [E, K_a, N_a] and values [E, K_b, N_b]), from one zero fill and one reduction
 * launch instead of two of each (moe_layer_aihwkit_lightning.py:480-487, once per projection there). */
/* The per-expert tables one layer's forward needs, from one small launch and one reduction launch: the two max |W|
 * tables of amoe_weight_abs_max_pair and -- with input_range != NULL -- the fp32 input-range tables of the two
 * projections, cut out of the layer's parameter input_range [2, E, ir_cols] (element type ir_dtype):
 * ir_up [E, n_up] = input_range[0, :, :n_up], ir_dn [E, n_dn] = input_range[1, :, :n_dn].  The reference reads that
 * parameter through input_range[ir_idx][sel_indices.sel] once per projection and call
 * (moe_layer_aihwkit_lightning.py:447-448); the kernels here take the table itself (ir_by_expert). */
int amoe_layer_tables(int32_t dtype, const void* w_a, int32_t K_a, int32_t N_a, float* wmax_a, const void* w_b,
                      int32_t K_b, int32_t N_b, float* wmax_b, int32_t E, int32_t ir_dtype, const void* input_range,
                      int32_t ir_cols, int32_t n_up, float* ir_up, int32_t n_dn, float* ir_dn, void* stream);
int amoe_weight_abs_max_pair(int32_t dtype, const void* w_a, int32_t K_a, int32_t N_a, float* wmax_a,
                             const void* w_b, int32_t K_b, int32_t N_b, float* wmax_b, int32_t E, void* stream);
/* out[e * ldout + t] = sum_{i in expert e} v[i, t]: index backward of input_range[sel]
 * (moe_layer_aihwkit_lightning.py:447-448), fixed order, fp32 sums rounded once to out_dtype (the parameter's type).
 * ldout >= n_tiles + zero_cols: the row stride of out, so that the sums can land in a slice of a wider table; the
 * zero_cols columns after the sums are set to zero (tile columns of the table that this projection does not have). */
int amoe_segment_sum(const float* v, const int32_t* offsets, int32_t E, int32_t n_tiles, int32_t out_dtype,
                     void* out, int64_t ldout, int32_t zero_cols, void* stream);

/* ---------------------------------------------------------------------------------------
 * Per-expert unbiased standard deviation of the routed rows' elements, for input-range
 * initialisation from data.  Replaces cvmm_std and its two kernels (cvmm.py:400-526).
 * Returns the exact estimate sqrt(SS/(n-1)); an expert without rows gives -0.0, as the
 * reference's sqrt(0/-1) does.  out is fp32 [E]. */
int amoe_expert_std(int32_t dtype, const void* x, int64_t ldx, int32_t K,
                    const int32_t* in_index, const int32_t* offsets, int32_t E,
                    float* out, void* stream);

/* ---------------------------------------------------------------------------------------
 * Weight modifier of a training forward: out [E, K, N] = modified copy of w
 * (AnalogSigmaMoELayerAIHWKITLightning.modify_weight, moe_layer_aihwkit_lightning.py:313-382;
 * the ADD_NORMAL case of moe_layer_aihwkit.py:144-196).
 *   n_states > 0:  res = wmax * (1 / n_states);  w = round(w / res) * res  (:346-363; torch's GPU
 *                  kernels divide a tensor by a host scalar through the fp32 reciprocal)
 *   std_dev  > 0:  w += std_dev * wmax * z,  z standard normal             (:364-379)
 * wmax is the assumed max |W|: [E] (wmax_cols == 1) or [E, N] (wmax_cols == N), fp32, as
 * amoe_weight_abs_max writes it (:333-344).  z comes from `noise` (fp32 [E, K, N]) when given,
 * else from the counter-based generator keyed by noise_seed (+ *noise_seed_dev) and the
 * element's position.  For bf16 every intermediate is rounded where the reference's tensor
 * expression rounds it; round_noise != 0 also rounds z to the weights' type first (randn_like
 * of the weights, :366) and 0 leaves it fp32 (moe_layer_aihwkit.py:188-194).
 * The gradient of the modified weights is passed to w unchanged by the caller. */
int amoe_modify_weight(int32_t dtype, const void* w, int32_t E, int32_t K, int32_t N,
                       const float* wmax, int32_t wmax_cols, float n_states, float std_dev,
                       const float* noise, int32_t round_noise, uint64_t noise_seed,
                       const uint64_t* noise_seed_dev, void* out, void* stream);

/* Unbiased standard deviation of the weights per expert (cols == 1: std_out [E]) or per
 * channel (cols == N: std_out [E, N]): the std((1, 2)) / std(1) of clip_weights
 * (moe_layer_aihwkit_lightning.py:529-534; moe_layer_aihwkit.py:327-331).  fp32 result.
 * workspace: amoe_weight_std_workspace bytes, 8-byte aligned (partial sums in fp64, added in a
 * fixed order). */
size_t amoe_weight_std_workspace(int32_t E, int32_t K, int32_t N, int32_t cols);
int amoe_weight_std(int32_t dtype, const void* w, int32_t E, int32_t K, int32_t N, int32_t cols,
                    float* std_out, void* workspace, size_t workspace_bytes, void* stream);

/* w = clamp(w, -bound, +bound) in place, bound [E] (cols == 1) or [E, N] (cols == N), fp32
 * (moe_layer_aihwkit_lightning.py:535-541; moe_layer_aihwkit.py:321-335). */
int amoe_clamp_weights(int32_t dtype, void* w, int32_t E, int32_t K, int32_t N,
                       const float* bound, int32_t cols, void* stream);

/* ---------------------------------------------------------------------------------------
 * Router epilogue: gate values and top-k experts of every token from the router's logits
 * [T, E], and the regulariser of the mean expert usage.  The reference's layer inherits this
 * step from sigma_moe.SigmaMoELayer (absent from the checkout); its per-token form is
 * tests/test_moe_layer_aihwkit_lightning.py:82-90: sel = sigmoid(expert_sel(x));
 * sel_val, sel_idx = sel.topk(k, dim=-1, sorted=False).
 *   sel_val [T, k] (dtype), sel_idx [T, k] int64: descending gate value, ties to the lower id
 *   reg (optional, fp32 scalar): sum_e pbar_e log pbar_e, pbar = mean_t softmax(logits[t])
 *   reg_c (with reg, fp32 [E]): 1 + log pbar_e, which amoe_select_bwd reads
 * E <= 512.  workspace: amoe_select_workspace bytes when reg is asked for. */
size_t amoe_select_workspace(int64_t T, int32_t E);
int amoe_select_fwd(int32_t dtype, const void* logits, int64_t T, int32_t E, int32_t k,
                    void* sel_val, int64_t* sel_idx, float* reg, float* reg_c,
                    void* workspace, size_t workspace_bytes, void* stream);
/* grad_logits [T, E] from grad_val [T, k] (optional) through the sigmoid of the chosen experts and
 * from *grad_reg (device fp32 scalar, optional, with reg_c) through the regulariser. */
int amoe_select_bwd(int32_t dtype, const void* logits, int64_t T, int32_t E, int32_t k,
                    const int64_t* sel_idx, const void* grad_val, const float* reg_c,
                    const float* grad_reg, void* grad_logits, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* AMOE_H */
