// C ABI of libamoe: argument checks on the host, then kernel launches on the caller's stream.
#include <amoe.h>

#include <atomic>

#include "gemm_rows.h"
#include "gemm_fwd256.h"
#include "gemm_bwdx256.h"
#include "gemm_ws256.h"
#include "gemm_wgrad256.h"
#include "gemm_wgrad.h"
#include "misc_kernels.h"
#include "weight_kernels.h"
#include "select_kernels.h"
#include "prepare_sel.h"

using namespace amoe;

namespace {

inline bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }
inline int launch_rc() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? AMOE_OK : (int)e;
}
inline int check_bounds(int n_tiles, const int32_t* b, int K) {
  if (n_tiles < 1 || n_tiles > AMOE_MAX_TILES) return AMOE_EINVAL;
  if (b[0] != 0 || b[n_tiles] != K) return AMOE_ESHAPE;
  for (int t = 0; t < n_tiles; t++)
    if (b[t + 1] <= b[t]) return AMOE_ESHAPE;
  return AMOE_OK;
}
inline bool bounds_multiple_of(int n_tiles, const int32_t* b, int m) {
  for (int t = 0; t <= n_tiles; t++)
    if (b[t] % m) return false;
  return true;
}
inline size_t esize(int dtype) { return dtype == AMOE_F32 ? 4 : 2; }
// Whether every DAC code of a quantiser with step inp_res (codes -1/inp_res .. 1/inp_res) is exact in the type.
inline bool dac_codes_fit(int dtype, float inp_res) {
  if (dtype == AMOE_F32 || !(inp_res > 0.f)) return true;
  return 1.0f / inp_res <= (dtype == AMOE_BF16 ? 256.f : 2048.f) * (1.0f + 1e-6f);
}
inline int max_row_tiles(int64_t M, int E) { return (int)(M / kTileRows) + E; }

// Compute units of the current device (read once; the value cannot change while the process lives).
inline int num_compute_units() {
  static const int n = [] {
    int dev = 0, cu = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 256;
    if (hipDeviceGetAttribute(&cu, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cu <= 0) return 256;
    return cu;
  }();
  return n;
}

// Persistent grid of the row-gather GEMM: two workgroups per compute unit, more if a workgroup
// would otherwise get more work items than its descriptor table holds, rounded up to a multiple
// of the column-block count (so that the column blocks of one row tile run side by side), never
// more than there are work items.
inline int persistent_grid(int row_tiles, int col_blocks, int per_cu = 2) {
  const long long work = (long long)row_tiles * col_blocks;
  long long g = (long long)per_cu * num_compute_units();
  const long long need = (work + kMaxDesc - 1) / kMaxDesc;
  if (need > g) g = need;
  if (g % col_blocks) g += col_blocks - g % col_blocks;
  if (g > work) g = work;
  return g < 1 ? 1 : (int)g;
}

// Every tile of the launch is interior: the FAST instantiation applies.
inline bool rows_all_interior(const RowsParams& p, int mode, int bk) {
  if (!p.a_vec || !p.w_vec || !p.out_stage || !p.buf_ok || p.abs_max != nullptr) return false;
  if (p.xq_out != nullptr && !p.xq_stage) return false;
  if (p.xc_out != nullptr && !p.xc_vec) return false;
  // forward: the edge-free code has the clip-and-quantise input stage or none at all
  if (mode != MODE_BWDX && (p.ir != nullptr) != (p.inp_res > 0.f)) return false;
  if (p.noise != nullptr && !p.noise_vec) return false;
  if (p.xf != nullptr && !p.xf_vec) return false;
  for (int t = 0; t < p.n_col_tiles; t++)
    if ((p.col_bounds[t + 1] - p.col_bounds[t]) % kTileCols) return false;
  for (int t = 0; t < p.n_kd_tiles; t++)
    if ((p.kd_bounds[t + 1] - p.kd_bounds[t]) % bk) return false;
  return true;
}

template <typename T, bool W_KC, bool FAST>
int launch_rows_mode(const RowsParams& p, int mode, int grid, hipStream_t st) {
  if (mode == MODE_FWD) {
    auto k = &gemm_rows_kernel<T, W_KC, MODE_FWD, FAST>;
    hipLaunchKernelGGL(k, dim3(grid), dim3(kThreads), 0, st, p);
  } else if (mode == MODE_FWD_SPLIT) {
    auto k = &gemm_rows_kernel<T, W_KC, MODE_FWD_SPLIT, FAST>;
    hipLaunchKernelGGL(k, dim3(grid), dim3(kThreads), 0, st, p);
  } else {
    auto k = &gemm_rows_kernel<T, W_KC, MODE_BWDX, FAST>;
    hipLaunchKernelGGL(k, dim3(grid), dim3(kThreads), 0, st, p);
  }
  return launch_rc();
}

template <typename T, bool W_KC>
int launch_rows(const RowsParams& p, int mode, int grid, hipStream_t st) {
  return rows_all_interior(p, mode, Elem<T>::kBK) ? launch_rows_mode<T, W_KC, true>(p, mode, grid, st)
                                            : launch_rows_mode<T, W_KC, false>(p, mode, grid, st);
}

// The 128 x 256 forward kernel for the usual training shapes (bf16 or fp16, every tile interior, per-expert input
// ranges, one max |W| per expert).  AMOE_EUNSUPPORTED: this launch is not one of them; the general kernel runs.
template <typename T, int A_MODE, bool ANALOG, bool NOISE, bool SPLIT2, bool ZCODES = false>
int launch_fwd256_as(const RowsParams& p, int grid, hipStream_t st) {
  auto k = &fwd256_kernel<T, A_MODE, ANALOG, NOISE, SPLIT2, ZCODES>;
  hipLaunchKernelGGL(k, dim3(grid), dim3(kThreads), 0, st, p);
  return launch_rc();
}

// The input gradient reads the forward input x (through xf_index) only for the features that need it: the
// input-range clip, the ReLU mask, the clipped-input output.  A caller that passes x without any of them has not
// been asked for xf_index, and its launch is a plain product.
inline bool bwdx_reads_x(const amoe_bwd_x_args* a) {
  return a->x != nullptr && a->xf_index != nullptr && (a->ir != nullptr || a->relu_mask != 0 || a->xc_out != nullptr);
}

// The 128 x 256 input-gradient kernel, for the same launches (and column tiles that are multiples of 256).  The
// partial sums of the input-range gradient then cover 256 columns each; *n_count_blocks is the grid that ran.
template <typename T, int COLS>
int launch_bwdx256_cols(RowsParams p, const amoe_bwd_x_args* a, hipStream_t st, int* n_count_blocks) {
  p.n_col_blocks = count_col_blocks(p.col_bounds, p.n_col_tiles, COLS);
  const int grid = persistent_grid(max_row_tiles(a->M, a->E), p.n_col_blocks, COLS == 128 ? 3 : 2);
  *n_count_blocks = grid;
  const bool relu = a->relu_mask != 0, xc = a->xc_out != nullptr;
  if (!bwdx_reads_x(a)) {
    hipLaunchKernelGGL((&bwdx256_kernel<T, false, false, false, COLS>), dim3(grid), dim3(kThreads), 0, st, p);
  } else if (!relu) {
    if (xc) hipLaunchKernelGGL((&bwdx256_kernel<T, true, false, true, COLS>), dim3(grid), dim3(kThreads), 0, st, p);
    else hipLaunchKernelGGL((&bwdx256_kernel<T, true, false, false, COLS>), dim3(grid), dim3(kThreads), 0, st, p);
  } else {
    if (xc) hipLaunchKernelGGL((&bwdx256_kernel<T, true, true, true, COLS>), dim3(grid), dim3(kThreads), 0, st, p);
    else hipLaunchKernelGGL((&bwdx256_kernel<T, true, true, false, COLS>), dim3(grid), dim3(kThreads), 0, st, p);
  }
  return launch_rc();
}

// The kernel that keeps the weights in registers (gemm_ws256.h): a contraction of exactly 256, output columns in
// groups of 256, interior launches.  Two workgroups per CU, in equal shares per column group, and more if a
// workgroup's run of 32-row blocks would not fit its descriptor table; returns the grid, or 0 when the launch is not
// one of these.
inline int ws256_plan(RowsParams& p, int64_t out_rows, int64_t out_row_bytes) {
  if (p.KD != kWsK || p.ND % 256 || !p.a_vec || !p.w_vec || !p.buf_ok || p.abs_max != nullptr) return 0;
  if (out_rows * out_row_bytes >= (int64_t)kWsOutLimit || (int64_t)p.M * 4 >= (1LL << 31)) return 0;
  p.n_col_blocks = p.ND / 256;
  const long long blocks = (long long)p.M / kWsRows + p.E;                 // bound on the 32-row blocks
  long long runs = 2LL * num_compute_units() / p.n_col_blocks;
  if (runs < 1) runs = 1;
  if (runs * kMaxDesc < blocks) runs = (blocks + kMaxDesc - 1) / kMaxDesc;
  if (runs > blocks) runs = blocks;
  return (int)(runs * p.n_col_blocks);
}

template <typename T>
int launch_bwdx256(RowsParams p, const amoe_bwd_x_args* a, hipStream_t st, int* n_count_blocks, int* block_cols) {
  if (!rows_all_interior(p, MODE_BWDX, kFBK)) return AMOE_EUNSUPPORTED;
  if (!bwdx_reads_x(a) && a->ir == nullptr && a->gate == nullptr && p.out_stage) {
    // a plain product with a contraction of 256: the weights stay in registers and the rows stream past them
    RowsParams q = p;
    if (const int grid = ws256_plan(q, a->M, a->ldo * 2)) {
      hipLaunchKernelGGL((&ws256_kernel<T, true, 64, WS_PLAIN, false>), dim3(grid), dim3(kThreads), 0, st, q);
      return launch_rc();
    }
  }
  if (a->ir != nullptr && !a->ir_by_expert) return AMOE_EUNSUPPORTED;
  if (a->x != nullptr && (!aligned(a->x, 16) || a->ldx % 8)) return AMOE_EUNSUPPORTED;   // 16-byte pieces of x rows
  // With a short contraction an item is mostly its mask stage: 128-column tiles at three workgroups per CU then
  // hide more of it (C3's up-projection, contraction 256: 0.197 vs 0.212 ms; at 512 the wide tile wins again).
  const bool narrow = bwdx_reads_x(a) && a->N <= 256;
  const int cols = narrow ? 128 : kFCols;
  for (int t = 0; t < a->n_tiles; t++)
    if ((a->tile_bounds[t + 1] - a->tile_bounds[t]) % cols) return AMOE_EUNSUPPORTED;
  *block_cols = cols;
  return narrow ? launch_bwdx256_cols<T, 128>(p, a, st, n_count_blocks)
                : launch_bwdx256_cols<T, kFCols>(p, a, st, n_count_blocks);
}

template <typename T>
int launch_fwd256(RowsParams p, int mode, const amoe_fwd_args* a, hipStream_t st) {
  if (!rows_all_interior(p, mode, kFBK) || a->N % kFCols) return AMOE_EUNSUPPORTED;
  if (a->noise != nullptr || a->n_tiles > 2) return AMOE_EUNSUPPORTED;
  const bool dac = a->ir != nullptr;                 // (interior launches have the range and the quantiser, or neither)
  if (dac && !a->ir_by_expert) return AMOE_EUNSUPPORTED;
  const bool adc = a->out_bound > 0.f, noisy = a->noise_std > 0.f;
  const bool analog = adc && a->out_res > 0.f && a->wmax_cols == 1 && dac;
  if ((adc || noisy) && !analog) return AMOE_EUNSUPPORTED;
  if (a->n_tiles == 2 && !(analog && !a->x_is_quantized)) return AMOE_EUNSUPPORTED;
  // the two-K-tile variant parks the first tile's ADC codes as bytes (code + 128): a finer output quantiser than
  // 254 states does not fit them, and the general kernel (fp32 partial results) serves the launch
  if (a->n_tiles == 2 && !(p.out_half_states <= 127.f)) return AMOE_EUNSUPPORTED;
  if (a->code_out && !analog) return AMOE_EUNSUPPORTED;
  if (a->code_out && (!amoe_fwd_codes_supported(a) || !aligned(a->code_out, 16))) return AMOE_EUNSUPPORTED;
  if (a->n_tiles == 1 && !a->relu && !a->xq_out && (a->x_is_quantized || !dac) && (a->code_out || !analog)) {
    // one K-tile of 256, the operand plain or already coded, the result plain, rescaled or as ADC codes: the
    // weights stay in registers and the rows stream past them
    RowsParams q = p;
    const int grid = a->code_out ? ws256_plan(q, a->n_out_rows, a->ldcode) : ws256_plan(q, a->n_out_rows, a->ldo * 2);
    if (grid > 0) {
      if (a->code_out) {
        if (noisy) hipLaunchKernelGGL((&ws256_kernel<T, false, 64, WS_ZCODES, true>), dim3(grid), dim3(kThreads), 0, st, q);
        else hipLaunchKernelGGL((&ws256_kernel<T, false, 64, WS_ZCODES, false>), dim3(grid), dim3(kThreads), 0, st, q);
      } else if (dac) {
        hipLaunchKernelGGL((&ws256_kernel<T, false, 64, WS_SCALE, false>), dim3(grid), dim3(kThreads), 0, st, q);
      } else {
        hipLaunchKernelGGL((&ws256_kernel<T, false, 64, WS_PLAIN, false>), dim3(grid), dim3(kThreads), 0, st, q);
      }
      return launch_rc();
    }
  }
  p.n_col_blocks = a->N / kFCols;
  const int grid = persistent_grid(max_row_tiles(a->M, a->E), p.n_col_blocks);
  if (!dac) return launch_fwd256_as<T, FA_PLAIN, false, false, false>(p, grid, st);
  if (!analog)
    return a->x_is_quantized ? launch_fwd256_as<T, FA_CODES, false, false, false>(p, grid, st)
                             : launch_fwd256_as<T, FA_DAC, false, false, false>(p, grid, st);
  if (a->code_out) {
    // codes leave instead of values: one output quantiser whose half range fits a byte, no second output
    if (a->x_is_quantized)
      return noisy ? launch_fwd256_as<T, FA_CODES, true, true, false, true>(p, grid, st)
                   : launch_fwd256_as<T, FA_CODES, true, false, false, true>(p, grid, st);
    return noisy ? launch_fwd256_as<T, FA_DAC, true, true, false, true>(p, grid, st)
                 : launch_fwd256_as<T, FA_DAC, true, false, false, true>(p, grid, st);
  }
  if (a->x_is_quantized)
    return noisy ? launch_fwd256_as<T, FA_CODES, true, true, false>(p, grid, st)
                 : launch_fwd256_as<T, FA_CODES, true, false, false>(p, grid, st);
  if (a->n_tiles == 2)
    return noisy ? launch_fwd256_as<T, FA_DAC, true, true, true>(p, grid, st)
                 : launch_fwd256_as<T, FA_DAC, true, false, true>(p, grid, st);
  return noisy ? launch_fwd256_as<T, FA_DAC, true, true, false>(p, grid, st)
               : launch_fwd256_as<T, FA_DAC, true, false, false>(p, grid, st);
}

}  // namespace

extern "C" {

int amoe_version(void) { return AMOE_VERSION; }

const char* amoe_strerror(int rc) {
  switch (rc) {
    case AMOE_OK: return "ok";
    case AMOE_EINVAL: return "invalid size, stride or scalar";
    case AMOE_ENULL: return "required pointer is NULL";
    case AMOE_ESHAPE: return "inconsistent sizes";
    case AMOE_EALIGN: return "pointer not aligned to 4 bytes";
    case AMOE_EWORKSPACE: return "workspace too small (or the call exceeds the library's own scratch array)";
    case AMOE_EUNSUPPORTED: return "not supported by this build";
    default: return rc > 0 ? "HIP launch error" : "unknown error";
  }
}

// ------------------------------------------------------------------------------ selection
size_t amoe_prepare_sel_workspace(int64_t M, int32_t E) {
  if (M < 0 || E < 1) return 0;
  const int64_t units = (M + sel_unit(M) - 1) / sel_unit(M);
  return (size_t)(units > 0 ? units : 1) * (size_t)E * sizeof(int32_t);
}

int amoe_prepare_sel(const void* sel, int32_t sel_is_i64, int64_t M, int32_t E, int32_t k,
                     int32_t* sel_sorted, int32_t* perm, int32_t* in_index, int32_t* offsets,
                     int32_t* bad_flag, void* workspace, size_t workspace_bytes, void* stream) {
  if (M < 0 || M > 0x7fffffffLL || E < 1 || k < 1) return AMOE_EINVAL;
  if (E > kSelMaxExperts) return AMOE_EUNSUPPORTED;
  if (!offsets || !workspace || (M > 0 && (!sel || !sel_sorted || !perm || !in_index))) return AMOE_ENULL;
  if (!aligned(sel, sel_is_i64 ? 8 : 4) || !aligned(sel_sorted, 4) || !aligned(perm, 4) ||
      !aligned(in_index, 4) || !aligned(offsets, 4) || !aligned(workspace, 4) || !aligned(bad_flag, 4))
    return AMOE_EALIGN;
  if (workspace_bytes < amoe_prepare_sel_workspace(M, E)) return AMOE_EWORKSPACE;
  SelParams p;
  p.sel = sel; p.sel_is_i64 = sel_is_i64; p.M = M; p.E = E; p.k = k;
  p.unit = sel_unit(M);
  p.n_units = (int)((M + p.unit - 1) / p.unit);
  p.key_bits = 0;
  while ((1 << p.key_bits) < E) p.key_bits++;
  p.sel_sorted = sel_sorted; p.perm = perm; p.in_index = in_index; p.offsets = offsets;
  p.bad_flag = bad_flag; p.unit_hist = static_cast<int32_t*>(workspace);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int blocks = (p.n_units + 3) / 4;
  if (blocks > 0) {
    hipLaunchKernelGGL(sel_hist_kernel, dim3(blocks), dim3(kThreads), 0, st, p);
    if (int rc = launch_rc()) return rc;
  }
  if (blocks > 0 && E <= kThreads && (long long)p.n_units * E <= kSelFuseMax && aligned(workspace, 16)) {
    // a small table of unit counts: every workgroup of the scatter pass scans it for itself
    hipLaunchKernelGGL(sel_scan_scatter_kernel, dim3(blocks), dim3(kThreads), 0, st, p);
    return launch_rc();
  }
  hipLaunchKernelGGL(sel_unit_scan_kernel, dim3((E + 3) / 4), dim3(kThreads), 0, st, p);
  if (int rc = launch_rc()) return rc;
  hipLaunchKernelGGL(sel_offsets_kernel, dim3(1), dim3(kThreads), 0, st, p);
  if (int rc = launch_rc()) return rc;
  if (blocks > 0) {
    hipLaunchKernelGGL(sel_scatter_kernel, dim3(blocks), dim3(kThreads), 0, st, p);
    if (int rc = launch_rc()) return rc;
  }
  return AMOE_OK;
}

// ---- selection without any allocation: the unit histograms live in a device array of the library ----------
}  // extern "C"

// One copy per GPU the library runs on, held until the process ends.  In host code the array's NAME is only a
// stand-in for the symbol, not a device address: the device address is asked for once per device and kept.
static __device__ __align__(256) unsigned char scratch[AMOE_NOALLOC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxDevices];

// Device address of `scratch` on the current device (looked up on the first call per device).
int scratch_address(void** out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= kMaxDevices) return AMOE_EUNSUPPORTED;
  void* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (ptr == nullptr) {
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return (int)e;
    if (ptr == nullptr) return AMOE_EUNSUPPORTED;
    g_scratch_ptr[dev].store(ptr, std::memory_order_release);   // every thread would store the same address
  }
  *out = ptr;
  return AMOE_OK;
}
}  // namespace

extern "C" {

size_t amoe_noalloc_scratch_bytes(void) { return AMOE_NOALLOC_SCRATCH_BYTES; }

int amoe_prepare_sel_noalloc(const void* sel, int32_t sel_is_i64, int64_t M, int32_t E, int32_t k,
                             int32_t* sel_sorted, int32_t* perm, int32_t* in_index, int32_t* offsets,
                             int32_t* bad_flag, void* stream) {
  if (M < 0 || M > 0x7fffffffLL || E < 1 || k < 1) return AMOE_EINVAL;
  if (E > kSelMaxExperts) return AMOE_EUNSUPPORTED;
  // the histograms of this call must fit the library's array; nothing is allocated to make room
  if (amoe_prepare_sel_workspace(M, E) > (size_t)AMOE_NOALLOC_SCRATCH_BYTES) return AMOE_EWORKSPACE;
  void* ws = nullptr;
  if (int rc = scratch_address(&ws)) return rc;
  // every unit's histogram row is written by the first pass before anything reads it, so what the previous
  // call left in the array does not matter and nothing has to be cleared
  return amoe_prepare_sel(sel, sel_is_i64, M, E, k, sel_sorted, perm, in_index, offsets, bad_flag, ws,
                          (size_t)AMOE_NOALLOC_SCRATCH_BYTES, stream);
}

int amoe_offsets_from_sorted(const int32_t* sel_sorted, int64_t M, int32_t E, int32_t* offsets, void* stream) {
  if (M < 0 || M > 0x7fffffffLL || E < 1) return AMOE_EINVAL;
  if (!offsets || (M > 0 && !sel_sorted)) return AMOE_ENULL;
  if (!aligned(sel_sorted, 4) || !aligned(offsets, 4)) return AMOE_EALIGN;
  const int blocks = (int)((M + 1 + kThreads - 1) / kThreads);
  hipLaunchKernelGGL(offsets_from_sorted_kernel, dim3(blocks), dim3(kThreads), 0, static_cast<hipStream_t>(stream),
                     sel_sorted, (long long)M, (int)E, offsets);
  return launch_rc();
}

// ------------------------------------------------------------------------------ forward
int amoe_fwd_codes_supported(const amoe_fwd_args* a) {
  if (!a || (a->dtype != AMOE_BF16 && a->dtype != AMOE_F16)) return 0;
  if (a->N < 1 || a->K < 1 || a->E < 1 || a->n_tiles != 1 || a->w_stride_n != 1) return 0;
  // every tile interior, 16-byte pieces everywhere, 32-bit byte offsets
  if (a->N % kFCols || a->K % kFBK || a->ldx % 8 || a->w_stride_e % 8 || a->w_stride_k % 8 || a->ldcode % 16) return 0;
  if (a->ldx < a->K || a->w_stride_k < a->N || a->ldcode < a->N) return 0;
  const long long lim = 1LL << 31;
  if (a->n_in_rows <= 0 || (long long)a->n_in_rows * a->ldx * 2 >= lim ||
      ((long long)a->K * a->w_stride_k + (long long)a->N) * 2 >= lim)
    return 0;
  // the analog stages the kernel is built for: per-expert input ranges with an input quantiser whose codes the type
  // holds, one max |W| per expert, generated noise or none, an output quantiser whose codes fit a byte
  if (!a->ir || !a->ir_by_expert || !(a->inp_res > 0.f) || !dac_codes_fit(a->dtype, a->inp_res) || a->abs_max) return 0;
  if (a->noise || !a->wmax || a->wmax_cols != 1 || !(a->out_bound > 0.f) || !(a->out_res > 0.f)) return 0;
  if (!(0.5f * fmaxf(a->out_res, 1.0f / a->out_res) <= 127.f)) return 0;
  if (a->xq_out || a->relu) return 0;
  return 1;
}

int amoe_cvmm_fwd(const amoe_fwd_args* a, void* stream) {
  if (!a) return AMOE_ENULL;
  if (a->dtype != AMOE_F32 && a->dtype != AMOE_BF16 && a->dtype != AMOE_F16) return AMOE_EINVAL;
  if (a->M < 0 || a->N < 1 || a->K < 1 || a->E < 1 || a->n_in_rows < 0 || a->n_out_rows < 0) return AMOE_EINVAL;
  if (a->M == 0) return AMOE_OK;
  if (!a->x || !a->w || (!a->out && !a->code_out) || !a->offsets || !a->in_index) return AMOE_ENULL;
  if (a->code_out && (!a->code_scale_out || a->ldcode < a->N)) return AMOE_EINVAL;
  if (int rc = check_bounds(a->n_tiles, a->tile_bounds, a->K)) return rc;
  if (a->ldx < a->K || (a->out && a->ldo < a->N)) return AMOE_ESHAPE;
  if (a->w_stride_n != 1 && a->w_stride_k != 1) return AMOE_EUNSUPPORTED;
  const bool gen_noise = a->noise == nullptr && a->noise_std > 0.f;
  const bool adc = a->out_bound > 0.f;
  if ((gen_noise || adc) && (!a->wmax || (a->wmax_cols != 1 && a->wmax_cols != a->N))) return AMOE_ESHAPE;
  if (a->noise && (a->ldnoise < a->N)) return AMOE_ESHAPE;
  if (a->xq_out && (!a->xq_ir || !(a->xq_inp_res > 0.f))) return AMOE_EINVAL;
  if (a->xq_out && a->ldxq < a->N) return AMOE_ESHAPE;
  if (a->x_is_quantized && (!a->ir || !(a->inp_res > 0.f) || a->abs_max || a->n_tiles != 1)) return AMOE_EINVAL;
  // 16-bit element types carry the DAC codes themselves to the matrix unit (and in xq_out): integers are exact up
  // to 256 in bf16 and 2048 in fp16, so a finer input quantiser needs fp32 tensors
  if (!dac_codes_fit(a->dtype, a->inp_res) || (a->xq_out && !dac_codes_fit(a->dtype, a->xq_inp_res)))
    return AMOE_EUNSUPPORTED;
  const size_t es = esize(a->dtype);
  if (!aligned(a->x, es) || !aligned(a->w, es) || !aligned(a->out, es) || !aligned(a->offsets, 4) ||
      !aligned(a->in_index, 4) || !aligned(a->out_index, 4) || !aligned(a->ir, 4) || !aligned(a->abs_max, 4) ||
      !aligned(a->noise, 4) || !aligned(a->wmax, 4) || !aligned(a->range_flag, 4) || !aligned(a->noise_seed_dev, 8) ||
      !aligned(a->xq_out, es) || !aligned(a->xq_ir, 4))
    return AMOE_EALIGN;

  const int CH = a->dtype == AMOE_F32 ? 4 : 8;
  RowsParams p{};
  p.M = a->M; p.E = a->E; p.KD = a->K; p.ND = a->N;
  p.a = a->x; p.lda = a->ldx;
  p.w = a->w; p.w_se = a->w_stride_e; p.w_skd = a->w_stride_k; p.w_snd = a->w_stride_n;
  p.out = a->out; p.ldo = a->ldo;
  p.offsets = a->offsets; p.a_index = a->in_index; p.out_index = a->out_index;
  p.n_kd_tiles = a->n_tiles;
  for (int t = 0; t <= a->n_tiles; t++) p.kd_bounds[t] = a->tile_bounds[t];
  p.n_col_tiles = 1; p.col_bounds[0] = 0; p.col_bounds[1] = a->N;
  p.n_col_blocks = count_col_blocks(p.col_bounds, 1);
  p.ir = a->ir; p.ir_cols = a->n_tiles; p.ir_by_expert = a->ir_by_expert; p.abs_max = a->abs_max;
  p.inp_res = a->inp_res;
  p.noise = a->noise; p.noise_ts = a->noise_tile_stride; p.ldnoise = a->ldnoise;
  p.noise_std = a->noise_std; p.seed = a->noise_seed; p.seed_dev = a->noise_seed_dev;
  p.wmax = a->wmax; p.wmax_cols = a->wmax_cols;
  p.out_bound = a->out_bound;
  p.out_half_states = (adc && a->out_res > 0.f) ? 0.5f * fmaxf(a->out_res, 1.0f / a->out_res) : 0.f;
  p.relu = a->relu; p.range_flag = a->range_flag;
  p.xq_out = a->xq_out; p.ldxq = a->ldxq; p.xq_ir = a->xq_ir; p.xq_inp_res = a->xq_inp_res;
  p.xq_vec = a->xq_out && aligned(a->xq_out, 16) && (a->ldxq % 4 == 0);
  p.xq_stage = a->xq_out && aligned(a->xq_out, 16) && (a->ldxq % CH == 0);
  p.a_prequant = a->x_is_quantized;
  p.code_out = a->code_out; p.ldcode = a->ldcode; p.code_scale_out = a->code_scale_out;
  const bool w_kc = a->w_stride_n != 1;
  p.a_vec = aligned(a->x, 16) && (a->ldx % CH == 0) && bounds_multiple_of(a->n_tiles, a->tile_bounds, CH);
  p.w_vec = aligned(a->w, 16) && (a->w_stride_e % CH == 0) &&
            (w_kc ? (a->w_stride_n % CH == 0 && bounds_multiple_of(a->n_tiles, a->tile_bounds, CH))
                  : (a->w_stride_k % CH == 0));
  p.out_vec = aligned(a->out, 16) && (a->ldo % 4 == 0);
  p.out_stage = aligned(a->out, 16) && (a->ldo % CH == 0);
  p.noise_vec = a->noise && aligned(a->noise, 16) && (a->ldnoise % 4 == 0) && (a->noise_tile_stride % 4 == 0);
  const long long lim = 1LL << 31;
  // (n_in_rows == 0: the caller does not state the rows of x, so nothing bounds its extent)
  p.buf_ok = a->n_in_rows > 0 && (long long)a->n_in_rows * a->ldx * (long long)es < lim &&
             ((long long)a->K * a->w_stride_k + (long long)a->N * a->w_stride_n) * (long long)es < lim;
  const int mode = a->n_tiles > 1 ? MODE_FWD_SPLIT : MODE_FWD;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (a->dtype != AMOE_F32 && !w_kc) {
    const int rc = a->dtype == AMOE_F16 ? launch_fwd256<f16_t>(p, mode, a, st) : launch_fwd256<uint16_t>(p, mode, a, st);
    if (rc != AMOE_EUNSUPPORTED) return rc;
  }
  if (a->code_out) return AMOE_EUNSUPPORTED;      // only the kernel above writes codes
  const int grid = persistent_grid(max_row_tiles(a->M, a->E), p.n_col_blocks);
  if (a->dtype == AMOE_F32)
    return w_kc ? launch_rows<float, true>(p, mode, grid, st) : launch_rows<float, false>(p, mode, grid, st);
  if (a->dtype == AMOE_F16)
    return w_kc ? launch_rows<f16_t, true>(p, mode, grid, st) : launch_rows<f16_t, false>(p, mode, grid, st);
  return w_kc ? launch_rows<uint16_t, true>(p, mode, grid, st) : launch_rows<uint16_t, false>(p, mode, grid, st);
}

// ------------------------------------------------------------------------------ weight gradient
namespace {
// Rows per chunk of the weight gradient: enough (expert, chunk, tile) workgroups to fill the chip
// twice over, chunks of 256 .. 4096 rows; 0 when one chunk per expert already does that.
struct WgradSplit { int rows_per_chunk; long long slots; int tiles; };
WgradSplit wgrad_split(const amoe_bwd_w_args* a) {
  WgradSplit s{0, 0, 0};
  const int kb = count_col_blocks(a->tile_bounds, a->n_tiles);
  const int nb = (a->N + kTileCols - 1) / kTileCols;
  s.tiles = kb * nb;
  long long R;
  if (a->rows_per_chunk > 0) {
    R = ((long long)a->rows_per_chunk + 63) / 64 * 64;
  } else {
    const long long target = 4LL * num_compute_units();
    const long long chunks = (target + s.tiles - 1) / s.tiles;
    R = chunks > 0 ? (a->M + chunks - 1) / chunks : a->M;
    R = (R + 255) / 256 * 256;
    R = R < 256 ? 256 : (R > 4096 ? 4096 : R);
  }
  if (R >= a->M) return s;                 // a single chunk everywhere
  s.rows_per_chunk = (int)R;
  s.slots = 2LL * a->M / R + 1;            // bound on the chunks of the experts that are cut
  return s;
}
}  // namespace

size_t amoe_bwd_w_workspace(const amoe_bwd_w_args* a) {
  if (!a || a->M < 1 || a->N < 1 || a->K < 1 || a->E < 1) return 0;
  if (check_bounds(a->n_tiles, a->tile_bounds, a->K)) return 0;
  const WgradSplit s = wgrad_split(a);
  if (s.rows_per_chunk == 0) return 0;
  return (size_t)s.slots * s.tiles * kWgradTileElems * sizeof(float);
}

int amoe_cvmm_bwd_w(const amoe_bwd_w_args* a, void* stream) {
  if (!a) return AMOE_ENULL;
  if (a->dtype != AMOE_F32 && a->dtype != AMOE_BF16 && a->dtype != AMOE_F16) return AMOE_EINVAL;
  if (a->M < 0 || a->N < 1 || a->K < 1 || a->E < 1 || a->n_x_rows < 0 || a->n_g_rows < 0) return AMOE_EINVAL;
  if (!a->grad_w || !a->offsets) return AMOE_ENULL;
  if (a->M > 0 && (!a->x || !a->g || !a->in_index)) return AMOE_ENULL;
  if (int rc = check_bounds(a->n_tiles, a->tile_bounds, a->K)) return rc;
  if (a->M > 0 && (a->ldx < a->K || a->ldg < a->N)) return AMOE_ESHAPE;
  const size_t es = esize(a->dtype);
  if (!aligned(a->x, es) || !aligned(a->g, es) || !aligned(a->grad_w, es) || !aligned(a->offsets, 4) ||
      !aligned(a->in_index, 4) || !aligned(a->g_index, 4) || !aligned(a->ir, 4) || !aligned(a->g_scale, es))
    return AMOE_EALIGN;
  const int CH = a->dtype == AMOE_F32 ? 4 : 8;
  WgradParams p{};
  p.M = a->M; p.N = a->N; p.K = a->K; p.E = a->E;
  p.x = a->x; p.ldx = a->ldx; p.g = a->g; p.ldg = a->ldg; p.grad_w = a->grad_w;
  p.offsets = a->offsets; p.in_index = a->in_index; p.g_index = a->g_index;
  p.ir = a->ir; p.ir_by_expert = a->ir_by_expert; p.g_scale = a->g_scale; p.n_tiles = a->n_tiles;
  for (int t = 0; t <= a->n_tiles; t++) p.bounds[t] = a->tile_bounds[t];
  p.n_k_blocks = count_col_blocks(p.bounds, p.n_tiles);
  p.n_n_blocks = (a->N + kTileCols - 1) / kTileCols;
  p.x_vec = aligned(a->x, 16) && (a->ldx % CH == 0) && bounds_multiple_of(a->n_tiles, a->tile_bounds, CH);
  p.g_vec = aligned(a->g, 16) && (a->ldg % CH == 0);
  p.out_vec = aligned(a->grad_w, 16) && (a->N % 4 == 0);
  p.out_stage = aligned(a->grad_w, 16) && (a->N % CH == 0);
  p.buf_ok = a->n_x_rows > 0 && a->n_g_rows > 0 && a->n_x_rows * a->ldx * (long long)es < (1LL << 31) &&
             a->n_g_rows * a->ldg * (long long)es < (1LL << 31);
  hipStream_t st = static_cast<hipStream_t>(stream);
  long long pairs = a->E;                  // (expert, chunk) pairs, worst case
  if (a->workspace != nullptr && a->M > 0) {
    const WgradSplit s = wgrad_split(a);
    if (s.rows_per_chunk > 0) {
      if (!aligned(a->workspace, 16)) return AMOE_EALIGN;
      if (a->workspace_bytes < amoe_bwd_w_workspace(a)) return AMOE_EWORKSPACE;
      if (a->E > kSelMaxExperts) return AMOE_EUNSUPPORTED;
      p.rows_per_chunk = s.rows_per_chunk;
      p.partial = static_cast<float*>(a->workspace);
      pairs = a->M / s.rows_per_chunk + a->E;
    }
  }
  const long long grid = 8LL * ((pairs + 7) / 8) * p.n_k_blocks * p.n_n_blocks;   // see the id mapping in the kernel
  if (grid > 0x7fffffffLL) return AMOE_EUNSUPPORTED;
  const long long rgrid = (long long)a->E * p.n_k_blocks * p.n_n_blocks * kWgradReduceSplit;
  if (rgrid > 0x7fffffffLL) return AMOE_EUNSUPPORTED;
  // the 256 x 256 kernel for the training shapes (16-bit elements, interior tiles, per-expert ranges)
  bool wide = a->dtype != AMOE_F32 && p.x_vec && p.g_vec && p.out_stage && p.buf_ok && a->N % kW256Tile == 0 &&
              (a->ir == nullptr || a->ir_by_expert);
  for (int t = 0; t < a->n_tiles && wide; t++) wide = (a->tile_bounds[t + 1] - a->tile_bounds[t]) % kW256Tile == 0;
  if (wide) {
    const long long grid256 = 8LL * ((pairs + 7) / 8) * (p.n_k_blocks / 2) * (p.n_n_blocks / 2);
    if (a->dtype == AMOE_BF16) {
      hipLaunchKernelGGL((&wgrad256_kernel<uint16_t>), dim3((unsigned)grid256), dim3(kW256Threads), 0, st, p);
    } else {
      hipLaunchKernelGGL((&wgrad256_kernel<f16_t>), dim3((unsigned)grid256), dim3(kW256Threads), 0, st, p);
    }
    if (int rc = launch_rc()) return rc;
    if (p.rows_per_chunk > 0) {
      if (a->dtype == AMOE_BF16) {
        hipLaunchKernelGGL((&wgrad_reduce_kernel<uint16_t>), dim3((unsigned)rgrid), dim3(kThreads), 0, st, p);
      } else {
        hipLaunchKernelGGL((&wgrad_reduce_kernel<f16_t>), dim3((unsigned)rgrid), dim3(kThreads), 0, st, p);
      }
    }
    return launch_rc();
  }
  if (a->dtype == AMOE_F32) {
    auto k = &gemm_wgrad_kernel<float>;
    hipLaunchKernelGGL(k, dim3((unsigned)grid), dim3(kThreads), 0, st, p);
    if (int rc = launch_rc()) return rc;
    if (p.rows_per_chunk > 0) {
      auto r = &wgrad_reduce_kernel<float>;
      hipLaunchKernelGGL(r, dim3((unsigned)rgrid), dim3(kThreads), 0, st, p);
    }
  } else if (a->dtype == AMOE_BF16) {
    auto k = &gemm_wgrad_kernel<uint16_t>;
    hipLaunchKernelGGL(k, dim3((unsigned)grid), dim3(kThreads), 0, st, p);
    if (int rc = launch_rc()) return rc;
    if (p.rows_per_chunk > 0) {
      auto r = &wgrad_reduce_kernel<uint16_t>;
      hipLaunchKernelGGL(r, dim3((unsigned)rgrid), dim3(kThreads), 0, st, p);
    }
  } else {
    auto k = &gemm_wgrad_kernel<f16_t>;
    hipLaunchKernelGGL(k, dim3((unsigned)grid), dim3(kThreads), 0, st, p);
    if (int rc = launch_rc()) return rc;
    if (p.rows_per_chunk > 0) {
      auto r = &wgrad_reduce_kernel<f16_t>;
      hipLaunchKernelGGL(r, dim3((unsigned)rgrid), dim3(kThreads), 0, st, p);
    }
  }
  return launch_rc();
}

// ------------------------------------------------------------------------------ input gradient
size_t amoe_bwd_x_workspace(int64_t M, int32_t K, int32_t n_tiles) {
  if (M < 0 || K < 1 || n_tiles < 1) return 0;
  // worst case: every K-tile adds one partial column block
  const int64_t col_blocks = (K + kTileCols - 1) / kTileCols + n_tiles;
  const int64_t row_tiles = M / kTileRows + kSelMaxExperts;
  return (size_t)(col_blocks * (M > 0 ? M : 1)) * sizeof(float) + (size_t)(row_tiles * col_blocks) * sizeof(int32_t);
}

int amoe_cvmm_bwd_x(const amoe_bwd_x_args* a, void* stream) {
  if (!a) return AMOE_ENULL;
  if (a->dtype != AMOE_F32 && a->dtype != AMOE_BF16 && a->dtype != AMOE_F16) return AMOE_EINVAL;
  if (a->M < 0 || a->N < 1 || a->K < 1 || a->E < 1 || a->E > kSelMaxExperts || a->n_g_rows < 0) return AMOE_EINVAL;
  if (a->M == 0) return AMOE_OK;
  if (!a->g || !a->w || !a->grad_x_full || !a->offsets || !a->g_index || !a->out_index) return AMOE_ENULL;
  if (int rc = check_bounds(a->n_tiles, a->tile_bounds, a->K)) return rc;
  const bool use_ir = a->ir != nullptr;
  if ((use_ir || a->relu_mask) && (!a->x || !a->xf_index)) return AMOE_ENULL;
  if (use_ir && (!a->ir_grad || !a->workspace)) return AMOE_ENULL;
  if (a->xc_out && (!a->x || !a->xf_index)) return AMOE_ENULL;
  if (a->xc_out && a->ldxc < a->K) return AMOE_ESHAPE;
  if (a->ldg < a->N || a->ldo < a->K || (a->x && a->ldx < a->K) || a->w_stride_k < a->N) return AMOE_ESHAPE;
  const size_t es = esize(a->dtype);
  if (!aligned(a->g, es) || !aligned(a->w, es) || !aligned(a->grad_x_full, es) || !aligned(a->x, es) ||
      !aligned(a->gate, es) || !aligned(a->offsets, 4) || !aligned(a->g_index, 4) || !aligned(a->out_index, 4) ||
      !aligned(a->xf_index, 4) || !aligned(a->ir, 4) || !aligned(a->ir_grad, 4) || !aligned(a->workspace, 4))
    return AMOE_EALIGN;
  const int CH = a->dtype == AMOE_F32 ? 4 : 8;
  RowsParams p{};
  p.M = a->M; p.E = a->E; p.KD = a->N; p.ND = a->K;
  p.a = a->g; p.lda = a->ldg;
  p.w = a->w; p.w_se = a->w_stride_e; p.w_skd = 1; p.w_snd = a->w_stride_k;
  p.out = a->grad_x_full; p.ldo = a->ldo;
  p.offsets = a->offsets; p.a_index = a->g_index; p.out_index = a->out_index;
  p.n_kd_tiles = 1; p.kd_bounds[0] = 0; p.kd_bounds[1] = a->N;
  p.n_col_tiles = a->n_tiles;
  for (int t = 0; t <= a->n_tiles; t++) p.col_bounds[t] = a->tile_bounds[t];
  p.n_col_blocks = count_col_blocks(p.col_bounds, p.n_col_tiles);
  p.ir = a->ir; p.ir_cols = a->n_tiles; p.ir_by_expert = a->ir_by_expert; p.inp_res = -1.f;
  p.xf = a->x; p.ldxf = a->ldx; p.xf_index = a->xf_index; p.gate = a->gate; p.relu_mask = a->relu_mask;
  p.xc_out = a->xc_out; p.ldxc = a->ldxc;
  p.xc_vec = a->xc_out && aligned(a->xc_out, 16) && (a->ldxc % CH == 0) && bounds_multiple_of(a->n_tiles, a->tile_bounds, CH);
  const int grid = persistent_grid(max_row_tiles(a->M, a->E), p.n_col_blocks);
  if (use_ir) {
    // (one count per workgroup; no grid is larger than the number of work items)
    const size_t need = (size_t)p.n_col_blocks * a->M * sizeof(float) +
                        (size_t)max_row_tiles(a->M, a->E) * p.n_col_blocks * sizeof(int32_t);
    if (a->workspace_bytes < need) return AMOE_EWORKSPACE;
    p.irg_partial = static_cast<float*>(a->workspace);
    p.notclip_count = reinterpret_cast<int32_t*>(p.irg_partial + (size_t)p.n_col_blocks * a->M);
  }
  p.a_vec = aligned(a->g, 16) && (a->ldg % CH == 0);
  p.w_vec = aligned(a->w, 16) && (a->w_stride_e % CH == 0) && (a->w_stride_k % CH == 0);
  p.buf_ok = a->n_g_rows > 0 && (long long)a->n_g_rows * a->ldg * (long long)es < (1LL << 31) &&
             (long long)a->K * a->w_stride_k * (long long)es < (1LL << 31);
  p.out_vec = aligned(a->grad_x_full, 16) && (a->ldo % 4 == 0) && bounds_multiple_of(a->n_tiles, a->tile_bounds, 4);
  p.out_stage = aligned(a->grad_x_full, 16) && (a->ldo % CH == 0) && bounds_multiple_of(a->n_tiles, a->tile_bounds, CH);
  p.xf_vec = a->x && aligned(a->x, 16) && (a->ldx % 4 == 0) && bounds_multiple_of(a->n_tiles, a->tile_bounds, 4);
  hipStream_t st = static_cast<hipStream_t>(stream);
  int block_cols = kTileCols, n_count_blocks = grid;
  int rc = AMOE_EUNSUPPORTED;
  if (a->dtype != AMOE_F32) {
    int cols = kTileCols;
    rc = a->dtype == AMOE_F16 ? launch_bwdx256<f16_t>(p, a, st, &n_count_blocks, &cols)
                              : launch_bwdx256<uint16_t>(p, a, st, &n_count_blocks, &cols);
    if (rc == AMOE_OK) block_cols = cols;
  }
  if (rc == AMOE_EUNSUPPORTED)
    rc = a->dtype == AMOE_F32   ? launch_rows<float, true>(p, MODE_BWDX, grid, st)
         : a->dtype == AMOE_F16 ? launch_rows<f16_t, true>(p, MODE_BWDX, grid, st)
                                : launch_rows<uint16_t, true>(p, MODE_BWDX, grid, st);
  if (rc) return rc;
  if (use_ir) {
    IrFinalizeParams f{};
    f.M = a->M; f.n_tiles = a->n_tiles; f.KD_total = a->K; f.block_cols = block_cols;
    for (int t = 0; t <= a->n_tiles; t++) f.col_bounds[t] = a->tile_bounds[t];
    f.irg_partial = p.irg_partial; f.notclip_count = p.notclip_count; f.n_blocks = n_count_blocks;
    f.ir = a->ir; f.ir_by_expert = a->ir_by_expert; f.offsets = a->offsets; f.E = a->E; f.ir_grad = a->ir_grad;
    f.relative = a->gradient_relative; f.scale = a->gradient_scale; f.decay = a->decay;
    f.min_pct = a->input_min_percentage;
    hipLaunchKernelGGL(ir_grad_finalize_kernel, dim3((a->M + kThreads - 1) / kThreads), dim3(kThreads), 0, st, f);
    rc = launch_rc();
  }
  return rc;
}

// ------------------------------------------------------------------------------ row-wise companions
static int bump_only(int64_t* counter, int64_t counter_add, void* stream);

static int head_reduce(int32_t dtype, const void* z, const void* gate, void* y, int64_t T, int32_t k, int32_t D,
                       void* stream, int64_t* counter_ = nullptr, int64_t counter_add_ = 0) {
  if (dtype != AMOE_F32 && dtype != AMOE_BF16 && dtype != AMOE_F16) return AMOE_EINVAL;
  if (T < 0 || k < 1 || D < 1) return AMOE_EINVAL;
  if (!aligned(counter_, 8)) return AMOE_EALIGN;
  if (T == 0) return bump_only(counter_, counter_add_, stream);
  long long* counter = reinterpret_cast<long long*>(counter_);
  const long long counter_add = counter_add_;
  if (!z || !y) return AMOE_ENULL;
  const size_t es = esize(dtype);
  if (!aligned(z, es) || !aligned(y, es) || !aligned(gate, es)) return AMOE_EALIGN;
  const int CH = dtype == AMOE_F32 ? 4 : 8;
  const int vec = aligned(z, 16) && aligned(y, 16) && (D % CH == 0);
  const long long work = (long long)T * ((D + CH - 1) / CH);
  const long long blocks = (work + kThreads - 1) / kThreads;
  if (blocks > 0x7fffffffLL) return AMOE_EUNSUPPORTED;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == AMOE_F32) {
    auto kf = &head_reduce_kernel<float>;
    hipLaunchKernelGGL(kf, dim3((unsigned)blocks), dim3(kThreads), 0, st, static_cast<const float*>(z),
                       static_cast<const float*>(gate), static_cast<float*>(y), (long long)T, (int)k, (int)D, vec,
                       counter, counter_add);
  } else if (dtype == AMOE_BF16) {
    auto kf = &head_reduce_kernel<uint16_t>;
    hipLaunchKernelGGL(kf, dim3((unsigned)blocks), dim3(kThreads), 0, st, static_cast<const uint16_t*>(z),
                       static_cast<const uint16_t*>(gate), static_cast<uint16_t*>(y), (long long)T, (int)k, (int)D,
                       vec, counter, counter_add);
  } else {
    auto kf = &head_reduce_kernel<f16_t>;
    hipLaunchKernelGGL(kf, dim3((unsigned)blocks), dim3(kThreads), 0, st, static_cast<const f16_t*>(z),
                       static_cast<const f16_t*>(gate), static_cast<f16_t*>(y), (long long)T, (int)k, (int)D,
                       vec, counter, counter_add);
  }
  return launch_rc();
}

// the counter still moves when a call has no rows to reduce
__global__ void bump_kernel(long long* counter, long long add) { bump_counter(counter, add); }
static int bump_only(int64_t* counter, int64_t counter_add, void* stream) {
  if (!counter) return AMOE_OK;
  hipLaunchKernelGGL(bump_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream),
                     reinterpret_cast<long long*>(counter), (long long)counter_add);
  return launch_rc();
}

int amoe_gate_reduce(int32_t dtype, const void* z, const void* gate, void* y, int64_t T, int32_t k, int32_t D,
                     int64_t* counter, int64_t counter_add, void* stream) {
  if (T > 0 && !gate) return AMOE_ENULL;
  return head_reduce(dtype, z, gate, y, T, k, D, stream, counter, counter_add);
}

int amoe_ksum(int32_t dtype, const void* full, void* out, int64_t T, int32_t k, int32_t D, void* stream) {
  return head_reduce(dtype, full, nullptr, out, T, k, D, stream);
}

constexpr int kHeadClipBlocks = 1024;      // workgroups of the head sum with the clip: four per CU, all resident

size_t amoe_ksum_clip_workspace(int64_t T, int32_t k, int32_t n_tiles) {
  if (T < 0 || k < 1 || n_tiles < 1) return 0;
  return (size_t)n_tiles * (size_t)(T > 0 ? T * k : 1) * sizeof(float) + (size_t)kHeadClipBlocks * sizeof(int32_t);
}

int amoe_ksum_clip(const amoe_ksum_clip_args* a, void* stream) {
  if (!a) return AMOE_ENULL;
  if (a->dtype != AMOE_F32 && a->dtype != AMOE_BF16 && a->dtype != AMOE_F16) return AMOE_EINVAL;
  if (a->T < 0 || a->k < 1 || a->D < 1 || a->E < 1 || a->E > kSelMaxExperts) return AMOE_EINVAL;
  if (int rc = check_bounds(a->n_tiles, a->tile_bounds, a->D)) return rc;
  const long long M = (long long)a->T * a->k;
  if (M > 0x7fffffffLL) return AMOE_EUNSUPPORTED;
  if (a->T == 0) return AMOE_OK;
  if (!a->full || !a->x || !a->sel || !a->perm || !a->offsets || !a->ir || !a->grad_x || !a->ir_grad || !a->workspace)
    return AMOE_ENULL;
  if (a->ldx < a->D) return AMOE_ESHAPE;
  const int CH = a->dtype == AMOE_F32 ? 4 : 8;
  if (!aligned(a->full, 16) || !aligned(a->x, 16) || !aligned(a->grad_x, 16) || !aligned(a->sel, a->sel_is_i64 ? 8 : 4) ||
      !aligned(a->perm, 4) || !aligned(a->offsets, 4) || !aligned(a->ir, 4) || !aligned(a->ir_grad, 4) ||
      !aligned(a->workspace, 4))
    return AMOE_EALIGN;
  if (a->k > 8 || a->D % CH || a->ldx % CH || !bounds_multiple_of(a->n_tiles, a->tile_bounds, CH)) return AMOE_EUNSUPPORTED;
  if (a->workspace_bytes < amoe_ksum_clip_workspace(a->T, a->k, a->n_tiles)) return AMOE_EWORKSPACE;
  HeadClipParams p{};
  p.full = a->full; p.x = a->x; p.ldx = a->ldx; p.out = a->grad_x;
  p.sel = a->sel; p.sel_is_i64 = a->sel_is_i64;
  p.ir = a->ir; p.n_tiles = a->n_tiles;
  for (int t = 0; t <= a->n_tiles; t++) p.bounds[t] = a->tile_bounds[t];
  p.row_part = static_cast<float*>(a->workspace);
  p.count = reinterpret_cast<int32_t*>(p.row_part + (size_t)a->n_tiles * M);
  p.tokens = a->T; p.k = a->k; p.D = a->D;
  const long long want = (a->T + 3) / 4;
  const int blocks = (int)(want < kHeadClipBlocks ? want : kHeadClipBlocks);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (a->dtype == AMOE_F32) hipLaunchKernelGGL((&head_sum_clip_kernel<float>), dim3(blocks), dim3(kThreads), 0, st, p);
  else if (a->dtype == AMOE_BF16) hipLaunchKernelGGL((&head_sum_clip_kernel<uint16_t>), dim3(blocks), dim3(kThreads), 0, st, p);
  else hipLaunchKernelGGL((&head_sum_clip_kernel<f16_t>), dim3(blocks), dim3(kThreads), 0, st, p);
  if (int rc = launch_rc()) return rc;
  IrFinalizeParams f{};
  f.M = (int)M; f.n_tiles = a->n_tiles; f.KD_total = a->D; f.block_cols = a->D;     // one partial sum per K-tile
  for (int t = 0; t <= a->n_tiles; t++) f.col_bounds[t] = a->tile_bounds[t];
  f.irg_partial = p.row_part; f.notclip_count = p.count; f.n_blocks = blocks; f.row_index = a->perm;
  f.ir = a->ir; f.ir_by_expert = 1; f.offsets = a->offsets; f.E = a->E; f.ir_grad = a->ir_grad;
  f.relative = a->gradient_relative; f.scale = a->gradient_scale; f.decay = a->decay;
  f.min_pct = a->input_min_percentage;
  hipLaunchKernelGGL(ir_grad_finalize_kernel, dim3((unsigned)((M + kThreads - 1) / kThreads)), dim3(kThreads), 0, st, f);
  return launch_rc();
}

int amoe_gate_grad(int32_t dtype, const void* z, const void* dy, void* grad_gate, int64_t T, int32_t k, int32_t D,
                   void* stream) {
  if (dtype != AMOE_F32 && dtype != AMOE_BF16 && dtype != AMOE_F16) return AMOE_EINVAL;
  if (T < 0 || k < 1 || D < 1) return AMOE_EINVAL;
  if (T == 0) return AMOE_OK;
  if (!z || !dy || !grad_gate) return AMOE_ENULL;
  const size_t es = esize(dtype);
  if (!aligned(z, es) || !aligned(dy, es) || !aligned(grad_gate, es)) return AMOE_EALIGN;
  const long long blocks = ((long long)T + 3) / 4;            // one wave per token
  if (blocks > 0x7fffffffLL) return AMOE_EUNSUPPORTED;
  const int vec = aligned(z, 16) && aligned(dy, 16) && (D % (dtype == AMOE_F32 ? 4 : 8) == 0);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == AMOE_F32) {
    auto kf = &gate_grad_kernel<float>;
    hipLaunchKernelGGL(kf, dim3((unsigned)blocks), dim3(kThreads), 0, st, static_cast<const float*>(z),
                       static_cast<const float*>(dy), static_cast<float*>(grad_gate), (long long)T, (int)k, (int)D, vec);
  } else if (dtype == AMOE_BF16) {
    auto kf = &gate_grad_kernel<uint16_t>;
    hipLaunchKernelGGL(kf, dim3((unsigned)blocks), dim3(kThreads), 0, st, static_cast<const uint16_t*>(z),
                       static_cast<const uint16_t*>(dy), static_cast<uint16_t*>(grad_gate), (long long)T, (int)k, (int)D, vec);
  } else {
    auto kf = &gate_grad_kernel<f16_t>;
    hipLaunchKernelGGL(kf, dim3((unsigned)blocks), dim3(kThreads), 0, st, static_cast<const f16_t*>(z),
                       static_cast<const f16_t*>(dy), static_cast<f16_t*>(grad_gate), (long long)T, (int)k, (int)D, vec);
  }
  return launch_rc();
}

static int codes_args_ok(int32_t dtype, const uint8_t* codes, const float* scale, const void* sel, int32_t sel_is_i64,
                         const void* a, const void* b, int64_t T, int32_t k, int32_t D) {
  if (dtype != AMOE_F32 && dtype != AMOE_BF16 && dtype != AMOE_F16) return AMOE_EINVAL;
  if (T < 0 || k < 1 || D < 1) return AMOE_EINVAL;
  if (D % 16) return AMOE_EUNSUPPORTED;
  if (T == 0) return AMOE_OK;
  if (!codes || !scale || !sel || !a || !b) return AMOE_ENULL;
  if (!aligned(codes, 16) || !aligned(scale, 4) || !aligned(sel, sel_is_i64 ? 8 : 4) || !aligned(a, esize(dtype)) ||
      !aligned(b, 16))
    return AMOE_EALIGN;
  return AMOE_OK;
}

int amoe_gate_reduce_codes(int32_t dtype, const uint8_t* codes, const float* scale, const void* sel, int32_t sel_is_i64,
                           const void* gate, void* y, int64_t T, int32_t k, int32_t D, int64_t* counter_,
                           int64_t counter_add_, void* stream) {
  if (int rc = codes_args_ok(dtype, codes, scale, sel, sel_is_i64, gate, y, T, k, D)) return rc;
  if (!aligned(counter_, 8)) return AMOE_EALIGN;
  if (T == 0) return bump_only(counter_, counter_add_, stream);
  long long* counter = reinterpret_cast<long long*>(counter_);
  const long long counter_add = counter_add_;
  const long long blocks = ((long long)T * (D / 16) + kThreads - 1) / kThreads;
  if (blocks > 0x7fffffffLL) return AMOE_EUNSUPPORTED;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == AMOE_F32) {
    auto kf = &head_reduce_codes_kernel<float>;
    hipLaunchKernelGGL(kf, dim3((unsigned)blocks), dim3(kThreads), 0, st, codes, scale, sel, (int)sel_is_i64,
                       static_cast<const float*>(gate), static_cast<float*>(y), (long long)T, (int)k, (int)D,
                       counter, counter_add);
  } else if (dtype == AMOE_BF16) {
    auto kf = &head_reduce_codes_kernel<uint16_t>;
    hipLaunchKernelGGL(kf, dim3((unsigned)blocks), dim3(kThreads), 0, st, codes, scale, sel, (int)sel_is_i64,
                       static_cast<const uint16_t*>(gate), static_cast<uint16_t*>(y), (long long)T, (int)k, (int)D,
                       counter, counter_add);
  } else {
    auto kf = &head_reduce_codes_kernel<f16_t>;
    hipLaunchKernelGGL(kf, dim3((unsigned)blocks), dim3(kThreads), 0, st, codes, scale, sel, (int)sel_is_i64,
                       static_cast<const f16_t*>(gate), static_cast<f16_t*>(y), (long long)T, (int)k, (int)D,
                       counter, counter_add);
  }
  return launch_rc();
}

int amoe_gate_grad_codes(int32_t dtype, const uint8_t* codes, const float* scale, const void* sel, int32_t sel_is_i64,
                         const void* dy, void* grad_gate, int64_t T, int32_t k, int32_t D, void* stream) {
  if (int rc = codes_args_ok(dtype, codes, scale, sel, sel_is_i64, grad_gate, dy, T, k, D)) return rc;
  if (T == 0) return AMOE_OK;
  const long long blocks = ((long long)T + 4 * kCodeTokens - 1) / (4 * kCodeTokens);
  if (blocks > 0x7fffffffLL) return AMOE_EUNSUPPORTED;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == AMOE_F32) {
    auto kf = &gate_grad_codes_kernel<float>;
    hipLaunchKernelGGL(kf, dim3((unsigned)blocks), dim3(kThreads), 0, st, codes, scale, sel, (int)sel_is_i64,
                       static_cast<const float*>(dy), static_cast<float*>(grad_gate), (long long)T, (int)k, (int)D);
  } else if (dtype == AMOE_BF16) {
    auto kf = &gate_grad_codes_kernel<uint16_t>;
    hipLaunchKernelGGL(kf, dim3((unsigned)blocks), dim3(kThreads), 0, st, codes, scale, sel, (int)sel_is_i64,
                       static_cast<const uint16_t*>(dy), static_cast<uint16_t*>(grad_gate), (long long)T, (int)k, (int)D);
  } else {
    auto kf = &gate_grad_codes_kernel<f16_t>;
    hipLaunchKernelGGL(kf, dim3((unsigned)blocks), dim3(kThreads), 0, st, codes, scale, sel, (int)sel_is_i64,
                       static_cast<const f16_t*>(dy), static_cast<f16_t*>(grad_gate), (long long)T, (int)k, (int)D);
  }
  return launch_rc();
}

int amoe_row_abs_max(int32_t dtype, const void* x, int64_t ldx, int64_t rows, int32_t K, float* abs_max,
                     void* stream) {
  if (dtype != AMOE_F32 && dtype != AMOE_BF16 && dtype != AMOE_F16) return AMOE_EINVAL;
  if (rows < 0 || K < 1 || ldx < K) return AMOE_EINVAL;
  if (rows == 0) return AMOE_OK;
  if (!x || !abs_max) return AMOE_ENULL;
  if (!aligned(x, esize(dtype)) || !aligned(abs_max, 4)) return AMOE_EALIGN;
  const long long blocks = (rows + 3) / 4;
  if (blocks > 0x7fffffffLL) return AMOE_EUNSUPPORTED;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == AMOE_F32) {
    auto kf = &row_abs_max_kernel<float>;
    hipLaunchKernelGGL(kf, dim3((unsigned)blocks), dim3(kThreads), 0, st, static_cast<const float*>(x),
                       (long long)ldx, (long long)rows, (int)K, abs_max);
  } else if (dtype == AMOE_BF16) {
    auto kf = &row_abs_max_kernel<uint16_t>;
    hipLaunchKernelGGL(kf, dim3((unsigned)blocks), dim3(kThreads), 0, st, static_cast<const uint16_t*>(x),
                       (long long)ldx, (long long)rows, (int)K, abs_max);
  } else {
    auto kf = &row_abs_max_kernel<f16_t>;
    hipLaunchKernelGGL(kf, dim3((unsigned)blocks), dim3(kThreads), 0, st, static_cast<const f16_t*>(x),
                       (long long)ldx, (long long)rows, (int)K, abs_max);
  }
  return launch_rc();
}

// Work split of the per-channel reductions over w [E, K, N]: lanes per row (a power of two covering the row's
// 16-byte chunks, at most 64) and K slices (at least eight loads per lane, about four workgroups per CU overall).
struct ColSplit { int width, slices, col_blocks; };
static ColSplit col_split(int dtype, int E, int K, int N) {
  const int CH = 16 / (int)esize(dtype);
  const int chunks = (N + CH - 1) / CH;
  ColSplit c;
  c.width = 64;
  while (c.width / 2 >= chunks) c.width /= 2;
  const int rows_per_block = 4 * (64 / c.width);
  const int most = (K + 8 * rows_per_block - 1) / (8 * rows_per_block);
  const int want = (1024 + E - 1) / E;
  c.slices = most < 1 ? 1 : (most > want ? want : most);
  c.col_blocks = (chunks + 63) / 64;
  return c;
}

int amoe_weight_abs_max_pair(int32_t dtype, const void* w_a, int32_t K_a, int32_t N_a, float* wmax_a,
                             const void* w_b, int32_t K_b, int32_t N_b, float* wmax_b, int32_t E, void* stream) {
  return amoe_layer_tables(dtype, w_a, K_a, N_a, wmax_a, w_b, K_b, N_b, wmax_b, E, AMOE_F32, nullptr, 0, 0, nullptr, 0,
                           nullptr, stream);
}

int amoe_layer_tables(int32_t dtype, const void* w_a, int32_t K_a, int32_t N_a, float* wmax_a, const void* w_b,
                      int32_t K_b, int32_t N_b, float* wmax_b, int32_t E, int32_t ir_dtype, const void* input_range,
                      int32_t ir_cols, int32_t n_up, float* ir_up, int32_t n_dn, float* ir_dn, void* stream) {
  if (dtype != AMOE_F32 && dtype != AMOE_BF16 && dtype != AMOE_F16) return AMOE_EINVAL;
  if (E < 1 || K_a < 1 || N_a < 1 || K_b < 1 || N_b < 1) return AMOE_EINVAL;
  if (!w_a || !w_b || !wmax_a || !wmax_b) return AMOE_ENULL;
  if (!aligned(w_a, esize(dtype)) || !aligned(w_b, esize(dtype)) || !aligned(wmax_a, 4) || !aligned(wmax_b, 4))
    return AMOE_EALIGN;
  if (input_range != nullptr) {
    if (ir_dtype != AMOE_F32 && ir_dtype != AMOE_BF16 && ir_dtype != AMOE_F16) return AMOE_EINVAL;
    if (n_up < 1 || n_dn < 1 || n_up > ir_cols || n_dn > ir_cols || ir_cols > AMOE_MAX_TILES) return AMOE_EINVAL;
    if (!ir_up || !ir_dn) return AMOE_ENULL;
    if (!aligned(input_range, esize(ir_dtype)) || !aligned(ir_up, 4) || !aligned(ir_dn, 4)) return AMOE_EALIGN;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  const long long per_a = (long long)K_a * N_a, per_b = (long long)K_b * N_b;
  const long long per = per_a > per_b ? per_a : per_b;
  int chunks = (int)((per + 32 * kThreads - 1) / (32 * kThreads));
  chunks = chunks < 1 ? 1 : (chunks > 64 ? 64 : chunks);
  const int vec_a = aligned(w_a, 16) && (per_a % 16 == 0), vec_b = aligned(w_b, 16) && (per_b % 16 == 0);
  {
    // one small launch: the zero fill the reduction's atomic maxima start from, and the input-range tables
    const int most = input_range ? E * (n_up > n_dn ? n_up : n_dn) : E;
    const dim3 pg((most + kThreads - 1) / kThreads);
    uint32_t* za = reinterpret_cast<uint32_t*>(wmax_a);
    uint32_t* zb = reinterpret_cast<uint32_t*>(wmax_b);
    if (ir_dtype == AMOE_F32 || input_range == nullptr)
      hipLaunchKernelGGL((&layer_tables_prep_kernel<float>), pg, dim3(kThreads), 0, st, za, zb, (int)E,
                         static_cast<const float*>(input_range), (int)ir_cols, (int)n_up, ir_up, (int)n_dn, ir_dn);
    else if (ir_dtype == AMOE_BF16)
      hipLaunchKernelGGL((&layer_tables_prep_kernel<uint16_t>), pg, dim3(kThreads), 0, st, za, zb, (int)E,
                         static_cast<const uint16_t*>(input_range), (int)ir_cols, (int)n_up, ir_up, (int)n_dn, ir_dn);
    else
      hipLaunchKernelGGL((&layer_tables_prep_kernel<f16_t>), pg, dim3(kThreads), 0, st, za, zb, (int)E,
                         static_cast<const f16_t*>(input_range), (int)ir_cols, (int)n_up, ir_up, (int)n_dn, ir_dn);
  }
  if (int rc = launch_rc()) return rc;
  const dim3 grid(chunks, E, 2);
  if (dtype == AMOE_F32) {
    auto kf = &weight_abs_max_kernel<float>;
    hipLaunchKernelGGL(kf, grid, dim3(kThreads), 0, st, static_cast<const float*>(w_a), per_a, wmax_a, vec_a,
                       static_cast<const float*>(w_b), per_b, wmax_b, vec_b);
  } else if (dtype == AMOE_BF16) {
    auto kf = &weight_abs_max_kernel<uint16_t>;
    hipLaunchKernelGGL(kf, grid, dim3(kThreads), 0, st, static_cast<const uint16_t*>(w_a), per_a, wmax_a, vec_a,
                       static_cast<const uint16_t*>(w_b), per_b, wmax_b, vec_b);
  } else {
    auto kf = &weight_abs_max_kernel<f16_t>;
    hipLaunchKernelGGL(kf, grid, dim3(kThreads), 0, st, static_cast<const f16_t*>(w_a), per_a, wmax_a, vec_a,
                       static_cast<const f16_t*>(w_b), per_b, wmax_b, vec_b);
  }
  return launch_rc();
}

int amoe_weight_abs_max(int32_t dtype, const void* w, int32_t E, int32_t K, int32_t N, int32_t cols, float* wmax,
                        void* stream) {
  if (dtype != AMOE_F32 && dtype != AMOE_BF16 && dtype != AMOE_F16) return AMOE_EINVAL;
  if (E < 1 || K < 1 || N < 1 || (cols != 1 && cols != N)) return AMOE_EINVAL;
  if (!w || !wmax) return AMOE_ENULL;
  if (!aligned(w, esize(dtype)) || !aligned(wmax, 4)) return AMOE_EALIGN;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (cols == 1 || N == 1) {
    const long long per = (long long)K * N;
    int chunks = (int)((per + 32 * kThreads - 1) / (32 * kThreads));
    chunks = chunks < 1 ? 1 : (chunks > 64 ? 64 : chunks);
    const int vec = aligned(w, 16) && (per % 16 == 0);
    hipLaunchKernelGGL(fill_zero_kernel, dim3((E + kThreads - 1) / kThreads), dim3(kThreads), 0, st,
                       reinterpret_cast<uint32_t*>(wmax), (int)E);
    if (int rc = launch_rc()) return rc;
    if (dtype == AMOE_F32) {
      auto kf = &weight_abs_max_kernel<float>;
      hipLaunchKernelGGL(kf, dim3(chunks, E), dim3(kThreads), 0, st, static_cast<const float*>(w), per, wmax, vec,
                         static_cast<const float*>(nullptr), 0LL, static_cast<float*>(nullptr), 0);
    } else if (dtype == AMOE_BF16) {
      auto kf = &weight_abs_max_kernel<uint16_t>;
      hipLaunchKernelGGL(kf, dim3(chunks, E), dim3(kThreads), 0, st, static_cast<const uint16_t*>(w), per, wmax, vec,
                         static_cast<const uint16_t*>(nullptr), 0LL, static_cast<float*>(nullptr), 0);
    } else {
      auto kf = &weight_abs_max_kernel<f16_t>;
      hipLaunchKernelGGL(kf, dim3(chunks, E), dim3(kThreads), 0, st, static_cast<const f16_t*>(w), per, wmax, vec,
                         static_cast<const f16_t*>(nullptr), 0LL, static_cast<float*>(nullptr), 0);
    }
  } else if (dtype == AMOE_BF16) {
    if ((long long)E * N > 0x7fffffffLL) return AMOE_EUNSUPPORTED;
    hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)(((long long)E * N + kThreads - 1) / kThreads)), dim3(kThreads), 0,
                       st, reinterpret_cast<uint32_t*>(wmax), (int)(E * N));
    if (int rc = launch_rc()) return rc;
    const ColSplit cs = col_split(dtype, E, K, N);
    const int width = cs.width;
    const int vec = aligned(w, 16) && (N % (16 / (int)esize(dtype)) == 0);
    dim3 grid(cs.col_blocks, cs.slices, E);
    if (dtype == AMOE_F32) {
      auto kf = &weight_col_abs_max_kernel<float>;
      hipLaunchKernelGGL(kf, grid, dim3(kThreads), 0, st, static_cast<const float*>(w), (int)K, (int)N, width, wmax, vec);
    } else {
      auto kf = &weight_col_abs_max_kernel<uint16_t>;
      hipLaunchKernelGGL(kf, grid, dim3(kThreads), 0, st, static_cast<const uint16_t*>(w), (int)K, (int)N, width, wmax,
                         vec);
    }
  } else {
    if ((long long)E * N > 0x7fffffffLL) return AMOE_EUNSUPPORTED;
    hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)(((long long)E * N + kThreads - 1) / kThreads)), dim3(kThreads), 0,
                       st, reinterpret_cast<uint32_t*>(wmax), (int)(E * N));
    if (int rc = launch_rc()) return rc;
    const ColSplit cs = col_split(dtype, E, K, N);
    const int width = cs.width;
    const int vec = aligned(w, 16) && (N % (16 / (int)esize(dtype)) == 0);
    dim3 grid(cs.col_blocks, cs.slices, E);
    if (dtype == AMOE_F32) {
      auto kf = &weight_col_abs_max_kernel<float>;
      hipLaunchKernelGGL(kf, grid, dim3(kThreads), 0, st, static_cast<const float*>(w), (int)K, (int)N, width, wmax, vec);
    } else {
      auto kf = &weight_col_abs_max_kernel<f16_t>;
      hipLaunchKernelGGL(kf, grid, dim3(kThreads), 0, st, static_cast<const f16_t*>(w), (int)K, (int)N, width, wmax,
                         vec);
    }
  }
  return launch_rc();
}

int amoe_segment_sum(const float* v, const int32_t* offsets, int32_t E, int32_t n_tiles, int32_t out_dtype, void* out,
                     int64_t ldout, int32_t zero_cols, void* stream) {
  if (out_dtype != AMOE_F32 && out_dtype != AMOE_BF16 && out_dtype != AMOE_F16) return AMOE_EINVAL;
  if (E < 1 || n_tiles < 1 || n_tiles > AMOE_MAX_TILES || zero_cols < 0 || zero_cols > AMOE_MAX_TILES ||
      ldout < n_tiles + zero_cols)
    return AMOE_EINVAL;
  if (!v || !offsets || !out) return AMOE_ENULL;
  if (!aligned(v, 4) || !aligned(offsets, 4) || !aligned(out, esize(out_dtype))) return AMOE_EALIGN;
  const dim3 grid(E, n_tiles + zero_cols);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (out_dtype == AMOE_F32) {
    auto kf = &segment_sum_kernel<float>;
    hipLaunchKernelGGL(kf, grid, dim3(kThreads), 0, st, v, offsets, (int)n_tiles, static_cast<float*>(out),
                       (long long)ldout);
  } else if (out_dtype == AMOE_BF16) {
    auto kf = &segment_sum_kernel<uint16_t>;
    hipLaunchKernelGGL(kf, grid, dim3(kThreads), 0, st, v, offsets, (int)n_tiles, static_cast<uint16_t*>(out),
                       (long long)ldout);
  } else {
    auto kf = &segment_sum_kernel<f16_t>;
    hipLaunchKernelGGL(kf, grid, dim3(kThreads), 0, st, v, offsets, (int)n_tiles, static_cast<f16_t*>(out),
                       (long long)ldout);
  }
  return launch_rc();
}

int amoe_expert_std(int32_t dtype, const void* x, int64_t ldx, int32_t K, const int32_t* in_index,
                    const int32_t* offsets, int32_t E, float* out, void* stream) {
  if (dtype != AMOE_F32 && dtype != AMOE_BF16 && dtype != AMOE_F16) return AMOE_EINVAL;
  if (K < 1 || E < 1 || ldx < K) return AMOE_EINVAL;
  if (!x || !in_index || !offsets || !out) return AMOE_ENULL;
  if (!aligned(x, esize(dtype)) || !aligned(in_index, 4) || !aligned(offsets, 4) || !aligned(out, 4))
    return AMOE_EALIGN;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == AMOE_F32) {
    auto kf = &expert_std_kernel<float>;
    hipLaunchKernelGGL(kf, dim3(E), dim3(kThreads), 0, st, static_cast<const float*>(x), (long long)ldx, (int)K,
                       in_index, offsets, out);
  } else if (dtype == AMOE_BF16) {
    auto kf = &expert_std_kernel<uint16_t>;
    hipLaunchKernelGGL(kf, dim3(E), dim3(kThreads), 0, st, static_cast<const uint16_t*>(x), (long long)ldx, (int)K,
                       in_index, offsets, out);
  } else {
    auto kf = &expert_std_kernel<f16_t>;
    hipLaunchKernelGGL(kf, dim3(E), dim3(kThreads), 0, st, static_cast<const f16_t*>(x), (long long)ldx, (int)K,
                       in_index, offsets, out);
  }
  return launch_rc();
}

int amoe_modify_weight(int32_t dtype, const void* w, int32_t E, int32_t K, int32_t N, const float* wmax,
                       int32_t wmax_cols, float n_states, float std_dev, const float* noise, int32_t round_noise,
                       uint64_t noise_seed, const uint64_t* noise_seed_dev, void* out, void* stream) {
  if (dtype != AMOE_F32 && dtype != AMOE_BF16 && dtype != AMOE_F16) return AMOE_EINVAL;
  if (E < 1 || K < 1 || N < 1 || (wmax_cols != 1 && wmax_cols != N)) return AMOE_EINVAL;
  if (!w || !out || !wmax) return AMOE_ENULL;
  if (!aligned(w, esize(dtype)) || !aligned(out, esize(dtype)) || !aligned(wmax, 4) || !aligned(noise, 4) ||
      !aligned(noise_seed_dev, 8))
    return AMOE_EALIGN;
  const int CH = 16 / esize(dtype);
  const long long rows = (long long)E * K;
  const long long blocks = (rows * ((N + CH - 1) / CH) + kThreads - 1) / kThreads;
  if (blocks > 0x7fffffffLL || rows > 0x7fffffffLL) return AMOE_EUNSUPPORTED;
  ModifyParams p{};
  p.w = w; p.out = out; p.wmax = wmax; p.noise = noise; p.rows = rows; p.K = K; p.N = N; p.wmax_cols = wmax_cols;
  p.inv_states = n_states > 0.f ? 1.0f / n_states : 0.f; p.std_dev = std_dev; p.round_noise = round_noise; p.seed = noise_seed;
  p.seed_dev = noise_seed_dev;
  p.vec = aligned(w, 16) && aligned(out, 16) && (N % CH == 0);
  p.cvec = aligned(wmax, 16) && (N % CH == 0);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == AMOE_F32) {
    auto kf = &modify_weight_kernel<float>;
    hipLaunchKernelGGL(kf, dim3((unsigned)blocks), dim3(kThreads), 0, st, p);
  } else if (dtype == AMOE_BF16) {
    auto kf = &modify_weight_kernel<uint16_t>;
    hipLaunchKernelGGL(kf, dim3((unsigned)blocks), dim3(kThreads), 0, st, p);
  } else {
    auto kf = &modify_weight_kernel<f16_t>;
    hipLaunchKernelGGL(kf, dim3((unsigned)blocks), dim3(kThreads), 0, st, p);
  }
  return launch_rc();
}

static int std_slices(long long per_expert) {
  const long long s = (per_expert + 32 * kThreads - 1) / (32 * kThreads);
  return s < 1 ? 1 : (s > kStdMaxSlices ? kStdMaxSlices : (int)s);
}

size_t amoe_weight_std_workspace(int32_t E, int32_t K, int32_t N, int32_t cols) {
  if (E < 1 || K < 1 || N < 1) return 0;
  if (cols == N && N != 1) return (size_t)E * col_split(AMOE_F32, E, K, N).slices * N * 2 * sizeof(double);
  return (size_t)E * std_slices((long long)K * N) * 2 * sizeof(double);
}

int amoe_weight_std(int32_t dtype, const void* w, int32_t E, int32_t K, int32_t N, int32_t cols, float* std_out,
                    void* workspace, size_t workspace_bytes, void* stream) {
  if (dtype != AMOE_F32 && dtype != AMOE_BF16 && dtype != AMOE_F16) return AMOE_EINVAL;
  if (E < 1 || K < 1 || N < 1 || (cols != 1 && cols != N)) return AMOE_EINVAL;
  if (!w || !std_out) return AMOE_ENULL;
  if (!aligned(w, esize(dtype)) || !aligned(std_out, 4) || !aligned(workspace, 8)) return AMOE_EALIGN;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (!workspace) return AMOE_ENULL;
  if (workspace_bytes < amoe_weight_std_workspace(E, K, N, cols)) return AMOE_EWORKSPACE;
  double* partial = static_cast<double*>(workspace);
  if (cols == N && N != 1) {
    if ((long long)E * N > 0x7fffffffLL) return AMOE_EUNSUPPORTED;
    ColSplit cs = col_split(dtype, E, K, N);
    const int most = col_split(AMOE_F32, E, K, N).slices;        // what the workspace was sized for
    if (cs.slices > most) cs.slices = most;
    const int vec = aligned(w, 16) && (N % (16 / (int)esize(dtype)) == 0);
    dim3 grid(cs.col_blocks, cs.slices, E);
    if (dtype == AMOE_F32) {
      auto kf = &weight_col_moments_kernel<float>;
      hipLaunchKernelGGL(kf, grid, dim3(kThreads), 0, st, static_cast<const float*>(w), (int)K, (int)N, cs.width, partial,
                         vec);
    } else if (dtype == AMOE_BF16) {
      auto kf = &weight_col_moments_kernel<uint16_t>;
      hipLaunchKernelGGL(kf, grid, dim3(kThreads), 0, st, static_cast<const uint16_t*>(w), (int)K, (int)N, cs.width,
                         partial, vec);
    } else {
      auto kf = &weight_col_moments_kernel<f16_t>;
      hipLaunchKernelGGL(kf, grid, dim3(kThreads), 0, st, static_cast<const f16_t*>(w), (int)K, (int)N, cs.width,
                         partial, vec);
    }
    if (int rc = launch_rc()) return rc;
    hipLaunchKernelGGL(weight_col_std_finalize_kernel, dim3((unsigned)(((long long)E * N + kThreads - 1) / kThreads)),
                       dim3(kThreads), 0, st, partial, cs.slices, (int)K, (int)N, (int)E, std_out);
    return launch_rc();
  }
  const long long per = (long long)K * N;
  const int slices = std_slices(per);
  const int vec = aligned(w, 16) && (per % 16 == 0);
  if (dtype == AMOE_F32) {
    auto kf = &weight_moments_kernel<float>;
    hipLaunchKernelGGL(kf, dim3(slices, E), dim3(kThreads), 0, st, static_cast<const float*>(w), per, partial, vec);
  } else if (dtype == AMOE_BF16) {
    auto kf = &weight_moments_kernel<uint16_t>;
    hipLaunchKernelGGL(kf, dim3(slices, E), dim3(kThreads), 0, st, static_cast<const uint16_t*>(w), per, partial, vec);
  } else {
    auto kf = &weight_moments_kernel<f16_t>;
    hipLaunchKernelGGL(kf, dim3(slices, E), dim3(kThreads), 0, st, static_cast<const f16_t*>(w), per, partial, vec);
  }
  if (int rc = launch_rc()) return rc;
  hipLaunchKernelGGL(weight_std_finalize_kernel, dim3((E + kThreads - 1) / kThreads), dim3(kThreads), 0, st, partial,
                     slices, per, (int)E, std_out);
  return launch_rc();
}

int amoe_clamp_weights(int32_t dtype, void* w, int32_t E, int32_t K, int32_t N, const float* bound, int32_t cols,
                       void* stream) {
  if (dtype != AMOE_F32 && dtype != AMOE_BF16 && dtype != AMOE_F16) return AMOE_EINVAL;
  if (E < 1 || K < 1 || N < 1 || (cols != 1 && cols != N)) return AMOE_EINVAL;
  if (!w || !bound) return AMOE_ENULL;
  if (!aligned(w, esize(dtype)) || !aligned(bound, 4)) return AMOE_EALIGN;
  const int CH = 16 / esize(dtype);
  const long long rows = (long long)E * K;
  const long long blocks = (rows * ((N + CH - 1) / CH) + kThreads - 1) / kThreads;
  if (blocks > 0x7fffffffLL) return AMOE_EUNSUPPORTED;
  const int vec = aligned(w, 16) && (N % CH == 0);
  const int cvec = aligned(bound, 16) && (N % CH == 0);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == AMOE_F32) {
    auto kf = &clamp_weights_kernel<float>;
    hipLaunchKernelGGL(kf, dim3((unsigned)blocks), dim3(kThreads), 0, st, static_cast<float*>(w), bound, rows, (int)K,
                       (int)N, (int)cols, vec, cvec);
  } else if (dtype == AMOE_BF16) {
    auto kf = &clamp_weights_kernel<uint16_t>;
    hipLaunchKernelGGL(kf, dim3((unsigned)blocks), dim3(kThreads), 0, st, static_cast<uint16_t*>(w), bound, rows,
                       (int)K, (int)N, (int)cols, vec, cvec);
  } else {
    auto kf = &clamp_weights_kernel<f16_t>;
    hipLaunchKernelGGL(kf, dim3((unsigned)blocks), dim3(kThreads), 0, st, static_cast<f16_t*>(w), bound, rows,
                       (int)K, (int)N, (int)cols, vec, cvec);
  }
  return launch_rc();
}

static long long select_blocks(long long T) { return (T + 4 * kSelRowsPerWave - 1) / (4 * kSelRowsPerWave); }

size_t amoe_select_workspace(int64_t T, int32_t E) {
  if (T < 1 || E < 1) return 0;
  const long long blocks = select_blocks(T);
  return (size_t)(blocks + (blocks + kSelSumChunk - 1) / kSelSumChunk) * E * sizeof(float);
}

int amoe_select_fwd(int32_t dtype, const void* logits, int64_t T, int32_t E, int32_t k, void* sel_val, int64_t* sel_idx,
                    float* reg, float* reg_c, void* workspace, size_t workspace_bytes, void* stream) {
  if (dtype != AMOE_F32 && dtype != AMOE_BF16 && dtype != AMOE_F16) return AMOE_EINVAL;
  if (T < 0 || E < 1 || k < 1 || k > E) return AMOE_EINVAL;
  if (E > 64 * kSelPerLane) return AMOE_EUNSUPPORTED;
  if (T == 0) return AMOE_OK;
  if (!logits || !sel_val || !sel_idx) return AMOE_ENULL;
  if ((reg != nullptr) != (reg_c != nullptr)) return AMOE_EINVAL;
  if (!aligned(logits, esize(dtype)) || !aligned(sel_val, esize(dtype)) || !aligned(sel_idx, 8) || !aligned(reg, 4) ||
      !aligned(reg_c, 4) || !aligned(workspace, 4))
    return AMOE_EALIGN;
  const long long blocks = select_blocks(T);
  if (blocks > 0x7fffffffLL) return AMOE_EUNSUPPORTED;
  float* partial = nullptr;
  if (reg != nullptr) {
    if (!workspace) return AMOE_ENULL;
    if (workspace_bytes < amoe_select_workspace(T, E)) return AMOE_EWORKSPACE;
    partial = static_cast<float*>(workspace);
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
#define AMOE_SELECT_FWD(PER)                                                                                           \
  do {                                                                                                                 \
    if (dtype == AMOE_F32) {                                                                                           \
      auto kf = &select_fwd_kernel<float, PER>;                                                                        \
      hipLaunchKernelGGL(kf, dim3((unsigned)blocks), dim3(kThreads), 0, st, static_cast<const float*>(logits),         \
                         (long long)T, (int)E, (int)k, static_cast<float*>(sel_val), sel_idx, partial);                \
    } else if (dtype == AMOE_BF16) {                                                                                   \
      auto kf = &select_fwd_kernel<uint16_t, PER>;                                                                     \
      hipLaunchKernelGGL(kf, dim3((unsigned)blocks), dim3(kThreads), 0, st, static_cast<const uint16_t*>(logits),      \
                         (long long)T, (int)E, (int)k, static_cast<uint16_t*>(sel_val), sel_idx, partial);             \
    } else {                                                                                                           \
      auto kf = &select_fwd_kernel<f16_t, PER>;                                                                        \
      hipLaunchKernelGGL(kf, dim3((unsigned)blocks), dim3(kThreads), 0, st, static_cast<const f16_t*>(logits),         \
                         (long long)T, (int)E, (int)k, static_cast<f16_t*>(sel_val), sel_idx, partial);                \
    }                                                                                                                  \
  } while (0)
  if (E <= 64) AMOE_SELECT_FWD(1);
  else if (E <= 128) AMOE_SELECT_FWD(2);
  else if (E <= 256) AMOE_SELECT_FWD(4);
  else AMOE_SELECT_FWD(8);
#undef AMOE_SELECT_FWD
  if (int rc = launch_rc()) return rc;
  if (reg != nullptr) {
    const int groups = (int)((blocks + kSelSumChunk - 1) / kSelSumChunk);
    float* level2 = partial + blocks * E;
    hipLaunchKernelGGL(select_usage_sum_kernel, dim3(groups), dim3(kThreads), 0, st, partial, (int)blocks, (int)E, level2);
    if (int rc = launch_rc()) return rc;
    hipLaunchKernelGGL(select_reg_kernel, dim3(1), dim3(kThreads), 0, st, level2, groups, (int)E, (long long)T, reg,
                       reg_c);
    return launch_rc();
  }
  return AMOE_OK;
}

int amoe_select_bwd(int32_t dtype, const void* logits, int64_t T, int32_t E, int32_t k, const int64_t* sel_idx,
                    const void* grad_val, const float* reg_c, const float* grad_reg, void* grad_logits, void* stream) {
  if (dtype != AMOE_F32 && dtype != AMOE_BF16 && dtype != AMOE_F16) return AMOE_EINVAL;
  if (T < 0 || E < 1 || k < 1 || k > E) return AMOE_EINVAL;
  if (E > 64 * kSelPerLane) return AMOE_EUNSUPPORTED;
  if (T == 0) return AMOE_OK;
  if (!logits || !grad_logits || (grad_val && !sel_idx)) return AMOE_ENULL;
  if ((reg_c != nullptr) != (grad_reg != nullptr)) return AMOE_EINVAL;
  if (!aligned(logits, esize(dtype)) || !aligned(grad_logits, esize(dtype)) || !aligned(grad_val, esize(dtype)) ||
      !aligned(sel_idx, 8) || !aligned(reg_c, 4) || !aligned(grad_reg, 4))
    return AMOE_EALIGN;
  const long long blocks = (T + 3) / 4;
  if (blocks > 0x7fffffffLL) return AMOE_EUNSUPPORTED;
  hipStream_t st = static_cast<hipStream_t>(stream);
#define AMOE_SELECT_BWD(PER)                                                                                           \
  do {                                                                                                                 \
    if (dtype == AMOE_F32) {                                                                                           \
      auto kf = &select_bwd_kernel<float, PER>;                                                                        \
      hipLaunchKernelGGL(kf, dim3((unsigned)blocks), dim3(kThreads), 0, st, static_cast<const float*>(logits),         \
                         (long long)T, (int)E, (int)k, sel_idx, static_cast<const float*>(grad_val), reg_c, grad_reg,  \
                         static_cast<float*>(grad_logits));                                                            \
    } else if (dtype == AMOE_BF16) {                                                                                   \
      auto kf = &select_bwd_kernel<uint16_t, PER>;                                                                     \
      hipLaunchKernelGGL(kf, dim3((unsigned)blocks), dim3(kThreads), 0, st, static_cast<const uint16_t*>(logits),      \
                         (long long)T, (int)E, (int)k, sel_idx, static_cast<const uint16_t*>(grad_val), reg_c,         \
                         grad_reg, static_cast<uint16_t*>(grad_logits));                                               \
    } else {                                                                                                           \
      auto kf = &select_bwd_kernel<f16_t, PER>;                                                                        \
      hipLaunchKernelGGL(kf, dim3((unsigned)blocks), dim3(kThreads), 0, st, static_cast<const f16_t*>(logits),         \
                         (long long)T, (int)E, (int)k, sel_idx, static_cast<const f16_t*>(grad_val), reg_c,            \
                         grad_reg, static_cast<f16_t*>(grad_logits));                                                  \
    }                                                                                                                  \
  } while (0)
  if (E <= 64) AMOE_SELECT_BWD(1);
  else if (E <= 128) AMOE_SELECT_BWD(2);
  else if (E <= 256) AMOE_SELECT_BWD(4);
  else AMOE_SELECT_BWD(8);
#undef AMOE_SELECT_BWD
  return launch_rc();
}

}  // extern "C"
