/*
 * cats_gemv.h -- C ABI of the gfx950 CATS sparse-MLP decode kernels.
 *
 * Every entry point takes plain device pointers, sizes and a HIP stream and returns a
 * cats_status_t.  Nothing here allocates, frees or synchronises (cats_read_count is the one
 * documented exception: it has to hand a device counter back to the host, and its first call
 * allocates one pinned host word for that).  A launch failure is reported as CATS_ERR_LAUNCH
 * from the status of that launch alone; errors left behind by the caller's earlier HIP calls are
 * neither returned nor cleared.  All launches go
 * to the stream that is passed in.  The entry points are what a `TORCH_LIBRARY(flash_gemv, m)`
 * shim, a ctypes loader or any other FFI binds; each one names the reference interface it
 * stands in for (paths relative to the CATS tree).
 *
 * Conventions
 *   B      rows of the activation matrix (batch * seq, decode => seq == 1); 1 <= B <= CATS_MAX_BATCH
 *   H      hidden size, I intermediate size
 *   dtype  cats_dtype_t; x, weights and dtype-typed outputs all share it
 *   x        (B, H)  row-major
 *   wgate    (I, H)  row-major  (nn.Linear layout: one row per neuron)
 *   wup      (I, H)  row-major
 *   wdown_t  (I, H)  row-major, "neuron-major": row j is column j of the HF down_proj.weight
 *   wdown    (H, I)  row-major  (HF nn.Linear layout)
 *   flag     (B, I)  one byte per entry, 0 or 1 (torch.bool storage)
 *   Rows must be 16-byte aligned: H * sizeof(dtype) % 16 == 0 and all base pointers 16-byte
 *   aligned (I * sizeof(dtype) % 16 == 0 as well where I is a row length: wdown, a, z).
 *
 * Activation and mask rule (experiments/models/sparse_silu/ugly_utils.py:895-899,
 * flash_gemv/flash_gemv/__init__.py:41,46):
 *   g  = round_dtype(sum_k x[b,k] * wgate[j,k])        fp32 accumulation
 *   a  = round_dtype(g / (1 + exp(-g)))                SiLU evaluated in fp32
 *   active(b,j)  <=>  |a| > round_dtype(threshold)     strict, compared on the stored value
 *   z  = active ? round_dtype(a * round_dtype(sum_k x[b,k] * wup[j,k])) : 0
 *   y  = round_dtype(sum_j z[b,j] * wdown_t[j,:])      fp32 accumulation
 * A weight row of wup / wdown_t is fetched only if some row b of the batch has it active.
 */
#ifndef CATS_GEMV_H
#define CATS_GEMV_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum { CATS_F16 = 0, CATS_BF16 = 1, CATS_F32 = 2 } cats_dtype_t;

typedef enum {
  CATS_OK = 0,
  CATS_ERR_DTYPE = 1,      /* dtype is not a cats_dtype_t */
  CATS_ERR_SHAPE = 2,      /* non-positive or unsupported H / I */
  CATS_ERR_ALIGN = 3,      /* a pointer or row pitch is not 16-byte aligned */
  CATS_ERR_BATCH = 4,      /* B outside 1..CATS_MAX_BATCH */
  CATS_ERR_NULL = 5,       /* a required pointer is NULL */
  CATS_ERR_WORKSPACE = 6,  /* workspace missing or smaller than cats_workspace_bytes() */
  CATS_ERR_LAUNCH = 7,     /* the HIP runtime refused a launch; hipGetLastError() has details */
  CATS_ERR_SCRATCH = 8     /* cats_mlp_noalloc: the call does not fit the library's built-in scratch */
} cats_status_t;

#define CATS_MAX_BATCH 16  /* 1..8 rows are one pass over the weights.  9..16 rows: the whole-MLP entry points (cats_mlp, the
                            * layer-tail calls, cats_up_down, cats_mlp_rowmajor_down), cats_gate_flag, cats_gate_up and cats_up_flag
                            * (16-bit types, rows of 2048 or 4096 elements) and cats_down_flag (16-bit types) still read
                            * every matrix once; every other case is two passes of at most eight rows */

/* Library identification / error text.  No reference counterpart (the reference printf()s and exit()s:
 * flash_gemv/csrc/cuda/fuse_gemv_cmp_cuda.cu:25-33,2397-2400). */
int cats_version(void);
const char* cats_status_string(int status);

/* Workspace: scratch for the per-workgroup partial sums, the mask bytes, the fp32 intermediate z and the
 * gate activations of the list-building call.  Replaces the per-call cudaMalloc/cudaFree pairs of the reference
 * (fuse_gemv_cmp_cuda.cu:2351-2354,2402-2403).  The caller allocates cats_workspace_bytes() once (256-byte
 * aligned), runs cats_workspace_init() once (it zero-fills with a kernel), and then passes the same buffer to
 * every call; no call relies on what an earlier call left in it (the counter words at its head are all zero
 * between calls: a call that uses them puts them back).  The size and the carving depend on (H, I)
 * only (B is checked; every region holds the 8 rows of one pass over the weights, and a call with 9..16 rows
 * reuses them pass by pass), so one workspace serves every batch size of one layer shape; for another (H, I)
 * use another workspace or initialise again.  One workspace serves one stream at a time. */
size_t cats_workspace_bytes(int B, int H, int I);
int cats_workspace_init(void* ws, size_t ws_bytes, void* stream);

/* Fused gate GEMV + SiLU + |a| > t.  Writes a (B,I) in dtype and/or flag (B,I) bytes; either may be NULL.
 * Replaces fuse_gemv_flag_local / fuse_gemv_flag / fuse_gemv_flag_batch
 * (flash_gemv/flash_gemv/flash_gemv.py:6-7,18-22; fuse_gemv_cmp_cuda.cu:1292-1486,2083-2117). */
int cats_gate_flag(const void* x, const void* wgate, void* a_out, uint8_t* flag_out,
                   int B, int H, int I, int dtype, float threshold, void* stream);

/* Same gate pass, B == 1, that also emits the compact active set: idx_out[0..count) ascending neuron
 * indices (int64), vals_out[0..count) the matching activations in dtype, *count_out (device int32) the
 * count.  Two launches: the gate pass (activations and mask bytes into the workspace), then a small kernel that
 * turns the mask bytes into the list with popcounts, wave prefix sums and bit expansion.
 * Replaces fuse_gemv_cmp (flash_gemv.py:3-4; fuse_gemv_cmp_cuda.cu:43-88,1962-1977), whose list is in
 * atomic arrival order and whose count lives in a process-global managed int. */
int cats_gate_compact(const void* x, const void* wgate, void* vals_out, int64_t* idx_out, int32_t* count_out,
                      int H, int I, int dtype, float threshold, void* ws, size_t ws_bytes, void* stream);

/* Blocking helper for the call above: copies *count_dev to pinned host memory behind the work already on the
 * stream, waits for the stream once and returns the value (or -1 on error). */
int cats_read_count(const int32_t* count_dev, void* stream);

/* Sparse up projection over a flag array.  out[b,j] = flag[b,j] ? a[b,j] * (x[b,:] . wup[j,:]) : 0.
 * Row j of wup is fetched iff any flag[b,j] is set.  a and out are (B,I); out may alias a (in place).
 * out_is_f32 != 0 writes fp32 instead of dtype.
 * Replaces fuse_flag_gemv_local (flash_gemv.py:24-25; fuse_gemv_cmp_cuda.cu:1507-1722,2123-2156) and the
 * Triton gather_gemv_elemul_flag_3d (flash_gemv/flash_gemv/kernels.py:69-254). */
int cats_up_flag(const void* x, const void* wup, const void* a, const uint8_t* flag, void* out, int out_is_f32,
                 int B, int H, int I, int dtype, void* stream);

/* Sparse down projection over neuron-major weights.  y[b,:] += sum_{j: any flag[.,j]} z[b,j] * wdown_t[j,:].
 * z is (B,I) in dtype.  Two output modes:
 *   y_f32 != NULL : fp32 atomics straight into the caller's (B,H) buffer, which the caller zeroed (or wants
 *                   accumulated into) -- atomic_gemv (flash_gemv.py:27-28; fuse_gemv_cmp_cuda.cu:1724-1783,2162-2194);
 *   y_out != NULL : (B,H) in dtype, zero-initialised and rounded inside the call -- the Triton
 *                   gather_transposed_gemv_flag_3d (kernels.py:324-462).
 * Exactly one of y_f32 / y_out must be non-NULL.  Needs a workspace. */
int cats_down_flag(const void* z, const void* wdown_t, const uint8_t* flag, float* y_f32, void* y_out,
                   int B, int H, int I, int dtype, void* ws, size_t ws_bytes, void* stream);

/* Index-list ("DejaVu") up projection: out[b, m] = scale[m] * act(x[b,:] . w[idx[m],:] + bias[idx[m]]) for the M entries
 * of idx (int64 weight-row numbers, any order, duplicates allowed; an entry outside [0, Z) yields 0).  Only the listed
 * rows of w (Z, H) are read.  bias (Z,) and scale (M,) are optional, in dtype; activation 0 = identity, 1 = relu,
 * 2 = squared relu, 3 = swish; fp32 throughout with one rounding at the store.  out (B, M) in dtype.
 * Replaces gather_gemv (flash_gemv/flash_gemv/kernels.py:484-695) and, with scale = the compact gate activations,
 * gather_gemv_elemul_indirect_index_2d (kernels.py:1112-1150, 1236-1274). */
int cats_up_index(const void* x, const void* w, const int64_t* idx, int M, const void* bias, const void* scale, int activation,
                  void* out, int B, int H, int Z, int dtype, void* stream);

/* Index-list down projection: y[b,:] = sum over m of z[b, m] * wdown_t[idx[m], :] (+ bias), z (B, M) aligned with the list,
 * wdown_t (Z, H) neuron-major, bias (H,) optional.  Duplicate entries add up (as the reference's atomics do), entries
 * outside [0, Z) contribute nothing.  y_out (B, H) in dtype, fp32 accumulation in a fixed order.  Needs a workspace.
 * Replaces gather_transposed_gemv (kernels.py:753-1094) and gather_transposed_gemv_indirect_index_2d
 * (kernels.py:1204-1234, 1276-1325). */
int cats_down_index(const void* z, const void* wdown_t, const int64_t* idx, int M, const void* bias, void* y_out,
                    int B, int H, int Z, int dtype, void* ws, size_t ws_bytes, void* stream);

/* Gate + sparse up in one pass: out[b,j] = active ? round(a * up) : 0 in dtype, flag_out optional.
 * Replaces fuse_gemv_flag_gemv (flash_gemv.py:9-10; fuse_gemv_cmp_cuda.cu:715-784,2006-2022). */
int cats_gate_up(const void* x, const void* wgate, const void* wup, void* out, uint8_t* flag_out,
                 int B, int H, int I, int dtype, float threshold, void* stream);

/* Whole CATS MLP with neuron-major down weights.  1..2 rows: one streaming kernel in which every workgroup takes its
 * neurons through gate, up and down; more rows: gate+up kernel, then sparse down kernel.
 *   y_out != NULL : (B,H) in dtype.  The workgroups leave fp32 partial sums and a second launch adds them in a fixed
 *                   order: the result is bitwise reproducible from run to run.
 *   y_f32 != NULL : fp32 accumulate into the caller's (B,H), which the caller has zeroed (or which holds what the result
 *                   is to be added to) -- the contract of the reference ops named below.  At 1..2 rows this is ONE launch:
 *                   the streaming kernel adds its sums into y_f32 with fp32 atomics (the order, and so the last bits,
 *                   vary from run to run).
 * flag_out (B,I) optional.  count_out (device int32, optional) receives the number of neurons active in any row of the
 * batch (the number of neurons fetched; where 9..16 rows run as two passes one small kernel counts the union of the
 * flags afterwards).  With y_f32 and count_out at 1..2 rows a second, tiny launch totals the count.
 * Replaces flag_gemv_gemv_atomic, fuse_gemv_gemv_gemv, fuse_gemv_flag_gemv_gemv (flash_gemv.py:12-16,30-31;
 * fuse_gemv_cmp_cuda.cu:786-1244,2196-2253) and the composite gemv_gemv_triton / flag_gemv_gemv_triton
 * (flash_gemv/flash_gemv/__init__.py:38-48). */
int cats_mlp(const void* x, const void* wgate, const void* wup, const void* wdown_t, void* y_out, float* y_f32,
             uint8_t* flag_out, int32_t* count_out, int B, int H, int I, int dtype, float threshold,
             void* ws, size_t ws_bytes, void* stream);

/* Sparse up + sparse down given the gate activations:  flags = |a| > t per row,  z = a * (x . wup[j]) for active j,
 * y = sum over active j of z[j] * wdown_t[j,:].  Two launches; the flags are derived inside the up kernel and
 * reach the down kernel as mask bytes in the workspace.  a (B,I) in dtype; y_out (B,H) in dtype.
 * Replaces the composite gemv_gemv_triton(x, x_1, Wup, Wdownt, threshold) (flash_gemv/flash_gemv/__init__.py:45-48),
 * the call the reference's sp_method 2 branch makes (experiments/models/sparse_silu/ugly_utils.py:887-894). */
int cats_up_down(const void* x, const void* a, const void* wup, const void* wdown_t, void* y_out, int B, int H, int I,
                 int dtype, float threshold, void* ws, size_t ws_bytes, void* stream);

/* The tail of a decoder layer in two launches:  out = h + MLP(norm_weight * rms_norm(h)).
 * The RMS norm (fp32 mean of squares, rsqrt(mean + eps), result rounded to dtype, then multiplied by norm_weight in
 * dtype -- the HF LlamaRMSNorm / MistralRMSNorm order) is applied while the gate+up kernel stages h in LDS; the
 * residual add happens where the down kernel writes its output (MLP result rounded to dtype first, then added).
 * h, out (B,H) in dtype; out may alias h.  norm_weight (H) in dtype.  Needs B*H*sizeof(dtype) <= 128 KiB.
 * Replaces the three module calls  residual = h; h = post_attention_layernorm(h); h = residual + mlp(h)
 * of the reference's decoder layer (experiments/models/sparse_silu/ugly_utils.py:1036-1057) for batch*seq <= 16. */
int cats_mlp_norm_residual(const void* h, const void* norm_weight, float eps, const void* wgate, const void* wup,
                           const void* wdown_t, void* out, int B, int H, int I, int dtype, float threshold,
                           void* ws, size_t ws_bytes, void* stream);

/* cats_mlp_norm_residual that also writes what the next consumer of the hidden state starts with:
 *   out = h + MLP(norm_weight * rms_norm(h, eps));   next_out = next_norm_weight * rms_norm(out, next_eps).
 * In a decoder stack next_norm_weight is the input_layernorm of the following layer (the final norm after the last
 * layer), so every layer boundary loses its stand-alone norm.  Same two launches: the launch that finishes `out` also
 * leaves each workgroup's finished columns and their sum of squares in the workspace, and per batch row the last of its
 * workgroups to arrive (counters in the workspace head, put back to zero by the call) adds the sums in a fixed order
 * and writes that row of next_out -- bitwise reproducible, +3.4 us on the Llama-2-7B layer.  next_out (B,H) in dtype
 * must not alias out or h.
 * Needs H % 32 == 0 on top of the limits of cats_mlp_norm_residual.
 * Replaces, for batch*seq <= 16, the module calls  residual = h; h = post_attention_layernorm(h); h = residual + mlp(h)
 * of one decoder layer and  hidden_states = self.input_layernorm(hidden_states)  of the next
 * (experiments/models/sparse_silu/ugly_utils.py:1016-1057). */
int cats_mlp_norm_residual_norm(const void* h, const void* norm_weight, float eps, const void* wgate, const void* wup,
                                const void* wdown_t, void* out, const void* next_norm_weight, float next_eps, void* next_out,
                                int B, int H, int I, int dtype, float threshold, void* ws, size_t ws_bytes, void* stream);

/* Whole CATS MLP with the HF (H,I) down weight: gate+up, then a dense row-major GEMV over the zero-filled
 * intermediate (all of wdown is read, as in the reference).
 * Replaces flag_gemv_gemv and flag_gemv_gemv_inner{,_fp32,_bf16} (flash_gemv.py:33-43;
 * fuse_gemv_cmp_cuda.cu:2255-2560). */
int cats_mlp_rowmajor_down(const void* x, const void* wgate, const void* wup, const void* wdown, void* y_out,
                           int B, int H, int I, int dtype, float threshold, void* ws, size_t ws_bytes, void* stream);

/* cats_mlp(y_out mode) for callers that cannot allocate device memory or carry a workspace -- code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference (whose ops
 * cudaMalloc per call).  The scratch of the single-pass kernels (per-workgroup partial sums and counts, 8 MiB + 4 KiB)
 * lives in a device array inside the library, one copy per GPU, held until the process ends; nothing is allocated or
 * freed by the call.  Limits: 1..2 rows, B * H <= 8192, rows of at most 1024 (one row) or 2048 (two rows) 16-byte
 * vectors (fp32 at one row: H <= 4096); anything else returns CATS_ERR_SCRATCH.  Same kernels and summation order as cats_mlp, so the same bits.  All calls on one GPU share
 * that GPU's array: calls that overlap in time on one GPU (different streams, or a graph replay next to an eager
 * call) race; calls on one stream, or otherwise ordered, are fine.  Nothing in the array has to be cleared between
 * calls (every call overwrites what it reads). */
int cats_mlp_noalloc(const void* x, const void* wgate, const void* wup, const void* wdown_t, void* y_out,
                     int B, int H, int I, int dtype, float threshold, void* stream);

/* One launch of cats_mlp(y_out mode) alone, for per-kernel timing and profiling: stage 1 = the streaming launch (gate, up
 * and, for 1..2 rows, down into per-workgroup partial sums), stage 2 = the launch that finishes y from what stage 1 left in
 * the workspace.  Calling stage 1 then stage 2 with the same arguments is cats_mlp.  Not in the reference. */
int cats_mlp_stage(int stage, const void* x, const void* wgate, const void* wup, const void* wdown_t, void* y_out,
                   int B, int H, int I, int dtype, float threshold, void* ws, size_t ws_bytes, void* stream);

/* Measurement aid, not in the reference: one kernel that reads `bytes` (a multiple of 16, 16-byte aligned) from src
 * with the streaming 128-bit loads the weight rows are read with, and writes nothing (sink, 4 bytes of device memory,
 * is stored to only if the XOR of everything read equals one fixed word).  Timing it over a buffer larger than the
 * 256 MB memory-side cache gives the read-stream bandwidth this GPU actually reaches, the practical ceiling next
 * to the published HBM peak. */
int cats_probe_read(const void* src, size_t bytes, uint32_t* sink, void* stream);

/* Launch-shape knobs for experiments; 0 keeps the built-in choice.  gate_variant N > 0 caps the gate / up kernel at N
 * resident workgroups per CU (N < 0 keeps 3..16 rows off the matrix-core kernels, gate / up and down); down_groups sets the
 * neuron groups of the sparse down kernels, down_block the workgroup size of the wave-per-row-pair one -- and keeps 3..16 rows
 * on that kernel, off the matrix-core one; path 1 keeps the whole-MLP entry points on the separate gate+up
 * and sparse-down kernels for every batch size (by default 1..2 rows take the single-pass kernel).  Every setting computes
 * the same function.  Process-global and not synchronised: set it before other threads call in.  Not in the reference. */
int cats_set_tuning(int gate_variant, int down_groups, int down_block, int path);

#ifdef __cplusplus
}
#endif
#endif /* CATS_GEMV_H */
