/*
 * mam_hip.h -- C ABI of libmam_hip.so: the Multiply-And-Max/min (MAM) fully-connected
 * hot path as hand-written HIP kernels for gfx950 (MI355X, wave64).
 *
 * Plain pointers and sizes only; every pointer is DEVICE memory of the current HIP
 * device unless stated otherwise; `stream` is a hipStream_t passed as void* (NULL = the
 * legacy default stream).  All calls are asynchronous on `stream`, never synchronise the
 * host, and allocate nothing: scratch memory is brought in by the caller as `workspace`.
 * Every function returns MAM_OK (0) or a negative MAM_ERR_* code; mam_error_string()
 * names a code and mam_last_error() gives the detail of this thread's last failure.
 *
 * Notation: N = batch rows, K = in_features, M = out_features.
 *   x        (N, K) fp32, row stride ldx (>= K)
 *   w        layout MAM_W_KM: (K, M) fp32, row stride ldw (>= M) -- operand `b` of the
 *            reference operators; layout MAM_W_MK: (M, K) fp32, row stride ldw (>= K) --
 *            the nn.Module's `weight` (out, in), so the module needs no transposed copy.
 *   c        (N, M) fp32 contiguous;   argmax/argmin (N, M) int32 contiguous.
 *
 * Each entry point names the interface of SSIGPRO/mamtorch 1.5.2 that it stands behind.
 */
#ifndef MAM_HIP_H
#define MAM_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MAM_OK 0
#define MAM_ERR_INVALID_ARGUMENT (-1) /* null pointer, negative size, bad enum          */
#define MAM_ERR_UNSUPPORTED (-2)      /* size outside what the kernels cover            */
#define MAM_ERR_WORKSPACE (-3)        /* workspace missing or smaller than required     */
#define MAM_ERR_LAUNCH (-4)           /* HIP reported an error at launch                */

#define MAM_W_KM 0
#define MAM_W_MK 1

#define MAM_PRUNE_MAGNITUDE 0    /* score = |w|                                  */
#define MAM_PRUNE_WEIGHT_TIMES 1 /* score = |w * aux|, aux (M,K) fp32 (e.g. w.grad) */
#define MAM_PRUNE_COUNT 2        /* score = aux (+ aux2), (M,K) int32 selection counts */

#define MAM_COUNT_REFERENCE 0 /* per call: +1 per (m,k) picked as max by >=1 row, +1 if picked as
                                 min by >=1 row, both into max_count (the module's literal rule) */
#define MAM_COUNT_HITS 1      /* true hit counts: max_count += #argmax hits, min_count += #argmin */
#define MAM_COUNT_FLAGS 2     /* per call: max_count += 1 where >=1 row picked the cell as max, min_count
                                 likewise for min (the retired convolution modules' literal rule)        */

/* Run-time switches for mam_set_option().  Their initial values come from the environment variables of
 * the same names, read once when the library is loaded: MAM_FORWARD_TILING = auto | wide | 0 | 1 | 2 | 3,
 * MAM_BACKWARD_FORK = auto | -1 | 0 | 1, MAM_BACKWARD_ONE_LAUNCH = auto | 0 (off) | 1 (auto) | 2 (on),
 * MAM_BACKWARD_EXACT = 0 | 1.  A value outside an
 * option's range is refused by mam_set_option() and ignored (with the default kept) in the environment. */
#define MAM_OPT_FORWARD_TILING 0 /* which dense forward tiling serves a call                      */
#define MAM_OPT_BACKWARD_FORK 1  /* x_grad on the library's second stream beside w_grad           */
#define MAM_OPT_BACKWARD_ONE_LAUNCH 2 /* both gradients in one launch where the shape allows it    */
#define MAM_OPT_BACKWARD_EXACT 3 /* w_grad accumulated in 64-bit fixed-point cells (exact sums)    */
#define MAM_OPT_COUNT_ 4
#define MAM_FORWARD_TILING_AUTO 0 /* wave-uniform-rows tiling where the layout allows it           */
#define MAM_FORWARD_TILING_WIDE 1 /* every call on the general 64 x 128 tiling                     */
#define MAM_FORWARD_TILING_GROUPS16 2 /* as AUTO, but indices recorded per 16 products at every K   */
#define MAM_FORWARD_TILING_FUSED_MERGE 3 /* as AUTO, but a K-split call merges inside the forward launch: the
                                            last of a tile's workgroups to finish combines and resolves   */
#define MAM_BACKWARD_FORK_AUTO (-1) /* where it pays: from 2^23 outputs on with at least 1024 neurons (dense),
                                       2^22 outputs (CSR); under stream capture from 2^16 outputs       */
#define MAM_BACKWARD_FORK_OFF 0
#define MAM_BACKWARD_FORK_ON 1
#define MAM_BACKWARD_ONE_LAUNCH_OFF 0
#define MAM_BACKWARD_ONE_LAUNCH_AUTO 1 /* small calls only (<= 2^16 outputs), where the launches are the cost */
#define MAM_BACKWARD_ONE_LAUNCH_ON 2   /* wherever the shape allows it: (M,K) weights, 16-byte aligned operands,
                                          batch below 2 x CUs, K <= 4096 */
#define MAM_BACKWARD_EXACT_OFF 0 /* w_grad in fp32 cells: each sum within the rounding floor of its order    */
#define MAM_BACKWARD_EXACT_ON 1  /* w_grad = the exact sum of its fp32 terms rounded once (the w_grad kernel
                                    takes 45 instead of 17 us at 256 x 4096 x 4096, 1.7 to 1.8 times as long at
                                    batch 12608); (M,K) weights with hand-over only                           */

/* Library version (major*10000 + minor*100 + patch). */
int mam_version(void);
const char *mam_error_string(int code);
const char *mam_last_error(void);

/*
 * Per-device set-up for the CURRENT HIP device: raises the LDS limit of the kernels that use more than
 * 64 KiB, creates the library's second stream (default priority) and its two events, and takes the
 * address of the library's file-scope scratch array.  Idempotent and thread-safe.  Every entry point
 * does the same on its first call on a device; a caller that records HIP graphs calls mam_init() (or
 * any entry point once, eagerly) on that device BEFORE capturing, because streams and events must not be
 * created inside a capture.  No counterpart in the reference, which has no per-device state.
 */
int mam_init(void);

/* Compute units and maximum engine clock (kHz) of the current device, as the library's launch heuristics
 * see them.  Either pointer may be NULL.  No counterpart in the reference. */
int mam_device_info(int *compute_units, int *max_clock_khz);

/* Sets a MAM_OPT_* switch for the whole process (all devices, all threads).  The reference has no
 * run-time switches; these exist for tests and comparisons. */
int mam_set_option(int option, int value);

/*
 * Exact MAM forward with indices.
 *   c[n,m]      = (max_k x[n,k]*w[k,m] + min_k x[n,k]*w[k,m]) (+ bias[m] if bias != NULL)
 *   argmax[n,m] = lowest k attaining the max; argmin[n,m] = lowest k attaining the min.
 * Replaces mamtorch_kernel_v1::fullyconnected_cuda
 * (mamtorch/kernel/v1/csrc/cuda/fullyconnected.cu:177-291, kernel :33-175) and serves
 * mamtorch_kernel_v4::fullyconnected_cuda (mamtorch/kernel/v4/csrc/cuda/fullyconnected.cu:41-149)
 * with zero approximation error; the bias add is nn/v4/fullyconnected.py:197-198.
 * NaN products are ignored, as by the reference kernel's ordered comparisons.
 * `workspace` may be NULL when mam_fc_forward_workspace() returns 0.
 * `w_sel` (optional, may be NULL): (2, N, M) fp32 contiguous; receives w[argmax[n,m], m] in plane 0 and
 * w[argmin[n,m], m] in plane 1.  Handing it to mam_fc_backward spares that call 2*N*M random reads of w.
 * `x_sel` (optional, may be NULL): the same for the inputs, x[n, argmax[n,m]] and x[n, argmin[n,m]]; it
 * spares mam_fc_backward the 2*N*M random reads of x behind w_grad.
 * mam_fc_forward_workspace_for() is the same query for a given operand layout and output set
 * (with_indices: mam_fc_forward, else mam_fc_forward_values): for MAM_W_KM it adds room for one transposed
 * copy of w, with which the call runs the faster (M, K) tiling (from 16 batch rows on, K a multiple of 64;
 * 1.5 times as fast at the 256 x 4096 x 4096 shape, 1.7 times at batch 16384).  A (K, M) call whose workspace only has
 * mam_fc_forward_workspace() bytes still works, on the general tiling.
 */
size_t mam_fc_forward_workspace(int64_t N, int64_t K, int64_t M);
size_t mam_fc_forward_workspace_for(int64_t N, int64_t K, int64_t M, int w_layout, int with_indices);
int mam_fc_forward(const float *x, int64_t ldx, const float *w, int64_t ldw, int w_layout,
                   const float *bias, float *c, int32_t *argmax, int32_t *argmin, float *w_sel,
                   float *x_sel, int64_t N, int64_t K, int64_t M,
                   void *workspace, size_t workspace_bytes, void *stream);

/*
 * Writes into `text` (a host buffer of `text_bytes` bytes, NUL-terminated) which kernels mam_fc_forward
 * (with_indices != 0) or mam_fc_forward_values (with_indices == 0) would launch for these operands: the
 * tiling, the tile grid, the number of K ranges and the bytes of partials.  The choice depends on the
 * alignment of x and w, so the pointers are looked at but never dereferenced.  Pure host call; for bench
 * labels and logs.  No counterpart in the reference, which has one kernel per operator.
 */
int mam_fc_forward_describe(const float *x, int64_t ldx, const float *w, int64_t ldw, int w_layout,
                            int64_t N, int64_t K, int64_t M, int with_indices, char *text, size_t text_bytes);

/*
 * mam_fc_forward for callers that can neither allocate nor bring a workspace (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc): the split-K partials go to a file-scope
 * device array of mam_fc_forward_static_limit() bytes (32 MiB) that every GPU the library runs on holds
 * until the process ends.  No counterpart in the reference (its launcher allocates padded copies and
 * outputs per call, mamtorch/kernel/v1/csrc/cuda/fullyconnected.cu:246-264).  Same arguments, results and
 * errors as mam_fc_forward without `workspace`; a call whose partials exceed the limit is refused with
 * MAM_ERR_UNSUPPORTED before anything is launched (mam_fc_forward_workspace(N, K, M) <=
 * mam_fc_forward_static_limit() guarantees a fit; the query covers the worst alignment, so a call may fit
 * although it says more).  It calls no allocating routine.  All calls on one GPU share that GPU's
 * array: calls that may overlap on one GPU (different streams, different threads) race on it -- serialise
 * them, or use mam_fc_forward with one workspace per stream.  The first call on a device performs that
 * device's one-time set-up (kernel attributes, the array's address; the library's second stream is left for
 * the first call outside a capture) unless mam_init() ran there before.  Nothing in the array has to be cleared
 * between calls (a call writes every word it later reads).
 */
size_t mam_fc_forward_static_limit(void);
int mam_fc_forward_static(const float *x, int64_t ldx, const float *w, int64_t ldw, int w_layout,
                          const float *bias, float *c, int32_t *argmax, int32_t *argmin, float *w_sel,
                          float *x_sel, int64_t N, int64_t K, int64_t M, void *stream);

/*
 * Values-only exact forward (no indices).  Replaces mamtorch_kernel_v4::fullyconnected_fast_cuda
 * (mamtorch/kernel/v4/csrc/cuda/fullyconnected_fast.cu:39-137, kernel
 * fullyconnected_fast_kernel.cu:29-161).  Same c as mam_fc_forward, bit for bit.
 */
size_t mam_fc_forward_values_workspace(int64_t N, int64_t K, int64_t M);
int mam_fc_forward_values(const float *x, int64_t ldx, const float *w, int64_t ldw, int w_layout,
                          const float *bias, float *c, int64_t N, int64_t K, int64_t M,
                          void *workspace, size_t workspace_bytes, void *stream);

/*
 * MAM backward: routes grad only through the selected positions.
 *   x_grad[n,k] = sum_m grad[n,m] * w[k,m] * ([k==argmax[n,m]] + [k==argmin[n,m]])
 *   w_grad[k,m] = sum_n grad[n,m] * x[n,k] * (same)          (argmax==argmin counts twice)
 * x_grad (N,K) and w_grad (layout and shape of w, contiguous) are fully overwritten.
 * Either output pointer may be NULL to skip it.  grad/argmax/argmin are (N,M) contiguous.
 * `w_sel` and `x_sel` (optional, each may be NULL) are the (2, N, M) arrays written by mam_fc_forward for
 * the same inputs; x_grad uses w_sel, w_grad uses x_sel, and whichever is NULL is gathered from w / x.
 * Summation: each term is one fp32 product.  x_grad is accumulated in 64-bit fixed-point cells and is the
 * exact sum of its terms rounded once (independent of the order of arrival, the same bits on every call) as
 * long as at most 512 terms of one workgroup's slab (a batch row, or a few of them) fall outside a window
 * that reaches ~2^25 below the slab's largest term; such terms are added in fp64 before the one rounding,
 * and a slab with more of them is summed with fp32 atomics instead (order-dependent, within rtol 1e-5 plus
 * the rounding floor of an fp32 sum).  w_grad is summed in fp32 in no fixed order, as the reference's
 * atomicAdd does, unless MAM_OPT_BACKWARD_EXACT is on: then it is accumulated the same exact way ((M,K)
 * weights, 16-byte aligned operands, M and K multiples of 4; other calls keep the fp32 route).
 * Replaces fullyconnected_backward_cuda
 * (mamtorch/kernel/v4/csrc/cuda/fullyconnected_backward.cu:80-135, kernel :24-78; v1 identical).
 * Indices outside [0,K) make the call's result undefined for that output only (they are skipped).
 */
int mam_fc_backward(const float *x, int64_t ldx, const float *w, int64_t ldw, int w_layout,
                    const float *grad, const int32_t *argmax, const int32_t *argmin, const float *w_sel,
                    const float *x_sel, float *x_grad, float *w_grad, int64_t N, int64_t K, int64_t M, void *stream);

/*
 * mam_fc_backward followed by mam_selection_count(argmax, argmin, max_count, min_count, ..., count_mode) as
 * ONE call: what a training step does after FullyConnected.forward when the layer keeps selection counts
 * (mamtorch/kernel/v4/csrc/cuda/fullyconnected_backward.cu:80-135 and then
 * mamtorch/nn/v4/fullyconnected.py:114-129).  For (M,K) weights, MAM_COUNT_HITS and a batch below 2048 rows the
 * workgroup that owns four neurons' rows of w_grad also owns their counters: the index arrays are read once
 * for both and one launch fewer is made; every other case runs the two calls one after the other.  Results
 * are those of the two calls (w_grad to the same tolerance, counts exact).
 */
int mam_fc_backward_count(const float *x, int64_t ldx, const float *w, int64_t ldw, int w_layout,
                          const float *grad, const int32_t *argmax, const int32_t *argmin,
                          const float *w_sel, const float *x_sel, float *x_grad, float *w_grad,
                          int32_t *max_count, int32_t *min_count, int count_mode, int64_t N, int64_t K,
                          int64_t M, void *stream);

/*
 * The module's `splits` in one call each way (mamtorch/nn/v4/fullyconnected.py:163-176 runs one operator
 * per slice of the input and adds the slices' outputs with ATen).  K is cut into consecutive ranges of
 * `range_len` inputs, the last one shorter; every range is a MAM neuron of its own:
 *   c[n,m] = ((v_0 + v_1) + v_2 ...) (+ bias[m]),  v_r = max_{k in range r} x*w + min_{k in range r} x*w,
 * added in ascending range order and then the bias, which is the rounding order of the reference's
 * `C_flat += ...` statements.  argmax / argmin (both or neither; NULL = values only, the eval path):
 * [ranges][N][M] int32, plane r holding the lowest ABSOLUTE k of range r attaining its extreme (the
 * reference's per-slice operators return k relative to the slice).  `workspace`:
 * mam_fc_forward_ranges_workspace() bytes (0 when range_len >= K, which is mam_fc_forward).
 *   mam_fc_backward_ranges: the gradient of that c: every range routes grad[n,m] to its own two
 * selected positions.  x_grad (N,K), w_grad (shape and layout of w), either may be NULL.
 */
size_t mam_fc_forward_ranges_workspace(int64_t N, int64_t K, int64_t M, int64_t range_len, int with_indices);
int mam_fc_forward_ranges(const float *x, int64_t ldx, const float *w, int64_t ldw, int w_layout,
                          const float *bias, float *c, int32_t *argmax, int32_t *argmin, int64_t N, int64_t K,
                          int64_t M, int64_t range_len, void *workspace, size_t workspace_bytes, void *stream);
int mam_fc_backward_ranges(const float *x, int64_t ldx, const float *w, int64_t ldw, int w_layout,
                           const float *grad, const int32_t *argmax, const int32_t *argmin, float *x_grad,
                           float *w_grad, int64_t N, int64_t K, int64_t M, int64_t range_len, void *stream);

/*
 * Selection-count accumulation for pruning: adds this batch's picks into (M,K) int32 counters
 * in place.  Replaces FullyConnected.update_selection_count
 * (mamtorch/nn/v4/fullyconnected.py:114-129).  min_count may be NULL in MAM_COUNT_REFERENCE mode.
 */
int mam_selection_count(const int32_t *argmax, const int32_t *argmin, int32_t *max_count,
                        int32_t *min_count, int64_t N, int64_t M, int64_t K, int mode, void *stream);

/*
 * CSR-sparse MAM forward over a pruned weight (M,K): CSR row m = output neuron m,
 * crow (M+1) / col (nnz) int64, val (nnz) fp32, column indices strictly ascending within a
 * row -- the operand convention of mamtorch_kernel_sparsev1::cusparsemm_csr
 * (mamtorch/sparse/kernel/v1/csrc/cuda/cusparsemm_csr.cu:25-45).  The result equals
 * mam_fc_forward on the densified weight: absent entries are zeros that take part in the
 * max/min and in the first-index tie-break.  The reference has no sparse MAM operator.
 * `workspace` (mam_csr_fc_forward_workspace() bytes, 16-byte aligned) receives x transposed.
 * `w_sel` and `pos_sel` (optional, may be NULL): (2, N, M) fp32 / int32 contiguous; receive, for the
 * argmax in plane 0 and the argmin in plane 1, the selected stored value and its position in
 * col/val (0.0f and -1 where an implicit zero was selected).  Handing both to mam_csr_fc_backward
 * spares that call a binary search per selection and all atomics in global memory.  `x_sel` (optional):
 * (2, N, M) fp32, the selected inputs x[n, argmax] / x[n, argmin] (0.0f where an implicit zero was
 * selected); handed to mam_csr_fc_backward it spares val_grad 2 * N * M single-word gathers from x.
 */
size_t mam_csr_fc_forward_workspace(int64_t N, int64_t K, int64_t M);
int mam_csr_fc_forward(const float *x, int64_t ldx, const int64_t *crow, const int64_t *col,
                       const float *val, const float *bias, float *c, int32_t *argmax,
                       int32_t *argmin, float *w_sel, int32_t *pos_sel, float *x_sel, int64_t N, int64_t K,
                       int64_t M, int64_t nnz, void *workspace, size_t workspace_bytes, void *stream);

/*
 * Checks, on the device, the CSR invariants that mam_csr_fc_forward / _backward / mam_csr_spmm take for
 * granted (they index x, b and the outputs with col[] and crow[] unchecked, as cusparseSpMM does behind
 * mamtorch/sparse/kernel/v1/csrc/cuda/cusparsemm_csr.cu:37-69): *status (one int32 in device memory)
 * receives 0 when all hold, else the OR of 1: crow[0] != 0 or crow[M] != nnz, 2: crow decreasing or out of
 * range, 4: a column index outside [0, K), 8: columns not strictly ascending within a row (the MAM forward
 * needs ascending columns; mam_csr_spmm does not).  Asynchronous like every other call; the caller reads
 * *status after synchronising.  No counterpart in the reference.
 */
int mam_csr_validate(const int64_t *crow, const int64_t *col, int64_t M, int64_t K, int64_t nnz, int *status,
                     void *stream);

/*
 * CSR-sparse MAM backward: x_grad (N,K) dense and val_grad (nnz), both fully overwritten; either may
 * be NULL to skip it.  A selected column that is not stored in its row (an implicit zero won) has no
 * weight gradient and adds nothing to x_grad.  `w_sel` / `pos_sel` (optional, both or neither) and `x_sel`
 * (optional, only together with the other two) are the arrays written by mam_csr_fc_forward for the same
 * inputs.
 */
int mam_csr_fc_backward(const float *x, int64_t ldx, const int64_t *crow, const int64_t *col,
                        const float *val, const float *grad, const int32_t *argmax,
                        const int32_t *argmin, const float *w_sel, const int32_t *pos_sel,
                        const float *x_sel, float *x_grad, float *val_grad, int64_t N, int64_t K, int64_t M,
                        int64_t nnz, void *stream);

/*
 * Sum-of-products SpMM: c (R, C) contiguous = A (R, K) sparse @ b (K, C) dense with row stride ldb,
 * fp32, alpha 1, beta 0.  Replace mamtorch_kernel_sparsev1::cusparsemm_csr
 * (mamtorch/sparse/kernel/v1/csrc/cuda/cusparsemm_csr.cu:19-77) and ::cusparsemm_coo
 * (mamtorch/sparse/kernel/v1/csrc/cuda/cusparsemm_coo.cu:19-76), both thin wrappers of cusparseSpMM with
 * int64 indices.  CSR: crow (R+1), col / val (nnz); any column order within a row.  COO: row / col / val
 * (nnz) in any order, repeated coordinates add up (as an uncoalesced torch COO tensor means); c is
 * accumulated with atomic adds, so its rounding can differ from run to run when a row spans more than
 * 64 consecutive entries.
 */
int mam_csr_spmm(const int64_t *crow, const int64_t *col, const float *val, const float *b, int64_t ldb,
                 float *c, int64_t R, int64_t K, int64_t C, void *stream);
int mam_coo_spmm(const int64_t *row, const int64_t *col, const float *val, int64_t nnz, const float *b,
                 int64_t ldb, float *c, int64_t R, int64_t K, int64_t C, void *stream);

/*
 * The sparse operand written out as a dense (R, K) fp32 matrix with row stride ld (cleared first; repeated
 * coordinates add up).  No counterpart in the reference: from about one stored entry in eight on, the
 * cusparsemm operator of this build forms a @ b as a dense GEMM of this matrix (the library GEMM of the
 * platform), which is then faster than any walk over the entries.
 */
int mam_csr_to_dense(const int64_t *crow, const int64_t *col, const float *val, float *dense, int64_t ld,
                     int64_t R, int64_t K, void *stream);
int mam_coo_to_dense(const int64_t *row, const int64_t *col, const float *val, int64_t nnz, float *dense,
                     int64_t ld, int64_t R, int64_t K, void *stream);

/*
 * out (N, M) = (alpha * mam_out + beta * mac_out) + bias, each an (N, M) contiguous fp32 array (out may
 * alias mam_out or mac_out), bias (M) or NULL: the vanishing-contribution blend of the module
 * (mamtorch/nn/v4/fullyconnected.py:190-198) in one pass, in the reference's rounding order (two
 * products, their sum, then the bias; nothing fused).
 */
int mam_blend(const float *mam_out, const float *mac_out, const float *bias, float alpha, float beta, float *out,
              int64_t N, int64_t M, void *stream);

/*
 * bias_grad[m] = sum over the batch rows of grad[n, m]: the gradient of the bias the layer adds after max + min
 * (mamtorch/nn/v4/fullyconnected.py:197-198; in the reference autograd derives this column sum from the `+`).
 * fp32 adds in a fixed order (the same bits on every call).  `workspace`: mam_bias_grad_workspace(N, M) bytes
 * (0 up to 512 batch rows).
 */
size_t mam_bias_grad_workspace(int64_t N, int64_t M);
int mam_bias_grad(const float *grad, int64_t ld, float *bias_grad, int64_t N, int64_t M, void *workspace,
                  size_t workspace_bytes, void *stream);

/*
 * out (M, K) contiguous = w (M, K, row stride ldw) * (keep ? 1 : 0), keep (M, K) contiguous bytes: the
 * training-time weight dropout of the module (mamtorch/nn/v4/fullyconnected.py:143-148, there a float
 * Bernoulli mask of the weight's size times the transposed weight) in one pass from a byte mask.  The
 * product is formed as the reference forms it, so a dropped weight is a zero with the weight's sign.  The
 * same call masks the weight gradient on the way back.
 */
int mam_apply_keep(const float *w, int64_t ldw, const unsigned char *keep, float *out, int64_t M, int64_t K,
                   void *stream);

/*
 * MAM convolution as the MAM fully-connected kernel over gathered windows.  x is (B, C, H, W) contiguous
 * (a 1-D convolution has H = k1 = s1 = 1), windows are k1 x k2 with strides s1, s2 and no padding (the
 * caller pads, as the reference's modules do), output positions L1 = (H - k1) / s1 + 1, L2 likewise.
 *   mam_im2col : cols (B * L1 * L2, k2 * k1 * C) contiguous; cols[(b, l1, l2), (j2 * k1 + j1) * C + c] =
 *                x[b, c, l1 * s1 + j1, l2 * s2 + j2].  The column order is the index order of the reference's
 *                retired kernels (mamtorch/kernel/backup/mamconv1d_forward.txt:128: arg = position * C +
 *                channel; mamconv2d_forward.txt with the window column outermost), so mam_fc_forward on
 *                (cols, weight reordered to (F, k2 * k1 * C)) yields their Y, argmax and argmin.
 *   mam_col2im : the adjoint, x_grad (B, C, H, W) fully overwritten = sum over the windows covering each cell
 *                of cols_grad; replaces the input-gradient half of mamconv1d/2d_backward
 *                (mamtorch/kernel/backup/mamconv1d_backward.txt).  No atomics; fixed summation order.
 */
int mam_im2col(const float *x, float *cols, int64_t B, int64_t C, int64_t H, int64_t W, int64_t k1, int64_t k2,
               int64_t s1, int64_t s2, void *stream);
int mam_col2im(const float *cols_grad, float *x_grad, int64_t B, int64_t C, int64_t H, int64_t W, int64_t k1,
               int64_t k2, int64_t s1, int64_t s2, void *stream);

/*
 * Pruning of a dense weight w (M,K), row stride ldw, and its compaction to CSR.  An entry is pruned when
 * its score is not above `threshold` -- the reference's `w[score.abs() <= threshold] = 0`
 * (examples/vitb16_imagenet1k/pruning_utils.py:103-111 magnitude, :190-203 weight x gradient) -- and the
 * score is chosen by `mode` (MAM_PRUNE_*); `aux` / `aux2` are (M,K) arrays of row stride ld_aux (aux2 only
 * for MAM_PRUNE_COUNT, may be NULL): the counters kept by mam_selection_count
 * (mamtorch/nn/v4/fullyconnected.py:107-131) are the third score.
 *   mam_prune_row_offsets : crow (M+1) int64 = CSR row offsets of the survivors; nnz = crow[M]
 *   mam_prune_fill_csr    : col (nnz) int64 ascending per row and val (nnz) fp32, for the same arguments
 *   mam_prune_apply       : the reference's in-place form, pruned entries of w become 0.0f
 * The reference itself keeps pruned weights dense; the CSR operands are what mam_csr_fc_forward and
 * mam_csr_spmm take.
 */
int mam_prune_row_offsets(const float *w, int64_t ldw, int mode, const void *aux, const void *aux2,
                          int64_t ld_aux, float threshold, int64_t *crow, int64_t M, int64_t K, void *stream);
int mam_prune_fill_csr(const float *w, int64_t ldw, int mode, const void *aux, const void *aux2,
                       int64_t ld_aux, float threshold, const int64_t *crow, int64_t *col, float *val,
                       int64_t M, int64_t K, void *stream);
int mam_prune_apply(float *w, int64_t ldw, int mode, const void *aux, const void *aux2, int64_t ld_aux,
                    float threshold, int64_t M, int64_t K, void *stream);

/*
 * The pruning threshold without a sort: the element(s) of given rank among the absolute scores of one or
 * several matrices.  Replaces `torch.quantile(flattened_weights.abs(), p)`
 * (examples/vitb16_imagenet1k/pruning_utils.py:103-104, :106-110) and the sort of the concatenated scores of
 * all layers followed by `concatenated_tensor[int(p * len)]` (:139-143, :246-250).  Scores are those of the
 * pruning calls above (`mode`, `aux`, `aux2`).  A radix select over the scores' bit patterns: three histogram
 * passes, each over every tensor, and a step after each pass:
 *     mam_select_begin(ws, bytes, ranks, nranks, stream)         ranks: HOST array of 1 or 2 ascending 0-based ranks
 *     for pass in 0, 1, 2:
 *         mam_select_accumulate(ws, w, ldw, mode, aux, aux2, ld_aux, M, K, pass, stream)     once per tensor
 *         mam_select_advance(ws, pass, stream)
 *     mam_select_result(ws, mode, out, stream)                   out: DEVICE array of nranks floats
 * The result is exactly the element a full ascending sort of the |scores| holds at each rank (NaN scores
 * order above infinity, as torch.sort places them); for MAM_PRUNE_COUNT it is the count as a float.
 * `ws` is device memory of mam_select_workspace() bytes, 16-byte aligned; nothing synchronises.
 */
size_t mam_select_workspace(void);
int mam_select_begin(void *workspace, size_t workspace_bytes, const int64_t *ranks, int nranks, void *stream);
int mam_select_accumulate(void *workspace, const float *w, int64_t ldw, int mode, const void *aux,
                          const void *aux2, int64_t ld_aux, int64_t M, int64_t K, int pass, void *stream);
int mam_select_advance(void *workspace, int pass, void *stream);
int mam_select_result(void *workspace, int mode, float *out, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* MAM_HIP_H */
