/* C ABI of libtriteia_hip.so -- the MI355X (gfx950) implementation of Triteia's
 * fp16 x (int4, 2:4-sparse) multi-model GEMM path and its LoRA companions.
 *
 * Every entry point takes plain device pointers and sizes, enqueues its work on
 * `stream` (a hipStream_t passed as void*; NULL = the default stream) of
 * device `dev`, and returns without synchronising.  Nothing is allocated or
 * freed by the library; all buffers, including workspaces, belong to the
 * caller and are borrowed until the enqueued work has run.
 *
 * Dimension names follow the reference launchers: prob_m = output features,
 * prob_n = tokens (rows of A / C), prob_k = input features.
 *
 * Tensor layouts (identical to the reference's, see its packer
 * triteia/python/nn/linear.py:79-141):
 *   A     fp16  [prob_n, prob_k]            row-major activations
 *   B     int32 [prob_k/32, 2*prob_m]       packed 2:4 int4 weights
 *   meta  int16 [prob_m, prob_k/16]         2:4 metadata (Sparse-Marlin order)
 *   s     fp16  [1, prob_m]                 per-output-channel scales
 *   C     fp16  [prob_n, prob_m]            row-major output
 * Batched variants carry a leading delta dimension on B / meta / s.
 *
 * Return codes: 0 on success, otherwise one of the TRITEIA_HIP_ERR_* values;
 * triteia_hip_last_error() describes the last failure on the calling thread.
 */
#ifndef TRITEIA_HIP_H_
#define TRITEIA_HIP_H_

#include <stddef.h>
#include <stdint.h>

#if defined(__GNUC__)
#define TRITEIA_HIP_API __attribute__((visibility("default")))
#else
#define TRITEIA_HIP_API
#endif

#ifdef __cplusplus
extern "C" {
#endif

#define TRITEIA_HIP_OK 0
#define TRITEIA_HIP_ERR_PROB_SHAPE 1 /* reference: ERR_PROB_SHAPE, csrc/ops/marlin_nm.cu:39 */
#define TRITEIA_HIP_ERR_KERN_SHAPE 2 /* reference: ERR_KERN_SHAPE, csrc/ops/marlin_nm.cu:40 */
#define TRITEIA_HIP_ERR_ARGUMENT 3   /* null pointer, undersized workspace, bad flag */
#define TRITEIA_HIP_ERR_RUNTIME 4    /* a HIP call failed */

/* Library / ABI version (major * 1000 + minor). */
TRITEIA_HIP_API int triteia_hip_version(void);

/* Text of the last error raised on this thread ("" if none). */
TRITEIA_HIP_API const char* triteia_hip_last_error(void);

/* The library's tuning knobs (environment variables TRITEIA_HIP_*, for tests and
 * measurements) are read once, at the first call into the library; this reads
 * them again.  Not to be called while another thread is inside the library, nor
 * between triteia_hip_route_plan and the calls that consume its plan (both sides
 * derive the plan's tile size from the knobs).  No counterpart in the reference. */
TRITEIA_HIP_API void triteia_hip_reload_env(void);

/* C = A @ dequant(B, meta, s) for one weight matrix.
 * Replaces marlin_cuda_2_4 (triteia/csrc/ops/marlin_nm.cu:42-46), bound by the
 * reference as mul_2_4 (triteia/csrc/ops/ops.cpp:88-116).
 * workspace: the reference's lock array (>= prob_m/128*max_par int32 zeros); it
 * is accepted, never read or written, and therefore left all-zero.
 * groupsize, in the reference's unit of compressed k (marlin_nm.cu:68): -1 = one scale per output column, s [1, m];
 * 64 = one per column and 128 dense k, s [prob_k / 128, m] with every run of 8 columns stored in the order
 * 0 4 1 5 2 6 3 7 (triteia/python/ops/utils/sparsity.py:54-57), prob_k % 128 == 0; anything else ERR_KERN_SHAPE
 * (the reference instantiates the same two, marlin_nm.cu:102-111).  The batched and routed entry points below take
 * -1 only.  thread_k, thread_m, sms, max_par
 * are the reference's tuning knobs; they are accepted and ignored.
 * Shape rules: prob_m % 128 == 0 and prob_k % 64 == 0, else ERR_PROB_SHAPE. */
TRITEIA_HIP_API int triteia_hip_mul_2_4(const void* A, const void* B, const void* meta, void* C, const void* s, int prob_m, int prob_n,
                        int prob_k, void* workspace, int groupsize, int dev, void* stream, int thread_k, int thread_m,
                        int sms, int max_par);

/* C[b, 0, :] = A[b, 0, :] @ dequant(B[b]) for b < prob_n: one token per matrix.
 * Replaces triteia_cuda_bmm_2_4 (triteia/csrc/ops/triteia_nm_bmm.cu:760-764),
 * bound as bmm_2_4 (triteia/csrc/ops/ops.cpp:240-277).  prob_n = batch. */
TRITEIA_HIP_API int triteia_hip_bmm_2_4(const void* A, const void* B, const void* meta, void* C, const void* s, int prob_m, int prob_n,
                        int prob_k, void* workspace, int groupsize, int dev, void* stream, int thread_k, int thread_m,
                        int sms, int max_par);

/* Same with `tokens` rows per matrix: A [batch, tokens, k], C [batch, tokens, m].
 * The reference kernel hard-codes tokens == 1 (triteia_nm_bmm.cu:736-739); its
 * Python for-loop variant (triteia/python/ops/matmul/bmm.py:6-18) defines the
 * semantics for tokens > 1. */
TRITEIA_HIP_API int triteia_hip_bmm_2_4_tokens(const void* A, const void* B, const void* meta, void* C, const void* s, int prob_m,
                               int batch, int tokens, int prob_k, int dev, void* stream);

/* The same with a scratch buffer of the caller's (device memory, 16-byte aligned, contents irrelevant, overwritten),
 * which lets a launch of few workgroups split K across workgroups: every workgroup writes the fp32 sums of its
 * share of K to the buffer and a second, small launch adds the shares in a fixed order (the result is a function of
 * the inputs only, but may differ in the last bit from the call without scratch, which adds over K in one
 * workgroup).  triteia_hip_bmm_scratch_bytes says how many bytes the split of a launch uses (0: this launch would not
 * be split and ignores the buffer); a smaller or null buffer simply leaves K unsplit.  batch = 1 is the single-matrix
 * product.  The counterpart in the reference is the stripe partitioning of one GEMM over all SMs with its
 * reduction through C under locks (triteia/csrc/ops/marlin.cuh:449-519, marlin_nm.cu:19-37): the lock array of its
 * argument list is too small for fp32 partial sums, hence the separate argument here. */
TRITEIA_HIP_API int triteia_hip_bmm_2_4_tokens_scratch(const void* A, const void* B, const void* meta, void* C, const void* s, int prob_m,
                                       int batch, int tokens, int prob_k, void* scratch, size_t scratch_bytes, int dev,
                                       void* stream);
TRITEIA_HIP_API size_t triteia_hip_bmm_scratch_bytes(int prob_m, int batch, int tokens, int prob_k);

/* Which kernel the uniform-group entry points (mul_2_4: batch = 1; bmm_2_4*) run most of a launch's rows on: 0 = the
 * K-split streaming kernel (sparse24_grouped_kernel), 16 = shares of 16, 32 or 64 columns on sparse24_share16_kernel (at most 16 tokens per
 * matrix, launches of at most 32 / 64 / 128 column blocks of 128), 1000 + n = the same with K split over n workgroups (only
 * with_scratch != 0), 32 / 64 = 32- / 64-token tiles of sparse24_wide_kernel (+ 1: on eight wavefronts), 256 =
 * sparse24_tile256_kernel; -1 for a shape the entry points reject.  No counterpart in the reference; for benchmarks,
 * profiles and the test that guards the dispatch thresholds. */
TRITEIA_HIP_API int triteia_hip_uniform_kernel(int prob_m, int batch, int tokens, int prob_k, int with_scratch);

/* Run-list form: for run r < prob_r, rows starts[r] .. starts[r]+counts[r]-1 of
 * C = same rows of A @ dequant(B[indices[r]]).  indices / starts / counts are
 * int32 device arrays.  Replaces triteia_cuda_sbmm_2_4
 * (triteia/csrc/ops/triteia_nm_sbmm.cu:809-815; the argument list is the same),
 * bound as sbmm_2_4 and, for the host-loop variant, sbmm_forloop
 * (triteia/csrc/ops/ops.cpp:279-327).  Rows not covered by a run are left
 * untouched; runs with a negative index are skipped.  Like the reference's, this
 * argument list does not say how many matrices B holds: every non-negative
 * index must be valid. */
TRITEIA_HIP_API int triteia_hip_sbmm_2_4(const void* A, const void* B, const void* meta, void* C, const void* s, const void* indices,
                         const void* starts, const void* counts, int prob_m, int prob_n, int prob_k, int prob_r,
                         void* workspace, int groupsize, int dev, void* stream, int thread_k, int thread_m, int sms,
                         int max_par);

/* The same with a trailing n_deltas = number of matrices in B: runs whose index
 * lies outside [0, n_deltas) are skipped instead of read out of bounds.  No
 * counterpart in the reference (whose kernel trusts the indices,
 * triteia_nm_sbmm.cu:743-748). */
TRITEIA_HIP_API int triteia_hip_sbmm_2_4_bounded(const void* A, const void* B, const void* meta, void* C, const void* s,
                                 const void* indices, const void* starts, const void* counts, int prob_m, int prob_n,
                                 int prob_k, int prob_r, void* workspace, int groupsize, int dev, void* stream,
                                 int thread_k, int thread_m, int sms, int max_par, int n_deltas);

/* Per-token routed form (no counterpart kernel in the reference; it replaces the
 * host-side routing prep of triteia/python/ops/matmul/sbmm.py:94-123 plus the
 * kernel above plus the trailing `y += output`, sbmm.py:141):
 *   d = token_indices[t] - index_offset
 *   0 <= d < n_deltas :  C[t] = (accumulate ? C[t] : 0) + A[t] @ dequant(B[d])
 *   otherwise         :  C[t] untouched
 * token_indices: int32 [prob_n] on the device, any order.  The tokens are
 * grouped on the device, so each delta's weights are read once per launch.
 * workspace: >= triteia_hip_sbmm_routed_workspace_bytes(prob_n, n_deltas) bytes
 * of device memory, contents irrelevant on entry, overwritten (batches of at most 64
 * tokens over at most 64 deltas are always routed inside the multiply kernel and leave it
 * untouched; so are most batches of up to 256 tokens over at most 16 deltas, but not all:
 * pass the workspace for every batch above 64 tokens).
 * n_deltas <= 8192. */
TRITEIA_HIP_API int triteia_hip_sbmm_2_4_routed(const void* A, const void* B, const void* meta, void* C, const void* s,
                                const void* token_indices, int index_offset, int n_deltas, int prob_m, int prob_n,
                                int prob_k, void* workspace, size_t workspace_bytes, int accumulate, int dev,
                                void* stream);
TRITEIA_HIP_API size_t triteia_hip_sbmm_routed_workspace_bytes(int prob_n, int n_deltas);

/* triteia_hip_sbmm_2_4_routed without the workspace argument, for callers that cannot allocate
 * device memory (code under HIP graph capture, tight serving loops, harnesses that forbid it).  It
 * has no counterpart in the reference.  The routing plan lives in a buffer inside the library's own
 * device image (triteia_hip_sbmm_routed_static_max_bytes() = 256 KiB per GPU, held until the process
 * ends); the call allocates and frees nothing.  Batches whose plan
 * (triteia_hip_sbmm_routed_workspace_bytes(prob_n, n_deltas)) does not fit return
 * TRITEIA_HIP_ERR_KERN_SHAPE: 8192 tokens over 1024 deltas fit, 65536 tokens over 64 deltas do not.
 * Every call on one GPU uses that GPU's one buffer: calls that overlap in time on the same GPU
 * (different streams, or one stream's call not finished when another's starts) race on it; calls in
 * stream order on one stream are safe.  Results are those of triteia_hip_sbmm_2_4_routed, bit for bit. */
TRITEIA_HIP_API int triteia_hip_sbmm_2_4_routed_static(const void* A, const void* B, const void* meta, void* C, const void* s,
                                       const void* token_indices, int index_offset, int n_deltas, int prob_m,
                                       int prob_n, int prob_k, int accumulate, int dev, void* stream);
TRITEIA_HIP_API size_t triteia_hip_sbmm_routed_static_max_bytes(void);

/* Only the routing step of triteia_hip_sbmm_2_4_routed: fills `workspace` (16-byte aligned) with
 *   int32 header[8] = {narrow tiles, routed tokens, deltas in use, narrow tile size,
 *                      wide tiles, tiles of all[], tiles of big[], 0}
 *   int32 tiles[max_tiles][4] = {delta, start, count, 0}: at most `tile size` tokens of one
 *         delta, listed at perm[start .. start+count); a delta's tiles are adjacent
 *   int32 wide[max_wide][4]   = the same for 64-token tiles; only batches of at least 256
 *         tokens (environment TRITEIA_HIP_WIDE_MIN_BATCH) with at least 8 tokens per delta on
 *         average get any: a delta with c tokens then has c/64 full wide tiles, one more if
 *         the rest exceeds 32 tokens, and narrow tiles for a smaller rest
 *   int32 perm[prob_n] = token rows grouped by delta, original order kept (stable)
 *   int32 all[max_tiles][4]   = at the next multiple of 4 ints: for plans with wide tiles, the
 *         same tokens cut into narrow tiles only (header[5] of them).  The multiply kernels pick
 *         {tiles, wide} or {all} per weight shape on the device: the wide kernel runs only if
 *         its tiles fill the chip (wide tiles x ceil(prob_m / 512) >= 150, environment
 *         TRITEIA_HIP_PLAN_WIDE_MIN_UNITS); the LoRA path always takes all[].
 *   int32 big[max_big][4]     = for batches of at least 24 tokens per delta (of min(prob_n, n_deltas) deltas) whose
 *         narrow tile size is 32: the same tokens cut into 64-token tiles only (header[6] of them), which wide layers
 *         take on the 64-token build of the wide kernel -- from 48 tokens per delta on, or in launches of three rounds
 *         of workgroups and more (environment TRITEIA_HIP_PLAN_BIG=0: never; above 1: the bar in tokens per delta)
 * with max_tiles = min(prob_n, n_deltas) + prob_n / 16, max_wide = prob_n / 33 + 1 and
 * max_big = min(prob_n, n_deltas) + prob_n / 64.  The
 * narrow tile size is triteia_hip_plan_tile_tokens(prob_n, n_deltas).  Exposed so that one
 * routing pass can serve every layer of a forward pass and the LoRA path. */
TRITEIA_HIP_API int triteia_hip_route_plan(const void* token_indices, int index_offset, int n_deltas, int prob_n, void* workspace,
                           size_t workspace_bytes, int dev, void* stream);

TRITEIA_HIP_API int triteia_hip_plan_tile_tokens(int prob_n, int n_deltas);

/* Which kernel triteia_hip_sbmm_2_4_planned runs a plan's narrow tiles on for this batch and layer:
 * 0 = the K-split narrow kernel (sparse24_grouped_kernel), 32 / 64 = the 32- / 64-token build of the
 * wide kernel taking the plan's narrow-only list, or its list of 64-token tiles where the narrow tiles are of 32
 * (wide layers; see the design notes).  No counterpart in
 * the reference; for benchmarks and profiles, and for tests that compare results bit for bit (the two
 * kernels add over K in different orders). */
TRITEIA_HIP_API int triteia_hip_planned_tile_kernel(int prob_n, int n_deltas, int prob_m, int prob_k);

/* The order in which sparse24_wide_kernel numbers its units (token tile x group of 512 columns) on a layer of prob_m
 * columns (1: column groups padded to a multiple of 8, a contiguous run per XCD; 3: the same with the padding's idle
 * slots put to work, on layers where the padding would leave XCDs short of work; 0 / 2 by environment only), and the
 * number of workgroups of a launch over `rows` tiles in a given order; for the order that the host picks per launch
 * (4: every XCD takes a block of `block_column_groups` column groups x a block of tiles), the number of workgroups
 * by block size, -1 where the layer's padded column groups cannot be cut that way over 8 XCDs.  No counterpart in the reference; for the tests
 * that check each order against a restatement of the kernel's index arithmetic. */
TRITEIA_HIP_API int triteia_hip_wide_unit_order(int prob_m);
TRITEIA_HIP_API long triteia_hip_wide_grid_units(long rows, int prob_m, int order);
TRITEIA_HIP_API long triteia_hip_wide_block_grid_units(long rows, int prob_m, int block_column_groups);

/* 1 or 2 if triteia_hip_sbmm_2_4_routed handles this batch and layer in one launch, routing inside the multiply kernel
 * (the workspace stays untouched; 2: at most 16 tokens on the column-share kernel, sparse24_share16_kernel, 1: the
 * streaming kernel), 0 if it builds a routing plan first.  No counterpart in the reference; for
 * benchmarks and profiles. */
TRITEIA_HIP_API int triteia_hip_routed_in_kernel(int prob_n, int n_deltas, int prob_m, int prob_k);


/* The multiply step alone, on a plan made by triteia_hip_route_plan for the same
 * (prob_n, n_deltas): C[t] (+)= A[t] @ dequant(B[d]) for every routed token.  One
 * plan serves every layer of a forward pass (the routing of a batch does not
 * change between layers) and the LoRA path.  No counterpart in the reference. */
TRITEIA_HIP_API int triteia_hip_sbmm_2_4_planned(const void* A, const void* B, const void* meta, void* C, const void* s,
                                 const void* plan, int n_deltas, int prob_m, int prob_n, int prob_k, int accumulate,
                                 int dev, void* stream);

/* BGMV: Y[b, :] += scale * W[indices[b] * num_layers + layer_idx] @ X[b, :]
 * with W [n, num_layers, h_out, h_in] fp16 (out-major) and indices int64 [batch]
 * (negative = skip).  Replaces bgmv_kernel<feat_in, feat_out, T>
 * (triteia/csrc/ops/bgmv_config.h:3-7, bgmv_impl.cuh:185-207), bound as
 * dispatch_bgmv (triteia/csrc/ops/ops.cpp:177-220).  Unlike the reference it
 * runs on `stream`, and shapes are run-time values: both sides multiples of 8
 * and min(h_in, h_out) <= 128, else ERR_KERN_SHAPE ("No suitable kernel"). */
TRITEIA_HIP_API int triteia_hip_bgmv(void* Y, const void* X, const void* W, const void* indices, int batch, int h_in, int h_out,
                     int num_layers, int layer_idx, float scale, int dev, void* stream);
/* The same for bf16 tensors (Y, X, W): the reference instantiates bgmv_kernel for nv_half and nv_bfloat16
 * (triteia/csrc/ops/bgmv_all.cu:4-5) and dispatches on the tensors' dtype (ops.cpp:199-214). */
TRITEIA_HIP_API int triteia_hip_bgmv_bf16(void* Y, const void* X, const void* W, const void* indices, int batch, int h_in, int h_out,
                          int num_layers, int layer_idx, float scale, int dev, void* stream);
/* Y[b, :] = scale * W[...] @ X[b, :]: the same product stored instead of added (Y is not read; rows with a negative
 * index are left as they are).  No counterpart in the reference, whose add_lora_bgmv clears a [batch, rank]
 * intermediate and adds into it (triteia/python/capi/punica.py:59-68): with this form the intermediate needs no clearing. */
TRITEIA_HIP_API int triteia_hip_bgmv_store(void* Y, const void* X, const void* W, const void* indices, int batch, int h_in, int h_out,
                           int num_layers, int layer_idx, float scale, int dev, void* stream);
TRITEIA_HIP_API int triteia_hip_bgmv_store_bf16(void* Y, const void* X, const void* W, const void* indices, int batch, int h_in, int h_out,
                                int num_layers, int layer_idx, float scale, int dev, void* stream);

/* SGMV: y[s[i] : s[i+1]] += x[s[i] : s[i+1]] @ W_i, W_i = (fp16*)w_ptrs[i] +
 * layer_idx * d_in * d_out, row-major [d_in, d_out]; s int32 [num_problems+1].
 * Replaces sgmv<T> (triteia/csrc/ops/sgmv.h:6-11, sgmv.cuh:61-174), bound as
 * dispatch_sgmv_cutlass (triteia/csrc/ops/ops.cpp:120-147).  tmp is the
 * reference's CUTLASS argument scratch; it is accepted and unused. */
TRITEIA_HIP_API int triteia_hip_sgmv(void* y, const void* x, const void* w_ptrs, const void* s, void* tmp, int num_problems, int d_in,
                     int d_out, int layer_idx, int dev, void* stream);
TRITEIA_HIP_API size_t triteia_hip_sgmv_tmp_size(int num_problems); /* reference: sgmv_tmp_size, sgmv.cuh:48-52 */
/* The same for bf16 tensors (y, x and the matrices behind w_ptrs): sgmv<nv_bfloat16> (triteia/csrc/ops/sgmv.cu:10,
 * dispatched on x's dtype, ops.cpp:132-143). */
TRITEIA_HIP_API int triteia_hip_sgmv_bf16(void* y, const void* x, const void* w_ptrs, const void* s, void* tmp, int num_problems, int d_in,
                          int d_out, int layer_idx, int dev, void* stream);
/* y[s[i] : s[i+1]] = x[s[i] : s[i+1]] @ W_i: the same product stored instead of added (y is not read; rows outside
 * every segment are left as they are).  No counterpart in the reference, whose add_lora_sgmv_cutlass clears the
 * [rows, rank] intermediate first (triteia/python/capi/punica.py:30-57). */
TRITEIA_HIP_API int triteia_hip_sgmv_store(void* y, const void* x, const void* w_ptrs, const void* s, int num_problems, int d_in, int d_out,
                           int layer_idx, int dev, void* stream);
TRITEIA_HIP_API int triteia_hip_sgmv_store_bf16(void* y, const void* x, const void* w_ptrs, const void* s, int num_problems, int d_in, int d_out,
                                int layer_idx, int dev, void* stream);

/* Routed SGMV on a routing plan made by triteia_hip_route_plan: for every group
 * g (adapter a = g_delta[g]) and every listed row t:
 *   y[t] (+)= scale * x[t] @ W[a],  W = w_base + a * w_stride (elements),
 *   row-major [d_in, d_out]; accumulate = 1 adds to y, 0 stores (y is not read, rows
 *   that the plan does not list are left as they are).
 * No counterpart in the reference, which builds the segment table on the host
 * (triteia/python/ops/matmul/lora.py:63-96). */
TRITEIA_HIP_API int triteia_hip_sgmv_routed(void* y, long y_stride, const void* x, long x_stride, const void* w_base, long w_stride,
                            int n_adapters, int d_in, int d_out, float scale, const void* plan, int prob_n,
                            int accumulate, int dev, void* stream);

/* The same for bf16 tensors (y, x, w_base). */
TRITEIA_HIP_API int triteia_hip_sgmv_routed_bf16(void* y, long y_stride, const void* x, long x_stride, const void* w_base, long w_stride,
                                 int n_adapters, int d_in, int d_out, float scale, const void* plan, int prob_n,
                                 int accumulate, int dev, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* TRITEIA_HIP_H_ */
