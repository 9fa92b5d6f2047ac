/*
 * C ABI of libmoe_hip.so -- the gfx950 (MI355X) implementation of the dropless MoE expert-MLP hot path.
 *
 * Conventions (all entry points):
 *   - plain C: device pointers as void*, sizes/strides as int64_t counted in ELEMENTS, no framework types;
 *   - the caller owns every buffer (inputs, outputs, workspace); nothing is allocated, freed or synchronised
 *     inside, every kernel is enqueued on `stream` (a hipStream_t passed as void*; NULL = default stream);
 *   - return value 0 = enqueued, negative = MOE_ERR_* below (nothing was enqueued for MOE_ERR_BAD_ARG,
 *     MOE_ERR_UNSUPPORTED and MOE_ERR_WORKSPACE);
 *   - dtype: MOE_BF16 / MOE_F16 / MOE_F32 selects the element type of activations, weights and outputs;
 *     bf16 with 16-byte aligned, unit-inner-stride operands runs on the matrix-core kernels, everything else on
 *     the generic fp32-FMA kernels of the same library (never on the host);
 *   - index tensors may be int32 or int64: the *_64 flags say which;
 *   - a call with zero rows / tokens is valid, enqueues nothing and may pass NULL for the tensors of that extent;
 *   - re-entrant: safe to call from the autograd engine's threads; the only process-wide state is the optional stage
 *     timer below.
 *
 * Each declaration cites the reference interface it stands in for (paths relative to the reference repository
 * foundation-model-stack/moe-distributed-training).
 */
#ifndef MOE_HIP_H
#define MOE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MOE_HIP_ABI_VERSION 2   /* 2: router weight gradient, static-scratch sort, stage-timer selection, moe_combine with k = 0; fp16 on the matrix cores (dtype argument of moe_mlp_fwd / moe_mlp_bwd) */

#define MOE_OK 0
#define MOE_ERR_BAD_ARG (-1)      /* inconsistent sizes / null pointers */
#define MOE_ERR_UNSUPPORTED (-2)  /* combination not implemented (e.g. LoRA rank > 32 on a fused path) */
#define MOE_ERR_WORKSPACE (-3)    /* workspace smaller than the matching *_workspace_bytes() */
#define MOE_ERR_LAUNCH (-4)       /* HIP reported a launch error */

#define MOE_BF16 0
#define MOE_F16 1
#define MOE_F32 2

int moe_hip_abi_version(void);
const char* moe_hip_strerror(int status);

/* ---- stage timer (measurement aid; no counterpart in the reference) ----------------------------------------
 * moe_profile_enable(1) clears the record list and makes the fused entry points (moe_mlp_fwd / moe_mlp_bwd) bracket
 * each kernel group they enqueue with a pair of events on the caller's stream; moe_profile_enable(0) stops it.
 * moe_profile_get(i, ...) waits for record i and returns its stage name and device time in milliseconds.
 * This is the only process-wide state of the library and is off unless a harness turns it on. */
int moe_profile_enable(int on);
/* restricts the bracketing to stages whose name contains one of the comma-separated substrings (NULL or "": every
 * stage).  A pair of events costs a few microseconds of device time, so a harness that times a whole step brackets only
 * what it prices inside that region. */
int moe_profile_select(const char* substrings);
int moe_profile_count(void);
int moe_profile_get(int i, char* name, int name_cap, float* ms);

/* ---- tile plan of the grouped GEMM (test aid; no counterpart in the reference) ------------------------------
 * The matrix-core grouped GEMM hands every workgroup one work item (an output tile of one expert, or one K part of a
 * tile).  moe_gemm_debug_plan_blocks() returns the number of workgroups a launch over R rows, E experts and N output
 * columns uses (pair != 0: the gate/up pair kernel with 128 columns per projection and tile);
 * moe_gemm_debug_plan() writes, for each of them, 9 ints into `out` (device memory): valid, expert, n tile, first
 * row, one-past-last row, K part, K parts, exchange slot, split-tile counter.  Tests use it to check that every tile
 * is covered exactly once for any group sizes. */
int64_t moe_gemm_debug_plan_blocks(int64_t R, int E, int64_t N, int pair);
/* number of matrix-core grouped GEMM launches this process has enqueued so far (any entry point): tests read it before
 * and after a call to tell that a shape ran on the matrix cores and not on the generic fallback kernels */
int64_t moe_gemm_debug_launch_count(void);
int moe_gemm_debug_plan(const void* offsets, int off64, int E, int64_t R, int64_t K, int64_t N, int pair, int nseg,
                        int32_t* out, void* stream);

/* ---- router: megablocks_utils/config_utils.py:255-280 (forward_router) ------------------------------------
 * logits[t][e] = sum_k x[t][k] * wg[e][k]  (config_utils.py:262, F.linear), fp32 accumulate and fp32 output. */
int moe_router_logits(const void* x, int64_t ldx, const void* wg, int64_t ldw, int dtype, float* logits,
                      int64_t ntok, int64_t d, int E, void* stream);
/* softmax over E (config_utils.py:262) -> top-k, ties to the lower expert id (config_utils.py:263) -> optional
 * division by the sum of the selected scores (config_utils.py:264-270).  scores (T,E), topw (T,k) fp32, topi (T,k) int32. */
int moe_router_topk(const float* logits, float* scores, float* topw, int32_t* topi, int64_t ntok, int E, int k,
                    int renorm, void* stream);
/* both of the above in one call (config_utils.py:262-270): logits (T,E), scores (T,E), topw (T,k), topi (T,k); a single
 * launch when x and the router weight are a 2-byte type, E <= 8 and d is a multiple of 32 (logits on the matrix cores,
 * eight partial sums per logit added in a fixed order: the same top-k indices as moe_router_logits + moe_router_topk,
 * logits equal to theirs up to fp32 rounding, not bit for bit), the two kernels of those entry points otherwise. */
int moe_router_forward(const void* x, int64_t ldx, const void* wg, int64_t ldw, int dtype, float* logits, float* scores,
                       float* topw, int32_t* topi, int64_t ntok, int64_t d, int E, int k, int renorm, void* stream);
/* gradient of moe_router_topk with respect to the logits given d(topw); the reference obtains it from autograd. */
int moe_router_topk_bwd(const float* dtopw, const float* topw, const int32_t* topi, const float* scores,
                        float* dlogits, int64_t ntok, int E, int k, int renorm, void* stream);

/* gradient of the router weight: dwg[e][c] = sum_t dlogits[t][e] * x[t][c] (autograd of the F.linear at
 * config_utils.py:262), from the fp32 dlogits with fp32 accumulation and a fixed summation order; dwg (E, d) in x's
 * dtype.  The gradient with respect to the router's input, dlogits @ wg, is moe_combine with k = 0 and the dense
 * tail (extra_coef = dlogits, extra_rows = wg). */
size_t moe_router_weight_grad_workspace_bytes(int64_t ntok, int64_t d, int E);
int moe_router_weight_grad(const void* x, int64_t ldx, const float* dlogits, void* dwg, int64_t ldo, int64_t ntok,
                           int64_t d, int E, int dtype, void* workspace, size_t workspace_bytes, void* stream);

/* ---- expert-grouped order: flatten_and_sort / histogram / cumsum / padded_block_indices ----------------------
 * Call sites: config_utils.py:114-118 (padded_block_indices), :131-132 (bin_ids, indices from megablocks'
 * stable radix sort), tests/test_scattermoe.py:84-85,161-163; block semantics scattermoe_utils/kernels/ops.py:39-51.
 * expert_idx: R flattened assignments (position t*k+j).  Outputs (any may be NULL except sorted_*):
 *   sorted_expert[i], sorted_pos[i]  stable ascending sort by expert id (width chosen by out64)
 *   counts[e], offsets[e]            histogram and inclusive running sum (same width)
 *   padded_blocks[0..*num_padded)    block starts, block_m rows per block, blocks never straddle experts
 *   inv[p] (int32)                   position of flat assignment p in the sorted order
 * 1 <= E <= 4096, else MOE_ERR_BAD_ARG before anything is enqueued.  Ids outside [0, E) take no part in the order:
 * the valid entries fill the front of sorted_*, offsets[E-1] counts them, and what lies behind them in sorted_* is
 * left untouched (a caller that cannot rule such ids out pre-fills sorted_* with a sentinel). */
size_t moe_sort_workspace_bytes(int64_t R, int E);
int moe_sort_by_expert(const void* expert_idx, int in64, int64_t R, int E, int block_m, void* sorted_expert,
                       void* sorted_pos, int out64, void* counts, void* offsets, void* padded_blocks,
                       int64_t padded_cap, int32_t* num_padded, int32_t* inv, void* workspace, size_t workspace_bytes,
                       void* stream);
/* moe_sort_by_expert for callers that cannot allocate (code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc).  No counterpart in the reference.  Same arguments, results and kernels as
 * moe_sort_by_expert minus the workspace: the per-chunk histograms live in a static device array of the library,
 * moe_sort_static_max_bytes() = 1 MiB per GPU, held until the process ends.  Limit: moe_sort_workspace_bytes(R, E)
 * = (ceil(R / 512) * E + 4) * 4 bytes must fit in it (e.g. R <= 16.7 M assignments at E = 8), otherwise
 * MOE_ERR_WORKSPACE and nothing is enqueued.  Calls no hipMalloc / hipFree and no allocating routine.  All calls on
 * one GPU share that GPU's array: calls that overlap on one GPU (two streams, two threads) race; calls on one stream
 * are ordered.  The first call on a device looks the array's address up (hipGetSymbolAddress) -- make that call
 * outside stream capture. */
size_t moe_sort_static_max_bytes(void);
int moe_sort_by_expert_static(const void* expert_idx, int in64, int64_t R, int E, int block_m, void* sorted_expert,
                              void* sorted_pos, int out64, void* counts, void* offsets, void* padded_blocks,
                              int64_t padded_cap, int32_t* num_padded, int32_t* inv, void* stream);
/* offsets[e] = #{i : sorted_expert[i] <= e}  (the expert_offsets consumed at ops.py:315-319) */
int moe_expert_offsets(const void* sorted_expert, int in64, int64_t R, int E, void* offsets, int out64, void* stream);
/* padded_block_indices from the inclusive offsets (ops.py:39-51) */
int moe_padded_block_indices(const void* offsets, int off64, int E, int block_m, void* padded_blocks, int out64,
                             int64_t cap, int32_t* num_padded, void* stream);

/* ---- scatter2scatter(_lora): scattermoe_utils/kernels/ops.py:156-212 (wrapper), :19-150 (kernel) ------------
 * For every sorted position m (expert e from `offsets`):
 *   Y[out_row] = X[in_row] @ (W[e] + scaling * A[e] @ B[e]),  in_row = x_grouped ? m : pos[m] / fan_out,
 *   out_row = y_grouped ? m : pos[m].   A == NULL selects the plain (no adapter) product.
 * W (E,K,N), A (E,K,rank), B (E,rank,N), arbitrary strides.  R = number of sorted positions. */
size_t moe_scatter2scatter_workspace_bytes(int64_t R, int E, int64_t K, int64_t N, int rank);
int moe_scatter2scatter(const void* X, int64_t sxm, int64_t sxk, const void* W, int64_t swe, int64_t swk, int64_t swn,
                        const void* A, int64_t sae, int64_t sak, int64_t sar, const void* B, int64_t sbe, int64_t sbr,
                        int64_t sbn, int rank, float scaling, void* Y, int64_t sym, int64_t syn, const void* pos,
                        int pos64, const void* offsets, int off64, int E, int64_t R, int64_t K, int64_t N, int fan_out,
                        int x_grouped, int y_grouped, int dtype, void* workspace, size_t workspace_bytes, void* stream);

/* ---- group_bwd_AB: scattermoe_utils/kernels/ops.py:220-255, definition :284-289 ------------------------------
 * DA[e] = scaling * X_e^T (DY_e B[e]^T),  DB[e] = scaling * (X_e A[e])^T DY_e over the rows of group e (full
 * reductions over N and K), zero for empty groups.  X (R,K) and DY (R,N) in grouped order. */
size_t moe_group_bwd_ab_workspace_bytes(int64_t R, int E, int64_t K, int64_t N, int rank, int dtype);
int moe_group_bwd_ab(const void* DY, int64_t sdm, int64_t sdn, const void* X, int64_t sxm, int64_t sxk, const void* A,
                     int64_t sae, int64_t sak, int64_t sar, const void* B, int64_t sbe, int64_t sbr, int64_t sbn,
                     int rank, float scaling, void* DA, int64_t sdae, int64_t sdak, int64_t sdar, void* DB,
                     int64_t sdbe, int64_t sdbr, int64_t sdbn, const void* offsets, int off64, int E, int64_t R,
                     int64_t K, int64_t N, int dtype, void* workspace, size_t workspace_bytes, void* stream);

/* ---- group_bwd_W: scattermoe.kernels.ops.group_bwd_W (selected at config_utils.py:124-125) -------------------
 * DW[e] = X_e^T DY_e over the R grouped rows; zeros for an empty expert.  bf16 operands with unit column strides run
 * on the matrix cores, everything else on the generic kernel. */
int moe_group_bwd_w(const void* DY, int64_t sdm, int64_t sdn, const void* X, int64_t sxm, int64_t sxk, void* DW,
                    int64_t swe, int64_t swk, int64_t swn, const void* offsets, int off64, int E, int64_t R, int64_t K,
                    int64_t N, int dtype, void* stream);

/* ---- group: scattermoe.kernels.ops.group, call sites scattermoe_utils/parallel_linear_lora.py:87-91,98 --------
 * out[i] = src[pos[i] / fan_out] * coeff[pos[i]]   (coeff may be NULL) */
int moe_group_rows(const void* src, int64_t lds, void* out, int64_t ldo, const void* pos, int pos64, int fan_out,
                   const void* coeff, int coeff_dtype, int64_t nrows, int64_t ncols, int dtype, void* stream);

/* ---- weighted combine: the gates bmm of parallel_linear_lora.py:30-35 / megablocks ops.scatter (config_utils.py:251)
 * out[t] = sum_j gates[t*k+j] * y[row(t,j)] (+ sum_e extra_coef[t][e] * extra_rows[e]),
 * row(t,j) = inv ? inv[t*k+j] : t*k+j; gates == NULL means 1 (the fan-out sum of parallel_linear_lora.py:134);
 * k == 0 (y may be NULL) leaves only the dense tail. */
int moe_combine(const void* y, int64_t ldy, void* out, int64_t ldo, const void* gates, int gates_dtype,
                const int32_t* inv, int k, int64_t ntok, int64_t ncols, int dtype, const float* extra_coef,
                const void* extra_rows, int64_t lde, int n_extra, void* stream);
/* d_gates[t*k+j] = <y[row(t,j)], dout[t]>   (parallel_linear_lora.py:70-72) */
int moe_combine_dgates(const void* y, int64_t ldy, const void* dout, int64_t ldd, void* dgates, int gates_dtype,
                       const int32_t* inv, int k, int64_t ntok, int64_t ncols, int dtype, void* stream);

/* ---- SwiGLU: F.silu(h1) * h3 at config_utils.py:151 and its autograd backward -------------------------------- */
int moe_swiglu(const void* gate, const void* up, void* h, int64_t n, int dtype, void* stream);
int moe_swiglu_bwd(const void* gate, const void* up, const void* dh, void* dgate, void* dup, int64_t n, int dtype,
                   void* stream);

/* ---- fused expert MLP: scattermoe_permute_and_compute, config_utils.py:99-185 ---------------------------------
 * bf16 or fp16 (`dtype`; the reference's `bf16` / `fp16` switches, megablocks_utils/shard_moe_utils.py:29-30,43-44), every
 * tensor of a call in that one type.  Weights in the reference's storage layout (sparse_mlp2.py:22-36 viewed as config_utils.py:31):
 * w1, w3, w2 each (E, f, d) contiguous.  Adapters as the strided views of config_utils.py:48-56:
 * a1,a3 (E,d,r)  b1,b3 (E,r,f)  a2 (E,f,r)  b2 (E,r,d), strides {expert, second dim, third dim} in lora_strides[6][3]
 * (order a1,b1,a3,b3,a2,b2); all NULL = no adapters.
 * Forward:  gate = x W1^T (+lora), up = x W3^T (+lora)   [one dual-weight GEMM, x gathered by pos/fan_out]
 *           h = silu(gate) * up                          [fused epilogue; gate/up saved when save_gate_up]
 *           y[out_row] = h W2 (+lora)                    [out_row = y_grouped ? m : pos[m]]
 * `saved` receives the low-rank interims needed by the backward (moe_mlp_saved_bytes).  Adapter rank <= 128 (an adapter is
 * worked through as up to eight chunks of 16 rank columns; one chunk has its products with h, dgate and dup folded into
 * the GEMM epilogues, more chunks take separate passes over those tensors); higher ranks: use the per-projection entry points. */
size_t moe_mlp_workspace_bytes(int64_t R, int E, int64_t d, int64_t f, int rank);
size_t moe_mlp_saved_bytes(int64_t R, int rank);
int moe_mlp_fwd(const void* x, int64_t ldx, const void* w1, const void* w3, const void* w2, const void* const* lora,
                const int64_t* lora_strides, int rank, float scaling, void* gate, void* up, void* h, void* y,
                int64_t ldy, const void* pos, int pos64, const void* offsets, int off64, int E, int64_t R, int64_t d,
                int64_t f, int fan_out, int y_grouped, int dtype, void* saved, void* workspace, size_t workspace_bytes,
                void* stream);
/* Backward of moe_mlp_fwd.  dy rows are addressed like y rows: row = dy_grouped ? m : pos[m] / dy_fan_out, and are
 * multiplied by row_scale[m] (fp32, may be NULL) -- this folds the combine's gate weights into the GEMM.
 * Outputs: dx_rows (R, d) written to row pos[m] (or m when dx_grouped), one row per assignment (the caller sums
 * the fan-out); adapter gradients in lora_grads (same order/strides convention as `lora`, same dtype). */
int moe_mlp_bwd(const void* dy, int64_t lddy, int dy_grouped, int dy_fan_out, const float* row_scale, const void* x,
                int64_t ldx, const void* w1, const void* w3, const void* w2, const void* const* lora,
                const int64_t* lora_strides, void* const* lora_grads, const int64_t* lora_grad_strides, int rank,
                float scaling, const void* gate, const void* up, const void* h, void* dgate, void* dup, void* dx_rows,
                int64_t lddx, int dx_grouped, const void* pos, int pos64, const void* offsets, int off64, int E,
                int64_t R, int64_t d, int64_t f, int fan_out, int dtype, const void* saved, void* workspace,
                size_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MOE_HIP_H */
