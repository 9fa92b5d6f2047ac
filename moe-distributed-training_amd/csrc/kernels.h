// Internal launcher interface between the kernel translation units and the C-ABI layer (moe_abi.hip).
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

// epilogues of the MFMA grouped GEMM
#define MOE_EPI_STORE 0        // Y0[out_row][n] = acc
#define MOE_EPI_SWIGLU 1       // weight pair (gate, up): Y0 = silu(gate)*up, optional Y1 = gate, Y2 = up (grouped rows)
#define MOE_EPI_SWIGLU_BWD 2   // acc = dh: Y0 = dgate, Y1 = dup from saved gate (H1) and up (H3)
#define MOE_EPI_SWIGLU_FUSED 4   // as MOE_EPI_SWIGLU, and the product of h with an adapter factor per column tile (CB[0] -> CCP[0], ncc = 1)
#define MOE_EPI_SWIGLU_BWD_FUSED 3   // ... and the low-rank products of dgate, dup and h that the adapters' backward needs (RC / CB below)

constexpr int MOE_MAX_SLABS = 4;            // slabs given by their own pointers
constexpr int MOE_MAX_STRIDED_SLABS = 16;   // slabs of a plain-epilogue launch laid out at a fixed stride (adapter rank up to 256)

struct MoeGemmParams {
    const uint16_t* X[2];   // A-operand segments, rows of K bf16, unit k stride
    int64_t ldx;
    int nseg;               // 1 or 2 K segments (X[s] x W[s]) accumulated into the same tile
    const uint16_t* W[2];   // weights; for MOE_EPI_SWIGLU W[0] = gate projection, W[1] = up projection
    int64_t swe;            // expert stride (elements)
    int64_t ldw;            // nn == 0: stride between n rows (k contiguous); nn == 1: stride between k rows (n contiguous)
    int nn;
    const uint16_t* Q[MOE_MAX_SLABS];   // low-rank A-side operands [R][16] bf16 in grouped order (already scaled)
    const uint16_t* LB[MOE_MAX_SLABS];  // low-rank B-side operands [E][N][16] bf16
    int nslab;              // 0..MOE_MAX_SLABS 16-wide K slabs (a rank-r adapter is ceil(r/16) slabs); more (up to MOE_MAX_STRIDED_SLABS, plain
                            // epilogue, slab_mode 0): slab s is Q[0] + s * q_slab_stride, LB[0] + s * lb_slab_stride
    int64_t q_slab_stride, lb_slab_stride;   // elements
    int slab_mode;          // 0: every slab feeds every column; 1: the first half of the slabs feeds the gate weight of the SwiGLU pair, the second half the up weight
    uint16_t* Y[3];
    int64_t ldy;
    const uint16_t* H1;     // saved gate / up for MOE_EPI_SWIGLU_BWD
    const uint16_t* H3;
    int64_t ldh;
    // MOE_EPI_SWIGLU_BWD_FUSED only: row contractions (nrc = 3).  RC[i]: bf16 [R][16] operands in grouped order;
    // RCP[i]: fp32 partials [row tile][N][16], row tiles of 256 rows per expert in order (the layout the fixed-order
    // reduction of the adapter gradients sums): RCP[0] = dgate^T RC[0], RCP[1] = dup^T RC[1], RCP[2] = h^T RC[2]
    const uint16_t* RC[3];
    float* RCP[3];
    int nrc;
    // ... and column contractions (MOE_EPI_SWIGLU_BWD_FUSED: ncc = 2; MOE_EPI_SWIGLU_FUSED: ncc = 1, CCP[0] = h CB[0] per column tile of 128): CB[i]: adapter factor in fragment order [E][N/32][64][8];
    // CCP[i]: fp32 partials [column tile of 256][cc_rows][16]: CCP[0] = dgate CB[0], CCP[1] = dup CB[1] over the tile's columns
    const uint16_t* CB[2];
    float* CCP[2];
    int ncc;
    int64_t cc_rows;
    const float* row_scale; // optional per sorted position factor applied to the accumulator (STORE, SWIGLU_BWD)
    const void* pos;        // sorted_scattered_idxs
    int pos64;
    const void* offsets;    // inclusive expert offsets
    int off64;
    int E;
    int64_t K;              // per segment
    int64_t N;
    int fan_out;
    int x_grouped;
    int y_grouped;
    int epi;
    int f16;                // operands and outputs are IEEE half instead of bfloat16
    int y_wide;             // scattered output rows need 64-bit addresses (Y spans 2 GiB or more), set by the launcher
    int max_split;          // K parts a tile of the last round may be cut into (1, 2 or 4), set by the launcher
    int num_cus;            // compute units the tile plan fills (a multiple of 8), set by the launcher
    float* sk_partials;     // K-split exchange area, see moe_gemm_sk_bytes / moe_gemm_sk_attach
    int* sk_counters;
    int counters_clean;     // the caller guarantees sk_counters is all zero at launch (every launch leaves it so)
};

size_t moe_gemm_sk_bytes(int64_t R, int E, int64_t N);
void moe_gemm_sk_attach(MoeGemmParams& p, void* ws, int64_t R, int E, int64_t N);
int moe_gemm_max_split(bool pair);
int moe_gemm_num_counters();   // ints at the start of the exchange area that must be zero at launch
// test aid: workgroups of a launch with this geometry, and each workgroup's work item (9 ints per workgroup)
int64_t moe_gemm_plan_blocks(int64_t R, int E, int64_t N, int pair);
int moe_launch_gemm_plan(const void* offsets, int off64, int E, int64_t R, int64_t K, int64_t N, int pair, int nseg, int* out,
                         hipStream_t stream);
size_t moe_gemm_sk_bytes(int64_t R, int E, int64_t N);
void moe_gemm_sk_attach(MoeGemmParams& p, void* ws, int64_t R, int E, int64_t N);
bool moe_gemm_mfma_supported(const MoeGemmParams& p, int64_t R);
int moe_launch_gemm_mfma(const MoeGemmParams& p, int64_t R, hipStream_t stream);
int64_t moe_gemm_mfma_launch_count();   // test aid: matrix-core grouped GEMM launches enqueued by this process so far

// weight gradient DW[e] = X_e^T DY_e on the matrix cores (bf16; unit column strides)
struct MoeXtyParams {
    const uint16_t* X;      // [R][K] grouped rows
    int64_t ldx;
    const uint16_t* DY;     // [R][N] grouped rows
    int64_t ldy;
    uint16_t* DW;           // [E][K][N]
    int64_t swe, ldw;       // expert stride, stride between k rows (elements)
    const void* offsets;    // inclusive expert offsets
    int off64;
    int E;
    int64_t K, N;
    int f16;                // operands and output are IEEE half instead of bfloat16
};
bool moe_xty_mfma_supported(const MoeXtyParams& p, int64_t R);
int moe_launch_xty_mfma(const MoeXtyParams& p, int64_t R, hipStream_t stream);

int moe_launch_generic_gemm(const void* X, int64_t sxm, int64_t sxk, const void* W, int64_t swe, int64_t swk,
                            int64_t swn, const void* A, int64_t sae, int64_t sak, int64_t sar, const void* B,
                            int64_t sbe, int64_t sbr, int64_t sbn, void* Y, int64_t sym, int64_t syn, const void* pos,
                            int pos64, const void* offsets, int off64, int E, int64_t R, int64_t K, int64_t N, int rank,
                            int fan_out, float scaling, int x_grouped, int y_grouped, int dtype, hipStream_t stream);
int moe_launch_generic_xty(const void* X, int64_t sxm, int64_t sxk, const void* Yp, int64_t sym, int64_t syn, void* O,
                           int64_t soe, int64_t sok, int64_t son, const void* offsets, int off64, int E, int64_t K,
                           int64_t N, float scale, int dtype, hipStream_t stream);

// low-rank helpers (16-bit storage: bf16, or IEEE half when f16 != 0; rank <= 16)
// a batch of pack jobs sharing E: src strides {expert, k, r}, dst as moe_launch_pack_lora
constexpr int MOE_PACK_MAX_JOBS = 12;
struct MoePackJob { const uint16_t* src; int64_t se, sk, sr; uint16_t* dst; int64_t K; int transpose; int rank; };   // rank <= 16 columns, zero padded to 16
struct MoePackBatch { MoePackJob job[MOE_PACK_MAX_JOBS]; int njobs; int E; int* zero_ptr; int zero_n; };   // zero_ptr[0..zero_n) is cleared by the launch
int moe_launch_pack_lora_batch(const MoePackBatch& jobs, hipStream_t stream);
int moe_launch_pack_lora(const void* src, int64_t se, int64_t sk, int64_t sr, void* dst, int E, int64_t K, int rank,
                         int transpose, hipStream_t stream);
int moe_launch_rows_lora(const void* X, int64_t ldx, const void* At, void* Q, void* Qt, int64_t ldqt, const void* pos,
                         int pos64, const void* offsets, int off64, int E, int64_t R, int64_t K, int fan_out,
                         int x_grouped, float scaling, const float* qt_row_scale, hipStream_t stream, int f16 = 0);
// two products over the same rows in one launch (X2 == nullptr: only the first)
// q_scaled (optional): a third output of the first product, [R][16] like Q but multiplied by qt_row_scale like Qt
int moe_launch_rows_lora2(const void* X, const void* X2, int64_t ldx, const void* At, const void* At2, void* Q, void* Q2,
                          void* Qt, void* Qt2, int64_t ldqt, const void* pos, int pos64, const void* offsets, int off64,
                          int E, int64_t R, int64_t K, int fan_out, int x_grouped, float scaling,
                          const float* qt_row_scale, hipStream_t stream, void* q_scaled = nullptr, int f16 = 0);
size_t moe_xtp_workspace_bytes(int64_t R, int E, int64_t K);
// Q[m][r] = bf16(scaling * sum over ntiles column-tile partials [ntiles][R][16]) and its transposed copy Qt[r][m], for one or
// two products (partial2 == nullptr: one)
int moe_launch_cc_reduce2(const float* partial, const float* partial2, int ntiles, int64_t R, float scaling, void* Q, void* Q2,
                          void* Qt, void* Qt2, int64_t ldqt, hipStream_t stream, int f16 = 0);
// the reduction half of moe_launch_xtp2 alone, for partials [row tile of 256][K][16] that another kernel produced
// (partial2 == nullptr: only the first)
int moe_launch_xtp_reduce2(const float* partial, const float* partial2, void* out, void* out2, const int64_t* so,
                           const int64_t* so2, int rank, int rank2, const void* offsets, int off64, int E, int64_t K,
                           float scale, hipStream_t stream, int f16 = 0);
// two reductions over the same rows in one launch pair (X2 == nullptr: only the first); so / so2: output strides
// {expert, k, r}; rank / rank2: columns each writes; needs twice moe_xtp_workspace_bytes when X2 is given
int moe_launch_xtp2(const void* X, const void* X2, int64_t ldx, const void* pos, int pos64, int fan_out, const void* Pt,
                    const void* Pt2, int64_t ldpt, const float* p_row_scale, void* out, void* out2, const int64_t* so,
                    const int64_t* so2, int rank, int rank2, const void* offsets, int off64, int E, int64_t R, int64_t K,
                    float scale, void* workspace, size_t workspace_bytes, hipStream_t stream, int f16 = 0);
int moe_launch_xtp(const void* X, int64_t ldx, const void* pos, int pos64, int fan_out, const void* Pt, int64_t ldpt,
                   const float* p_row_scale, void* out, int64_t soe, int64_t sok, int64_t sor, int rank,
                   const void* offsets, int off64, int E, int64_t R, int64_t K, float scale, void* workspace,
                   size_t workspace_bytes, hipStream_t stream, int f16 = 0);

// router + integer pipeline
int moe_launch_router_logits(const void* x, int64_t ldx, const void* wg, int64_t ldw, int dtype, float* logits,
                             int64_t ntok, int64_t d, int E, hipStream_t stream);
int moe_launch_router_forward(const void* x, int64_t ldx, const void* wg, int64_t ldw, int dtype, float* logits,
                              float* scores, float* topw, int32_t* topi, int64_t ntok, int64_t d, int E, int k,
                              int renorm, hipStream_t stream);
int moe_launch_router_topk(const float* logits, float* scores, float* topw, int32_t* topi, int64_t ntok, int E, int k,
                           int renorm, hipStream_t stream);
int moe_launch_router_bwd(const float* dw, const float* w, const int32_t* topi, const float* scores, float* dlogits,
                          int64_t ntok, int E, int k, int renorm, hipStream_t stream);
size_t moe_router_wgrad_ws_bytes(int64_t ntok, int64_t d, int E);
int moe_launch_router_wgrad(const void* x, int64_t ldx, const float* dlogits, void* dwg, int64_t ldo, int64_t ntok,
                            int64_t d, int E, int dtype, void* workspace, size_t workspace_bytes, hipStream_t stream);
size_t moe_sort_ws_bytes(int64_t R, int E);
int moe_launch_sort(const void* expert_idx, int in64, int64_t R, int E, int block_m, void* sorted_expert,
                    void* sorted_pos, int out64, void* counts, void* offsets, void* padded_blocks, int64_t padded_cap,
                    int32_t* num_padded, int32_t* inv, void* workspace, size_t workspace_bytes, hipStream_t stream);
// the same sort with its per-chunk histograms in a static device array of the library (no workspace, no allocation)
size_t moe_sort_static_capacity_bytes();
int moe_launch_sort_static(const void* expert_idx, int in64, int64_t R, int E, int block_m, void* sorted_expert,
                           void* sorted_pos, int out64, void* counts, void* offsets, void* padded_blocks,
                           int64_t padded_cap, int32_t* num_padded, int32_t* inv, hipStream_t stream);
int moe_launch_offsets_from_sorted(const void* sorted_expert, int in64, int64_t R, int E, void* offsets, int out64,
                                   hipStream_t stream);
int moe_launch_padded_blocks(const void* offsets, int off64, int E, int block_m, void* padded_blocks, int out64,
                             int64_t cap, int32_t* num_padded, hipStream_t stream);

// row kernels
int moe_launch_group_rows(const void* src, int64_t lds_, void* out, int64_t ldo, const void* pos, int pos64,
                          int fan_out, const void* coeff, int cdtype, int64_t nrows, int64_t ncols, int dtype,
                          hipStream_t stream);
int moe_launch_combine_fwd(const void* y, int64_t ldy, void* out, int64_t ldo, const void* gates, int gdtype,
                           const int32_t* inv, int k, int64_t ntok, int64_t ncols, int dtype,
                           const float* extra_coef, const void* extra_rows, int64_t lde, int n_extra,
                           hipStream_t stream);
int moe_launch_combine_dgates(const void* y, int64_t ldy, const void* dout, int64_t ldd, void* dgates, int gdtype,
                              const int32_t* inv, int k, int64_t ntok, int64_t ncols, int dtype, hipStream_t stream);
int moe_launch_swiglu_fwd(const void* g, const void* u, void* h, int64_t n, int dtype, hipStream_t stream);
int moe_launch_swiglu_bwd(const void* g, const void* u, const void* dh, void* dg, void* du, int64_t n, int dtype,
                          hipStream_t stream);
