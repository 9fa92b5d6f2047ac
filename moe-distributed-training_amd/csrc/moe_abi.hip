// C-ABI layer of libmoe_hip.so: argument checks, kernel selection (matrix-core path vs generic path) and the
// launch sequences of the composite operations.  Declarations and their contracts: include/moe_hip.h.
#include "../../include/moe_hip.h"
#include "common.h"
#include "kernels.h"
#include <mutex>
#include <string>
#include <string.h>
#include <vector>

namespace {

// Optional stage timer (off by default): when enabled, every kernel group enqueued by an entry point is bracketed
// by a pair of events on the caller's stream, so a harness can read per-stage device times of the very launches it
// timed as a whole.  Not used on the normal path.
struct ProfRec { const char* name; hipEvent_t a, b; };
std::mutex g_prof_mu;
bool g_prof_on = false;
std::string g_prof_select;   // comma-separated substrings; empty = every stage
std::vector<ProfRec> g_prof;
std::vector<hipEvent_t> g_prof_pool;

struct Timed {
    hipStream_t st; hipEvent_t b; bool on;
    Timed(hipStream_t s, const char* name) : st(s), b(nullptr), on(false) {
        std::lock_guard<std::mutex> lk(g_prof_mu);
        if (!g_prof_on) return;
        if (!g_prof_select.empty()) {   // only the selected stages are bracketed
            bool hit = false;
            size_t a = 0;
            while (a <= g_prof_select.size() && !hit) {
                size_t b = g_prof_select.find(',', a);
                if (b == std::string::npos) b = g_prof_select.size();
                if (b > a && strstr(name, g_prof_select.substr(a, b - a).c_str())) hit = true;
                a = b + 1;
            }
            if (!hit) return;
        }
        hipEvent_t ev[2];
        for (int i = 0; i < 2; ++i) {
            if (!g_prof_pool.empty()) { ev[i] = g_prof_pool.back(); g_prof_pool.pop_back(); }
            else if (hipEventCreate(&ev[i]) != hipSuccess) return;
        }
        g_prof.push_back({name, ev[0], ev[1]});
        b = ev[1]; on = true;
        (void)hipEventRecord(ev[0], st);
    }
    ~Timed() { if (on) (void)hipEventRecord(b, st); }
};
#define TIMED(name) Timed _timed_scope(st, name)

inline hipStream_t S(void* s) { return (hipStream_t)s; }
inline size_t al(size_t n) { return (n + 255) & ~(size_t)255; }
inline int64_t pad_rows(int64_t R) { return (R + 31) / 32 * 32 + 32; }

struct Bump {
    uint8_t* base; size_t size; size_t used;
    Bump(void* p, size_t n) : base((uint8_t*)p), size(n), used(0) {}
    void* take(size_t n) { void* r = base + used; used += al(n); return used <= size ? r : nullptr; }
};

inline bool aligned16(const void* p) { return ((uintptr_t)p % 16) == 0; }

#define TRY(expr) do { int _s = (expr); if (_s != MOE_OK) return _s; } while (0)

// sizes of the packed adapter images and low-rank interims
inline size_t pack_bytes(int E, int64_t K) { return al((size_t)E * 16 * (size_t)((K + 31) / 32 * 32) * 2); }   // fragment-order images cover K rounded up to 32
inline size_t q_bytes(int64_t R) { return al((size_t)pad_rows(R) * 16 * 2); }

}  // namespace

extern "C" {

int moe_hip_abi_version(void) { return MOE_HIP_ABI_VERSION; }

int moe_profile_enable(int on)
{
    std::lock_guard<std::mutex> lk(g_prof_mu);
    for (auto& r : g_prof) { g_prof_pool.push_back(r.a); g_prof_pool.push_back(r.b); }
    g_prof.clear();
    g_prof_on = on != 0;
    return MOE_OK;
}

int moe_profile_select(const char* substrings)
{
    std::lock_guard<std::mutex> lk(g_prof_mu);
    g_prof_select = substrings ? substrings : "";
    return MOE_OK;
}

int moe_profile_count(void)
{
    std::lock_guard<std::mutex> lk(g_prof_mu);
    return (int)g_prof.size();
}

int moe_profile_get(int i, char* name, int name_cap, float* ms)
{
    std::lock_guard<std::mutex> lk(g_prof_mu);
    if (i < 0 || i >= (int)g_prof.size() || !name || name_cap < 1 || !ms) return MOE_ERR_BAD_ARG;
    if (hipEventSynchronize(g_prof[i].b) != hipSuccess) return MOE_ERR_LAUNCH;
    if (hipEventElapsedTime(ms, g_prof[i].a, g_prof[i].b) != hipSuccess) return MOE_ERR_LAUNCH;
    strncpy(name, g_prof[i].name, (size_t)name_cap - 1);
    name[name_cap - 1] = 0;
    return MOE_OK;
}

const char* moe_hip_strerror(int status)
{
    switch (status) {
    case MOE_OK: return "ok";
    case MOE_ERR_BAD_ARG: return "bad argument";
    case MOE_ERR_UNSUPPORTED: return "unsupported combination";
    case MOE_ERR_WORKSPACE: return "workspace too small";
    case MOE_ERR_LAUNCH: return "HIP launch error";
    default: return "unknown status";
    }
}

int moe_router_logits(const void* x, int64_t ldx, const void* wg, int64_t ldw, int dtype, float* logits, int64_t ntok,
                      int64_t d, int E, void* stream)
{
    if (ntok < 0 || d < 1 || E < 1) return MOE_ERR_BAD_ARG;
    if (ntok == 0) return MOE_OK;
    if (!x || !wg || !logits) return MOE_ERR_BAD_ARG;
    return moe_launch_router_logits(x, ldx, wg, ldw, dtype, logits, ntok, d, E, S(stream));
}

int moe_router_topk(const float* logits, float* scores, float* topw, int32_t* topi, int64_t ntok, int E, int k,
                    int renorm, void* stream)
{
    if (ntok < 0 || E < 1 || k < 1 || k > E) return MOE_ERR_BAD_ARG;
    if (ntok == 0) return MOE_OK;
    if (!logits || !scores || !topw || !topi) return MOE_ERR_BAD_ARG;
    return moe_launch_router_topk(logits, scores, topw, topi, ntok, E, k, renorm, S(stream));
}

int moe_router_forward(const void* x, int64_t ldx, const void* wg, int64_t ldw, int dtype, float* logits, float* scores,
                       float* topw, int32_t* topi, int64_t ntok, int64_t d, int E, int k, int renorm, void* stream)
{
    if (ntok < 0 || d < 1 || E < 1 || k < 1 || k > E) return MOE_ERR_BAD_ARG;
    if (ntok == 0) return MOE_OK;
    if (!x || !wg || !logits || !scores || !topw || !topi) return MOE_ERR_BAD_ARG;
    hipStream_t st = S(stream);
    TIMED("route.router_forward");
    return moe_launch_router_forward(x, ldx, wg, ldw, dtype, logits, scores, topw, topi, ntok, d, E, k, renorm, st);
}

int moe_router_topk_bwd(const float* dtopw, const float* topw, const int32_t* topi, const float* scores,
                        float* dlogits, int64_t ntok, int E, int k, int renorm, void* stream)
{
    if (ntok < 0 || E < 1 || k < 1 || k > E) return MOE_ERR_BAD_ARG;
    if (ntok == 0) return MOE_OK;
    if (!dtopw || !topw || !topi || !scores || !dlogits) return MOE_ERR_BAD_ARG;
    hipStream_t st = S(stream);
    TIMED("route.router_bwd");
    return moe_launch_router_bwd(dtopw, topw, topi, scores, dlogits, ntok, E, k, renorm, st);
}

size_t moe_router_weight_grad_workspace_bytes(int64_t ntok, int64_t d, int E) { return moe_router_wgrad_ws_bytes(ntok, d, E); }

int moe_router_weight_grad(const void* x, int64_t ldx, const float* dlogits, void* dwg, int64_t ldo, int64_t ntok,
                           int64_t d, int E, int dtype, void* workspace, size_t workspace_bytes, void* stream)
{
    if (ntok < 0 || d < 1 || E < 1 || !dwg || !workspace || (ntok > 0 && (!x || !dlogits))) return MOE_ERR_BAD_ARG;
    hipStream_t st = S(stream);
    TIMED("route.router_weight_grad");
    return moe_launch_router_wgrad(x, ldx, dlogits, dwg, ldo, ntok, d, E, dtype, workspace, workspace_bytes, st);
}

size_t moe_sort_workspace_bytes(int64_t R, int E) { return moe_sort_ws_bytes(R, E); }

int moe_sort_by_expert(const void* expert_idx, int in64, int64_t R, int E, int block_m, void* sorted_expert,
                       void* sorted_pos, int out64, void* counts, void* offsets, void* padded_blocks,
                       int64_t padded_cap, int32_t* num_padded, int32_t* inv, void* workspace, size_t workspace_bytes,
                       void* stream)
{
    if ((R > 0 && (!expert_idx || !sorted_expert || !sorted_pos)) || !workspace) return MOE_ERR_BAD_ARG;
    if (R >= (int64_t)1 << 31) return MOE_ERR_UNSUPPORTED;
    hipStream_t st = S(stream);
    TIMED("route.sort");
    return moe_launch_sort(expert_idx, in64, R, E, block_m, sorted_expert, sorted_pos, out64, counts, offsets,
                           padded_blocks, padded_cap, num_padded, inv, workspace, workspace_bytes, st);
}

size_t moe_sort_static_max_bytes(void) { return moe_sort_static_capacity_bytes(); }

int moe_sort_by_expert_static(const void* expert_idx, int in64, int64_t R, int E, int block_m, void* sorted_expert,
                              void* sorted_pos, int out64, void* counts, void* offsets, void* padded_blocks,
                              int64_t padded_cap, int32_t* num_padded, int32_t* inv, void* stream)
{
    if (R > 0 && (!expert_idx || !sorted_expert || !sorted_pos)) return MOE_ERR_BAD_ARG;
    if (R >= (int64_t)1 << 31) return MOE_ERR_UNSUPPORTED;
    return moe_launch_sort_static(expert_idx, in64, R, E, block_m, sorted_expert, sorted_pos, out64, counts, offsets,
                                  padded_blocks, padded_cap, num_padded, inv, S(stream));
}

int moe_expert_offsets(const void* sorted_expert, int in64, int64_t R, int E, void* offsets, int out64, void* stream)
{
    if ((R > 0 && !sorted_expert) || !offsets || E < 1) return MOE_ERR_BAD_ARG;
    return moe_launch_offsets_from_sorted(sorted_expert, in64, R, E, offsets, out64, S(stream));
}

int moe_padded_block_indices(const void* offsets, int off64, int E, int block_m, void* padded_blocks, int out64,
                             int64_t cap, int32_t* num_padded, void* stream)
{
    if (!offsets || !num_padded || block_m < 1 || E < 1) return MOE_ERR_BAD_ARG;
    return moe_launch_padded_blocks(offsets, off64, E, block_m, padded_blocks, out64, cap, num_padded, S(stream));
}

int64_t moe_gemm_debug_launch_count(void) { return moe_gemm_mfma_launch_count(); }

int64_t moe_gemm_debug_plan_blocks(int64_t R, int E, int64_t N, int pair) { return moe_gemm_plan_blocks(R, E, N, pair); }

int moe_gemm_debug_plan(const void* offsets, int off64, int E, int64_t R, int64_t K, int64_t N, int pair, int nseg,
                        int32_t* out, void* stream)
{
    if (!offsets || !out || E < 1 || R < 0 || K < 1 || N < 1) return MOE_ERR_BAD_ARG;
    return moe_launch_gemm_plan(offsets, off64, E, R, K, N, pair, nseg, out, S(stream));
}

// ---------------------------------------------------------------------------------------------------------
size_t moe_scatter2scatter_workspace_bytes(int64_t R, int E, int64_t K, int64_t N, int rank)
{
    const size_t sk = al(moe_gemm_sk_bytes(R, E, N));
    if (rank <= 0) return sk + 256;
    const size_t chunks = (size_t)(rank + 15) / 16;   // a rank above 16 runs as several adapters of rank <= 16
    return sk + chunks * (pack_bytes(E, K) + pack_bytes(E, N) + q_bytes(R)) + 256;
}

int moe_scatter2scatter(const void* X, int64_t sxm, int64_t sxk, const void* W, int64_t swe, int64_t swk, int64_t swn,
                        const void* A, int64_t sae, int64_t sak, int64_t sar, const void* B, int64_t sbe, int64_t sbr,
                        int64_t sbn, int rank, float scaling, void* Y, int64_t sym, int64_t syn, const void* pos,
                        int pos64, const void* offsets, int off64, int E, int64_t R, int64_t K, int64_t N, int fan_out,
                        int x_grouped, int y_grouped, int dtype, void* workspace, size_t workspace_bytes, void* stream)
{
    if (!X || !W || !Y || !offsets || E < 1 || R < 0 || K < 1 || N < 1 || fan_out < 1) return MOE_ERR_BAD_ARG;
    if ((!x_grouped || !y_grouped) && !pos) return MOE_ERR_BAD_ARG;
    if ((A == nullptr) != (B == nullptr)) return MOE_ERR_BAD_ARG;
    if (A && rank < 1) return MOE_ERR_BAD_ARG;
    if (R == 0) return MOE_OK;

    // matrix-core path: bf16 or fp16, unit inner strides, weights either K-contiguous (NT) or N-contiguous (NN)
    const bool nt = (swk == 1), nn = (swn == 1) && !nt;
    const bool two_byte = dtype == MOE_BF16 || dtype == MOE_F16;
    const int f16 = dtype == MOE_F16;
    if (two_byte && sxk == 1 && syn == 1 && (nt || nn) && (!A || rank <= 16 * MOE_MAX_STRIDED_SLABS)) {
        MoeGemmParams p = {};
        p.X[0] = (const uint16_t*)X; p.ldx = sxm; p.nseg = 1;
        p.W[0] = (const uint16_t*)W; p.swe = swe; p.ldw = nt ? swn : swk; p.nn = nn ? 1 : 0;
        p.Y[0] = (uint16_t*)Y; p.ldy = sym;
        p.pos = pos; p.pos64 = pos64; p.offsets = offsets; p.off64 = off64;
        p.E = E; p.K = K; p.N = N; p.fan_out = fan_out; p.x_grouped = x_grouped; p.y_grouped = y_grouped;
        p.epi = MOE_EPI_STORE; p.f16 = f16;
        bool ok = moe_gemm_mfma_supported(p, R);
        if (ok) {
            if (workspace_bytes < moe_scatter2scatter_workspace_bytes(R, E, K, N, A ? rank : 0) || !workspace)
                return MOE_ERR_WORKSPACE;
            Bump ws(workspace, workspace_bytes);
            moe_gemm_sk_attach(p, ws.take(moe_gemm_sk_bytes(R, E, N)), R, E, N);
            if (A) {
                // x A B = sum over 16-wide chunks c of x A[:, c] B[c, :]: a rank above 16 enters as several 16-wide K slabs
                const int nh = (rank + 15) / 16;
                void *At[MOE_MAX_STRIDED_SLABS] = {}, *LB[MOE_MAX_STRIDED_SLABS] = {}, *Q[MOE_MAX_STRIDED_SLABS] = {};
                for (int hf = 0; hf < nh; ++hf) {
                    At[hf] = ws.take(pack_bytes(E, K));
                    LB[hf] = ws.take(pack_bytes(E, N));
                    Q[hf] = ws.take(q_bytes(R));
                    const int r0 = 16 * hf, rk = (rank - r0 < 16) ? rank - r0 : 16;
                    TRY(moe_launch_pack_lora((const uint16_t*)A + r0 * sar, sae, sak, sar, At[hf], E, K, rk, 1, S(stream)));
                    TRY(moe_launch_pack_lora((const uint16_t*)B + r0 * sbr, sbe, sbn, sbr, LB[hf], E, N, rk, 0, S(stream)));
                    if (hf < MOE_MAX_SLABS) { p.Q[hf] = (const uint16_t*)Q[hf]; p.LB[hf] = (const uint16_t*)LB[hf]; }
                }
                for (int hf = 0; hf < nh; hf += 2)   // two products over the same rows per launch
                    TRY(moe_launch_rows_lora2(X, hf + 1 < nh ? X : nullptr, sxm, At[hf], hf + 1 < nh ? At[hf + 1] : nullptr, Q[hf],
                                              hf + 1 < nh ? Q[hf + 1] : nullptr, nullptr, nullptr, 0, pos, pos64, offsets, off64, E, R, K,
                                              fan_out, x_grouped, scaling, nullptr, S(stream), nullptr, f16));
                p.nslab = nh; p.slab_mode = 0;
                if (nh > 1) {   // the chunks' buffers were taken in turn: a fixed stride from one chunk to the next
                    p.q_slab_stride = (int64_t)((const uint16_t*)Q[1] - (const uint16_t*)Q[0]);
                    p.lb_slab_stride = (int64_t)((const uint16_t*)LB[1] - (const uint16_t*)LB[0]);
                }
            }
            return moe_launch_gemm_mfma(p, R, S(stream));
        }
    }
    return moe_launch_generic_gemm(X, sxm, sxk, W, swe, swk, swn, A, sae, sak, sar, B, sbe, sbr, sbn, Y, sym, syn, pos,
                                   pos64, offsets, off64, E, R, K, N, A ? rank : 0, fan_out, scaling, x_grouped,
                                   y_grouped, dtype, S(stream));
}

// ---------------------------------------------------------------------------------------------------------
static inline bool bwd_ab_fast(int64_t K, int64_t N, int rank, int dtype, int64_t sdm, int64_t sdn, int64_t sxm,
                               int64_t sxk, const void* DY, const void* X)
{
    return (dtype == MOE_BF16 || dtype == MOE_F16) && rank >= 1 && sdn == 1 && sxk == 1 && K % 32 == 0 && N % 32 == 0 && sdm % 8 == 0 &&
           sxm % 8 == 0 && aligned16(DY) && aligned16(X);
}

size_t moe_group_bwd_ab_workspace_bytes(int64_t R, int E, int64_t K, int64_t N, int rank, int dtype)
{
    const size_t esz = dtype == MOE_F32 ? 4 : 2;
    const size_t generic = 2 * al((size_t)R * (size_t)(rank > 0 ? rank : 1) * esz) + 256;
    const int64_t mx = K > N ? K : N;
    const size_t fast = pack_bytes(E, K) + pack_bytes(E, N) + 4 * q_bytes(R) + al(moe_xtp_workspace_bytes(R, E, mx)) + 256;
    return generic > fast ? generic : fast;
}

int moe_group_bwd_ab(const void* DY, int64_t sdm, int64_t sdn, const void* X, int64_t sxm, int64_t sxk, const void* A,
                     int64_t sae, int64_t sak, int64_t sar, const void* B, int64_t sbe, int64_t sbr, int64_t sbn,
                     int rank, float scaling, void* DA, int64_t sdae, int64_t sdak, int64_t sdar, void* DB,
                     int64_t sdbe, int64_t sdbr, int64_t sdbn, const void* offsets, int off64, int E, int64_t R,
                     int64_t K, int64_t N, int dtype, void* workspace, size_t workspace_bytes, void* stream)
{
    if (!DY || !X || !A || !B || !DA || !DB || !offsets || !workspace || rank < 1 || E < 1) return MOE_ERR_BAD_ARG;
    if (workspace_bytes < moe_group_bwd_ab_workspace_bytes(R, E, K, N, rank, dtype)) return MOE_ERR_WORKSPACE;
    Bump ws(workspace, workspace_bytes);
    if (bwd_ab_fast(K, N, rank, dtype, sdm, sdn, sxm, sxk, DY, X)) {
        const int64_t ldt = pad_rows(R);
        void* At = ws.take(pack_bytes(E, K));   // [e][r][k] = A[e][k][r]
        void* Bt = ws.take(pack_bytes(E, N));   // [e][r][n] = B[e][r][n]
        void* Q = ws.take(q_bytes(R));
        void* Qt = ws.take(q_bytes(R));
        void* P = ws.take(q_bytes(R));
        void* Pt = ws.take(q_bytes(R));
        const int64_t mx = K > N ? K : N;
        const size_t xb = moe_xtp_workspace_bytes(R, E, mx);
        void* xw = ws.take(xb);
        if (!xw) return MOE_ERR_WORKSPACE;
        const int f16 = dtype == MOE_F16;
        // column r of dA depends only on row r of B and row r of dB only on column r of A, so a rank above 16 is
        // worked through in independent chunks of 16 rank columns
        for (int r0 = 0; r0 < rank; r0 += 16) {
            const int rk = (rank - r0 < 16) ? rank - r0 : 16;
            const uint16_t* Ac = (const uint16_t*)A + r0 * sar;
            const uint16_t* Bc = (const uint16_t*)B + r0 * sbr;
            uint16_t* DAc = (uint16_t*)DA + r0 * sdar;
            uint16_t* DBc = (uint16_t*)DB + r0 * sdbr;
            TRY(moe_launch_pack_lora(Ac, sae, sak, sar, At, E, K, rk, 1, S(stream)));
            TRY(moe_launch_pack_lora(Bc, sbe, sbn, sbr, Bt, E, N, rk, 1, S(stream)));
            TRY(moe_launch_rows_lora(X, sxm, At, Q, Qt, ldt, nullptr, 0, offsets, off64, E, R, K, 1, 1, scaling, nullptr, S(stream), f16));
            TRY(moe_launch_rows_lora(DY, sdm, Bt, P, Pt, ldt, nullptr, 0, offsets, off64, E, R, N, 1, 1, scaling, nullptr, S(stream), f16));
            TRY(moe_launch_xtp(X, sxm, nullptr, 0, 1, Pt, ldt, nullptr, DAc, sdae, sdak, sdar, rk, offsets, off64, E, R, K,
                               1.f, xw, xb, S(stream), f16));
            TRY(moe_launch_xtp(DY, sdm, nullptr, 0, 1, Qt, ldt, nullptr, DBc, sdbe, sdbn, sdbr, rk, offsets, off64, E, R, N,
                               1.f, xw, xb, S(stream), f16));
        }
        return MOE_OK;
    }
    // generic: P = DY B^T, Q = X A (both (R, rank), storage dtype), then the two grouped X^T Y products
    const size_t esz = dtype == MOE_F32 ? 4 : 2;
    void* P = ws.take((size_t)R * rank * esz);
    void* Q = ws.take((size_t)R * rank * esz);
    if (!Q) return MOE_ERR_WORKSPACE;
    TRY(moe_launch_generic_gemm(DY, sdm, sdn, B, sbe, sbn, sbr, nullptr, 0, 0, 0, nullptr, 0, 0, 0, P, rank, 1, nullptr, 0,
                                offsets, off64, E, R, N, rank, 0, 1, 0.f, 1, 1, dtype, S(stream)));
    TRY(moe_launch_generic_gemm(X, sxm, sxk, A, sae, sak, sar, nullptr, 0, 0, 0, nullptr, 0, 0, 0, Q, rank, 1, nullptr, 0,
                                offsets, off64, E, R, K, rank, 0, 1, 0.f, 1, 1, dtype, S(stream)));
    TRY(moe_launch_generic_xty(X, sxm, sxk, P, rank, 1, DA, sdae, sdak, sdar, offsets, off64, E, K, rank, scaling, dtype, S(stream)));
    TRY(moe_launch_generic_xty(Q, rank, 1, DY, sdm, sdn, DB, sdbe, sdbr, sdbn, offsets, off64, E, rank, N, scaling, dtype, S(stream)));
    return MOE_OK;
}

int moe_group_bwd_w(const void* DY, int64_t sdm, int64_t sdn, const void* X, int64_t sxm, int64_t sxk, void* DW,
                    int64_t swe, int64_t swk, int64_t swn, const void* offsets, int off64, int E, int64_t R, int64_t K,
                    int64_t N, int dtype, void* stream)
{
    if (!DY || !X || !DW || !offsets || E < 1 || R < 0 || K < 0 || N < 0) return MOE_ERR_BAD_ARG;
    if (K == 0 || N == 0) return MOE_OK;
    if ((dtype == MOE_BF16 || dtype == MOE_F16) && sdn == 1 && sxk == 1 && swn == 1) {
        MoeXtyParams p = {};
        p.f16 = dtype == MOE_F16;
        p.X = (const uint16_t*)X; p.ldx = sxm;
        p.DY = (const uint16_t*)DY; p.ldy = sdm;
        p.DW = (uint16_t*)DW; p.swe = swe; p.ldw = swk;
        p.offsets = offsets; p.off64 = off64; p.E = E; p.K = K; p.N = N;
        if (moe_xty_mfma_supported(p, R)) {
            hipStream_t st = S(stream);
            TIMED("bwd.group_bwd_w");
            return moe_launch_xty_mfma(p, R, st);
        }
    }
    return moe_launch_generic_xty(X, sxm, sxk, DY, sdm, sdn, DW, swe, swk, swn, offsets, off64, E, K, N, 1.f, dtype, S(stream));
}

int moe_group_rows(const void* src, int64_t lds_, void* out, int64_t ldo, const void* pos, int pos64, int fan_out,
                   const void* coeff, int coeff_dtype, int64_t nrows, int64_t ncols, int dtype, void* stream)
{
    if ((nrows > 0 && (!src || !out || !pos))) return MOE_ERR_BAD_ARG;
    hipStream_t st = S(stream);
    TIMED("rows.group");
    return moe_launch_group_rows(src, lds_, out, ldo, pos, pos64, fan_out, coeff, coeff_dtype, nrows, ncols, dtype,
                                 st);
}

int moe_combine(const void* y, int64_t ldy, void* out, int64_t ldo, const void* gates, int gates_dtype,
                const int32_t* inv, int k, int64_t ntok, int64_t ncols, int dtype, const float* extra_coef,
                const void* extra_rows, int64_t lde, int n_extra, void* stream)
{
    if (k < 0 || (ntok > 0 && (!out || (k > 0 && !y))) || (k == 0 && n_extra < 1)) return MOE_ERR_BAD_ARG;
    if (n_extra > 0 && (!extra_coef || !extra_rows)) return MOE_ERR_BAD_ARG;
    hipStream_t st = S(stream);
    TIMED("rows.combine");
    return moe_launch_combine_fwd(y, ldy, out, ldo, gates, gates_dtype, inv, k, ntok, ncols, dtype, extra_coef,
                                  extra_rows, lde, n_extra, st);
}

int moe_combine_dgates(const void* y, int64_t ldy, const void* dout, int64_t ldd, void* dgates, int gates_dtype,
                       const int32_t* inv, int k, int64_t ntok, int64_t ncols, int dtype, void* stream)
{
    if ((ntok > 0 && (!y || !dout || !dgates)) || k < 1) return MOE_ERR_BAD_ARG;
    hipStream_t st = S(stream);
    TIMED("rows.combine_dgates");
    return moe_launch_combine_dgates(y, ldy, dout, ldd, dgates, gates_dtype, inv, k, ntok, ncols, dtype, st);
}

int moe_swiglu(const void* gate, const void* up, void* h, int64_t n, int dtype, void* stream)
{
    if (n > 0 && (!gate || !up || !h)) return MOE_ERR_BAD_ARG;
    return moe_launch_swiglu_fwd(gate, up, h, n, dtype, S(stream));
}

int moe_swiglu_bwd(const void* gate, const void* up, const void* dh, void* dgate, void* dup, int64_t n, int dtype,
                   void* stream)
{
    if (n > 0 && (!gate || !up || !dh || !dgate || !dup)) return MOE_ERR_BAD_ARG;
    return moe_launch_swiglu_bwd(gate, up, dh, dgate, dup, n, dtype, S(stream));
}

// ---------------------------------------------------------------------------------------------------------
// fused expert MLP
static inline size_t sk_bytes_mlp(int64_t R, int E, int64_t d, int64_t f)
{
    const size_t a = moe_gemm_sk_bytes(R, E, d), b = moe_gemm_sk_bytes(R, E, f);
    return a > b ? a : b;
}
// column-tile partials of the two fused column contractions of the dh GEMM: [2][ceil(f / 256)][R][16] fp32
static inline size_t cc_bytes(int64_t R, int64_t f) { return (size_t)2 * (size_t)((f + 255) / 256) * (size_t)R * 16 * sizeof(float); }

size_t moe_mlp_workspace_bytes(int64_t R, int E, int64_t d, int64_t f, int rank)
{
    size_t n = al(sk_bytes_mlp(R, E, d, f)) + 256;
    if (rank <= 0) return n;
    const int64_t mx = d > f ? d : f;
    const size_t C = (size_t)(rank + 15) / 16;   // 16-wide chunks per adapter
    return n + C * (3 * pack_bytes(E, d) + 3 * pack_bytes(E, f) + 7 * q_bytes(R)) + al(3 * moe_xtp_workspace_bytes(R, E, mx)) + al(cc_bytes(R, f));
}

size_t moe_mlp_saved_bytes(int64_t R, int rank) { return rank > 0 ? (size_t)((rank + 15) / 16) * 6 * q_bytes(R) : 256; }

// An adapter of rank r enters the fused layer as C = ceil(r / 16) chunks of 16 rank columns; the gate/up launch takes
// the chunks of both its adapters as K slabs, which bounds C
constexpr int MLP_MAX_CHUNKS = MOE_MAX_STRIDED_SLABS / 2;
static bool mlp_shapes_ok(int64_t d, int64_t f, int64_t ldx, int rank, const void* a, const void* b, const void* c,
                          const void* x)
{
    return d % 64 == 0 && f % 64 == 0 && ldx % 8 == 0 && rank <= 16 * MLP_MAX_CHUNKS && aligned16(a) && aligned16(b) && aligned16(c) &&
           aligned16(x);
}
// What the grouped GEMM's 32-bit offsets allow, checked before anything is enqueued: gathered rows are addressed from
// the start of their matrix (below 4 GiB), one expert's weight matrix likewise, one 256-row tile of the (R, f)
// intermediates below 2 GiB.  The number of rows itself is not limited.
static bool mlp_sizes_ok(int64_t gathered_rows, int64_t ld_gathered, int64_t d, int64_t f)
{
    const int64_t g4 = (int64_t)1 << 32;
    return (gathered_rows * ld_gathered + d) * 2 < g4 && (f * d + d) * 2 < g4 && (256 * f + f) * 2 < g4 / 2 && (256 * d + d) * 2 < g4 / 2;
}

int moe_mlp_fwd(const void* x, int64_t ldx, const void* w1, const void* w3, const void* w2, const void* const* lora,
                const int64_t* ls, int rank, float scaling, void* gate, void* up, void* h, void* y, int64_t ldy,
                const void* pos, int pos64, const void* offsets, int off64, int E, int64_t R, int64_t d, int64_t f,
                int fan_out, int y_grouped, int dtype, void* saved, void* workspace, size_t workspace_bytes, void* stream)
{
    if (!x || !w1 || !w3 || !w2 || !h || !y || !pos || !offsets || E < 1 || fan_out < 1) return MOE_ERR_BAD_ARG;
    const bool has_lora = lora && lora[0];
    if (has_lora && (!ls || !saved || rank < 1)) return MOE_ERR_BAD_ARG;
    if (dtype != MOE_BF16 && dtype != MOE_F16) return MOE_ERR_UNSUPPORTED;
    const int f16 = dtype == MOE_F16;
    if (!mlp_shapes_ok(d, f, ldx, has_lora ? rank : 0, w1, w3, w2, x)) return MOE_ERR_UNSUPPORTED;
    if (!mlp_sizes_ok(R / fan_out, ldx, d, f)) return MOE_ERR_UNSUPPORTED;
    if (R == 0) return MOE_OK;
    hipStream_t st = S(stream);
    uint8_t* sv = (uint8_t*)saved;
    const size_t qb = q_bytes(R);
    const int64_t ldt = pad_rows(R);
    if (!workspace || workspace_bytes < moe_mlp_workspace_bytes(R, E, d, f, has_lora ? rank : 0)) return MOE_ERR_WORKSPACE;
    Bump ws(workspace, workspace_bytes);
    void* skws = ws.take(sk_bytes_mlp(R, E, d, f));
    bool counters_clean = has_lora;   // K-split counters: zeroed by the adapter pack launch; a GEMM launch that uses them leaves them zero
    // An adapter of rank r is worked through as C = ceil(r / 16) independent 16-wide chunks of its rank columns:
    // x A B = sum_c (x A[:, c]) B[c, :].  saved: six groups of C q_bytes blocks (one per chunk): Q1, Q3, Q2, Qt1, Qt3, Qt2.
    // The chunks of a group lie at one stride, and so do the packed B-side images, so that a launch with many slabs
    // finds slab s at base + s * stride (the gate/up launch: Q1 chunks then Q3 chunks, lb1 chunks then lb3 chunks).
    const int C = has_lora ? (rank + 15) / 16 : 0;
    auto svp = [&](int which, int c) { return sv + ((size_t)which * C + c) * qb; };   // which: 0 Q1, 1 Q3, 2 Q2, 3 Qt1, 4 Qt3, 5 Qt2
    const size_t pbd = pack_bytes(E, d), pbf = pack_bytes(E, f);
    void *At1[MLP_MAX_CHUNKS] = {}, *At3[MLP_MAX_CHUNKS] = {}, *At2c[MLP_MAX_CHUNKS] = {};
    uint8_t *lb13 = nullptr, *lb2 = nullptr;
    auto lb1 = [&](int c) { return lb13 + (size_t)c * pbf; };
    auto lb3 = [&](int c) { return lb13 + (size_t)(C + c) * pbf; };
    auto lb2c = [&](int c) { return lb2 + (size_t)c * pbd; };
    // the slabs of a launch: by their own pointers while they fit, else by base and stride
    auto set_slabs = [&](MoeGemmParams& p, int n, const uint8_t* q0, const uint8_t* b0, size_t bstride) {
        for (int i = 0; i < n && i < MOE_MAX_SLABS; ++i) {
            p.Q[i] = (const uint16_t*)(q0 + (size_t)i * qb);
            p.LB[i] = (const uint16_t*)(b0 + (size_t)i * bstride);
        }
        p.nslab = n; p.q_slab_stride = (int64_t)(qb / 2); p.lb_slab_stride = (int64_t)(bstride / 2);
    };
    // a rank of at most 16: the w2 GEMM's low-rank operand Q2 = h A2 comes out of the pair GEMM's epilogue as per-column-tile
    // partials (h is not read again for it); more chunks take separate passes over h
    const bool fuse_q2 = has_lora && rank <= 16;
    float* ccw = fuse_q2 ? (float*)ws.take(cc_bytes(R, f)) : nullptr;
    if (fuse_q2 && !ccw) return MOE_ERR_WORKSPACE;
    if (has_lora) {
        // lora order a1,b1,a3,b3,a2,b2; strides {expert, dim1, dim2}
        { TIMED("fwd.pack_lora");
        for (int c = 0; c < C; ++c) { At1[c] = ws.take(pbd); At3[c] = ws.take(pbd); At2c[c] = ws.take(pbf); }
        lb13 = (uint8_t*)ws.take((size_t)2 * C * pbf);
        lb2 = (uint8_t*)ws.take((size_t)C * pbd);
        if (!lb13 || !lb2 || !At2c[C - 1]) return MOE_ERR_WORKSPACE;
        for (int c0 = 0; c0 < C; c0 += 2) {   // six images per chunk, two chunks per launch
            MoePackBatch pb = {};
            pb.E = E;
            for (int c = c0; c < C && c < c0 + 2; ++c) {
                const int64_t r0 = 16 * c;
                const int rk = (rank - 16 * c < 16) ? rank - 16 * c : 16;
                auto L = [&](int i) { return (const uint16_t*)lora[i]; };
                MoePackJob* j = pb.job + pb.njobs;
                j[0] = {L(0) + r0 * ls[2], ls[0], ls[1], ls[2], (uint16_t*)At1[c], d, 1, rk};
                j[1] = {L(1) + r0 * ls[4], ls[3], ls[5], ls[4], (uint16_t*)lb1(c), f, 0, rk};
                j[2] = {L(2) + r0 * ls[8], ls[6], ls[7], ls[8], (uint16_t*)At3[c], d, 1, rk};
                j[3] = {L(3) + r0 * ls[10], ls[9], ls[11], ls[10], (uint16_t*)lb3(c), f, 0, rk};
                j[4] = {L(4) + r0 * ls[14], ls[12], ls[13], ls[14], (uint16_t*)At2c[c], f, 1, rk};
                j[5] = {L(5) + r0 * ls[16], ls[15], ls[17], ls[16], (uint16_t*)lb2c(c), d, 0, rk};
                pb.njobs += 6;
            }
            if (c0 == 0) { pb.zero_ptr = (int*)skws; pb.zero_n = moe_gemm_num_counters(); }   // the K-split counters of the GEMMs below
            TRY(moe_launch_pack_lora_batch(pb, st));
        } }
        { TIMED("fwd.rows_lora_x");
        for (int c = 0; c < C; ++c)
            TRY(moe_launch_rows_lora2(x, x, ldx, At1[c], At3[c], svp(0, c), svp(1, c), svp(3, c), svp(4, c), ldt, pos, pos64, offsets,
                                      off64, E, R, d, fan_out, 0, scaling, nullptr, st, nullptr, f16)); }
    }
    {
        MoeGemmParams p = {};
        p.X[0] = (const uint16_t*)x; p.ldx = ldx; p.nseg = 1;
        p.W[0] = (const uint16_t*)w1; p.W[1] = (const uint16_t*)w3; p.swe = f * d; p.ldw = d; p.nn = 0;
        if (has_lora) {   // gate slabs first, then up slabs
            set_slabs(p, 2 * C, svp(0, 0), lb13, pbf);
            p.slab_mode = 1;
        }
        p.Y[0] = (uint16_t*)h; p.Y[1] = (uint16_t*)gate; p.Y[2] = (uint16_t*)up; p.ldy = f;
        p.pos = pos; p.pos64 = pos64; p.offsets = offsets; p.off64 = off64;
        p.E = E; p.K = d; p.N = f; p.fan_out = fan_out; p.x_grouped = 0; p.y_grouped = 1; p.epi = MOE_EPI_SWIGLU; p.f16 = f16;
        if (fuse_q2) {   // Q2 = h A2 (the w2 GEMM's low-rank operand) as per-column-tile partials from the epilogue
            p.epi = MOE_EPI_SWIGLU_FUSED;
            p.CB[0] = (const uint16_t*)At2c[0]; p.CCP[0] = ccw; p.ncc = 1; p.cc_rows = R;
        }
        moe_gemm_sk_attach(p, skws, R, E, f);
        p.counters_clean = counters_clean;
        if (moe_gemm_max_split(p.epi == MOE_EPI_SWIGLU || p.epi == MOE_EPI_SWIGLU_FUSED) > 1) counters_clean = true;   // zeroed by that launch if they were not, and left zero
        TIMED("fwd.gemm_w1w3_swiglu");
        TRY(moe_launch_gemm_mfma(p, R, st));
    }
    if (has_lora) {
        TIMED("fwd.rows_lora_h");
        if (fuse_q2)   // the products over each column tile came out of the pair GEMM's epilogue: add the tiles, scale, round
            TRY(moe_launch_cc_reduce2(ccw, nullptr, (int)((f + 127) / 128), R, scaling, svp(2, 0), nullptr, svp(5, 0), nullptr, ldt, st, f16));
        else
        for (int c = 0; c < C; c += 2) {   // two chunks per launch: the twin's reads of h are served by L2
            const bool two = c + 1 < C;
            TRY(moe_launch_rows_lora2(h, two ? h : nullptr, f, At2c[c], two ? At2c[c + 1] : nullptr, svp(2, c), two ? svp(2, c + 1) : nullptr, svp(5, c),
                                      two ? svp(5, c + 1) : nullptr, ldt, nullptr, 0, offsets, off64, E, R, f, 1, 1, scaling, nullptr, st, nullptr, f16));
        }
    }
    {
        MoeGemmParams p = {};
        p.X[0] = (const uint16_t*)h; p.ldx = f; p.nseg = 1;
        p.W[0] = (const uint16_t*)w2; p.swe = f * d; p.ldw = d; p.nn = 1;
        if (has_lora) {
            set_slabs(p, C, svp(2, 0), lb2, pbd);
            p.slab_mode = 0;
        }
        p.Y[0] = (uint16_t*)y; p.ldy = ldy;
        p.pos = pos; p.pos64 = pos64; p.offsets = offsets; p.off64 = off64;
        p.E = E; p.K = f; p.N = d; p.fan_out = 1; p.x_grouped = 1; p.y_grouped = y_grouped; p.epi = MOE_EPI_STORE; p.f16 = f16;
        moe_gemm_sk_attach(p, skws, R, E, d);
        p.counters_clean = counters_clean;
        if (moe_gemm_max_split(p.epi == MOE_EPI_SWIGLU || p.epi == MOE_EPI_SWIGLU_FUSED) > 1) counters_clean = true;   // zeroed by that launch if they were not, and left zero
        TIMED("fwd.gemm_w2");
        TRY(moe_launch_gemm_mfma(p, R, st));
    }
    return MOE_OK;
}

int moe_mlp_bwd(const void* dy, int64_t lddy, int dy_grouped, int dy_fan_out, const float* row_scale, const void* x,
                int64_t ldx, const void* w1, const void* w3, const void* w2, const void* const* lora,
                const int64_t* ls, void* const* lg, const int64_t* gs, int rank, float scaling, const void* gate,
                const void* up, const void* h, void* dgate, void* dup, void* dx_rows, int64_t lddx, int dx_grouped,
                const void* pos, int pos64, const void* offsets, int off64, int E, int64_t R, int64_t d, int64_t f,
                int fan_out, int dtype, const void* saved, void* workspace, size_t workspace_bytes, void* stream)
{
    if (!dy || !x || !w1 || !w3 || !w2 || !gate || !up || !h || !dgate || !dup || !dx_rows || !pos || !offsets)
        return MOE_ERR_BAD_ARG;
    const bool has_lora = lora && lora[0];
    if (has_lora && (!ls || !lg || !gs || !saved || rank < 1)) return MOE_ERR_BAD_ARG;
    if (dtype != MOE_BF16 && dtype != MOE_F16) return MOE_ERR_UNSUPPORTED;
    const int f16 = dtype == MOE_F16;
    if (!mlp_shapes_ok(d, f, ldx, has_lora ? rank : 0, w1, w3, w2, x) || lddy % 8 != 0 || !aligned16(dy))
        return MOE_ERR_UNSUPPORTED;
    if (dy_fan_out < 1 || fan_out < 1) return MOE_ERR_BAD_ARG;
    if (!mlp_sizes_ok(dy_grouped ? 256 : R / dy_fan_out, lddy, d, f)) return MOE_ERR_UNSUPPORTED;
    hipStream_t st = S(stream);
    const size_t qb = q_bytes(R);
    const int64_t ldt = pad_rows(R);
    const uint8_t* sv = (const uint8_t*)saved;
    // adapters are worked through in C chunks of 16 rank columns (see moe_mlp_fwd): packed factors per chunk, and the
    // interims in six groups of C blocks: P2, P1, P3, P2t, P1t, P3t
    const int C = has_lora ? (rank + 15) / 16 : 0;
    const size_t pbd = pack_bytes(E, d), pbf = pack_bytes(E, f);
    void *bt2[MLP_MAX_CHUNKS] = {}, *bt1[MLP_MAX_CHUNKS] = {}, *bt3[MLP_MAX_CHUNKS] = {};
    uint8_t *la2 = nullptr, *la13 = nullptr;   // B-side images of the dh launch's slabs (a2 chunks) and of the dX launch's (a1 chunks, then a3 chunks)
    auto la2c = [&](int c) { return la2 + (size_t)c * pbf; };
    auto la1 = [&](int c) { return la13 + (size_t)c * pbd; };
    auto la3 = [&](int c) { return la13 + (size_t)(C + c) * pbd; };
    uint8_t* pq = nullptr;
    auto pqp = [&](int which, int c) { return pq + ((size_t)which * C + c) * qb; };   // which: 0 P2, 1 P1, 2 P3, 3 P2t, 4 P1t, 5 P3t
    auto svp = [&](int which, int c) { return sv + ((size_t)which * C + c) * qb; };   // which: 0 Q1, 1 Q3, 2 Q2, 3 Qt1, 4 Qt3, 5 Qt2
    auto set_slabs = [&](MoeGemmParams& p, int n, const uint8_t* q0, const uint8_t* b0, size_t bstride) {
        for (int i = 0; i < n && i < MOE_MAX_SLABS; ++i) {
            p.Q[i] = (const uint16_t*)(q0 + (size_t)i * qb);
            p.LB[i] = (const uint16_t*)(b0 + (size_t)i * bstride);
        }
        p.nslab = n; p.q_slab_stride = (int64_t)(qb / 2); p.lb_slab_stride = (int64_t)(bstride / 2);
    };
    auto chunk_rank = [&](int c) { return (rank - 16 * c < 16) ? rank - 16 * c : 16; };
    void* xw = nullptr;
    void* p2s = nullptr;
    float* ccw = nullptr;
    size_t xb = 0;
    // a rank of at most 16 (one chunk): the adapter gradients that sum over the rows of dgate, dup and h are produced by
    // the dh GEMM's epilogue as per-row-tile partials; more chunks take separate passes over those tensors
    const bool fuse_rc = has_lora && rank <= 16;
    if (!workspace || workspace_bytes < moe_mlp_workspace_bytes(R, E, d, f, has_lora ? rank : 0)) return MOE_ERR_WORKSPACE;
    Bump ws(workspace, workspace_bytes);
    void* skws = ws.take(sk_bytes_mlp(R, E, d, f));
    bool counters_clean = has_lora;   // K-split counters: zeroed by the adapter pack launch; a GEMM launch that uses them leaves them zero
    if (has_lora) {
        pq = (uint8_t*)ws.take((size_t)C * 6 * qb);
        if (fuse_rc) p2s = ws.take(qb);   // P2 times the row scale, row-major (the fused contraction's operand)
        if (fuse_rc) ccw = (float*)ws.take(cc_bytes(R, f));
        const int64_t mx = d > f ? d : f;
        xb = 3 * moe_xtp_workspace_bytes(R, E, mx);   // paired reductions keep two sets of partials, the fused ones of the dh GEMM three
        xw = ws.take(xb);
        TIMED("bwd.pack_lora");
        for (int c = 0; c < C; ++c) {
            bt2[c] = ws.take(pbd);  // fragment order of b2[e][r][n=d]
            bt1[c] = ws.take(pbf);  // fragment order of b1[e][r][n=f]
            bt3[c] = ws.take(pbf);
        }
        la2 = (uint8_t*)ws.take((size_t)C * pbf);        // [e][n=f][r] = a2[e][n][r]
        la13 = (uint8_t*)ws.take((size_t)2 * C * pbd);   // [e][n=d][r] = a1[e][n][r], a3 likewise
        if (!la2 || !la13 || !bt3[C - 1] || !xw) return MOE_ERR_WORKSPACE;
        for (int c0 = 0; c0 < C; c0 += 2) {   // six images per chunk, two chunks per launch
            MoePackBatch pb = {};
            pb.E = E;
            for (int c = c0; c < C && c < c0 + 2; ++c) {
                const int64_t r0 = 16 * c;
                const int rk = chunk_rank(c);
                auto L = [&](int i) { return (const uint16_t*)lora[i]; };
                MoePackJob* j = pb.job + pb.njobs;
                j[0] = {L(5) + r0 * ls[16], ls[15], ls[17], ls[16], (uint16_t*)bt2[c], d, 1, rk};
                j[1] = {L(4) + r0 * ls[14], ls[12], ls[13], ls[14], (uint16_t*)la2c(c), f, 0, rk};
                j[2] = {L(1) + r0 * ls[4], ls[3], ls[5], ls[4], (uint16_t*)bt1[c], f, 1, rk};
                j[3] = {L(3) + r0 * ls[10], ls[9], ls[11], ls[10], (uint16_t*)bt3[c], f, 1, rk};
                j[4] = {L(0) + r0 * ls[2], ls[0], ls[1], ls[2], (uint16_t*)la1(c), d, 0, rk};
                j[5] = {L(2) + r0 * ls[8], ls[6], ls[7], ls[8], (uint16_t*)la3(c), d, 0, rk};
                pb.njobs += 6;
            }
            if (c0 == 0) { pb.zero_ptr = (int*)skws; pb.zero_n = moe_gemm_num_counters(); }   // the K-split counters of the GEMMs below
            TRY(moe_launch_pack_lora_batch(pb, st));
        }
    }
    // ---- w2 backward: dh = (dy W2^T + P2 A2^T) * row_scale, SwiGLU backward in the epilogue
    if (has_lora) {
        TIMED("bwd.rows_lora_dy");
        for (int c = 0; c < C; c += 2) {
            const bool two = c + 1 < C;
            TRY(moe_launch_rows_lora2(dy, two ? dy : nullptr, lddy, bt2[c], two ? bt2[c + 1] : nullptr, pqp(0, c), two ? pqp(0, c + 1) : nullptr, pqp(3, c),
                                      two ? pqp(3, c + 1) : nullptr, ldt, pos, pos64, offsets, off64, E, R, d, dy_fan_out, dy_grouped, scaling,
                                      row_scale, st, p2s, f16));
        }
    }
    {
        MoeGemmParams p = {};
        p.X[0] = (const uint16_t*)dy; p.ldx = lddy; p.nseg = 1;
        p.W[0] = (const uint16_t*)w2; p.swe = f * d; p.ldw = d; p.nn = 0;  // (E, K=d, N=f): n rows, k contiguous
        if (has_lora) {
            set_slabs(p, C, pqp(0, 0), la2, pbf);
            p.slab_mode = 0;
        }
        p.Y[0] = (uint16_t*)dgate; p.Y[1] = (uint16_t*)dup; p.ldy = f;
        p.H1 = (const uint16_t*)gate; p.H3 = (const uint16_t*)up; p.ldh = f; p.row_scale = row_scale;
        p.pos = pos; p.pos64 = pos64; p.offsets = offsets; p.off64 = off64;
        p.E = E; p.K = d; p.N = f; p.fan_out = dy_fan_out; p.x_grouped = dy_grouped; p.y_grouped = 1;
        p.epi = MOE_EPI_SWIGLU_BWD; p.f16 = f16;
        if (fuse_rc) {   // dB1 = Q1^T dgate, dB3 = Q3^T dup, dA2 = h^T (row_scale P2) as per-row-tile partials from the epilogue
            const size_t one = moe_xtp_workspace_bytes(R, E, f);
            p.RC[0] = (const uint16_t*)svp(0, 0); p.RC[1] = (const uint16_t*)svp(1, 0); p.RC[2] = (const uint16_t*)p2s;
            for (int i = 0; i < 3; ++i) p.RCP[i] = (float*)((uint8_t*)xw + i * one);
            p.nrc = 3;
            // P1 = dgate B1^T, P3 = dup B3^T (the dX GEMM's low-rank operands) as per-column-tile partials
            const size_t cone = cc_bytes(R, f) / 2 / sizeof(float);
            p.CB[0] = (const uint16_t*)bt1[0]; p.CB[1] = (const uint16_t*)bt3[0];
            p.CCP[0] = ccw; p.CCP[1] = ccw + cone;
            p.ncc = 2; p.cc_rows = R;
            p.epi = MOE_EPI_SWIGLU_BWD_FUSED;
        }
        moe_gemm_sk_attach(p, skws, R, E, f);
        p.counters_clean = counters_clean;
        if (moe_gemm_max_split(p.epi == MOE_EPI_SWIGLU || p.epi == MOE_EPI_SWIGLU_FUSED) > 1) counters_clean = true;   // zeroed by that launch if they were not, and left zero
        TIMED("bwd.gemm_dh_swiglu_bwd");
        TRY(moe_launch_gemm_mfma(p, R, st));
    }
    if (has_lora) {
        // dA2[e][k=f][r] = sum_m h[m][k] * (row_scale[m] P2[m][r]);  dB2[e][r][n=d] = sum_m (row_scale[m] Q2[m][r]) dy[m][n]
        const int64_t sb1[3] = {gs[3], gs[5], gs[4]}, sb3[3] = {gs[9], gs[11], gs[10]};
        { TIMED("bwd.xtp_w2");
        const int64_t sa2[3] = {gs[12], gs[13], gs[14]}, sb2[3] = {gs[15], gs[17], gs[16]};
        uint16_t* dA2 = (uint16_t*)lg[4];
        uint16_t* dB2 = (uint16_t*)lg[5];
        if (fuse_rc) {   // the sums over each row tile came out of the dh GEMM's epilogue: add the tiles per expert
            const size_t one = moe_xtp_workspace_bytes(R, E, f);
            const float* part = (const float*)xw;
            TRY(moe_launch_xtp_reduce2(part, part + one / sizeof(float), lg[1], lg[3], sb1, sb3, rank, rank, offsets, off64, E, f, 1.f, st, f16));
            TRY(moe_launch_xtp_reduce2(part + 2 * (one / sizeof(float)), nullptr, dA2, nullptr, sa2, nullptr, rank, 0, offsets, off64, E, f, 1.f, st, f16));
        } else
        for (int c = 0; c < C; c += 2) {   // two chunks per launch: the twin's reads of h are served by L2
            const bool two = c + 1 < C;
            TRY(moe_launch_xtp2(h, two ? h : nullptr, f, nullptr, 0, 1, pqp(3, c), two ? pqp(3, c + 1) : nullptr, ldt, nullptr, dA2 + 16 * c * gs[14],
                                two ? dA2 + 16 * (c + 1) * gs[14] : nullptr, sa2, sa2, chunk_rank(c), two ? chunk_rank(c + 1) : 0, offsets, off64, E, R, f,
                                1.f, xw, xb, st, f16));
        }
        for (int c = 0; c < C; c += 2) {
            const bool two = c + 1 < C;
            TRY(moe_launch_xtp2(dy, two ? dy : nullptr, lddy, dy_grouped ? nullptr : pos, pos64, dy_fan_out, svp(5, c),
                                two ? svp(5, c + 1) : nullptr, ldt, row_scale, dB2 + 16 * c * gs[16], two ? dB2 + 16 * (c + 1) * gs[16] : nullptr, sb2, sb2,
                                chunk_rank(c), two ? chunk_rank(c + 1) : 0, offsets, off64, E, R, d, 1.f, xw, xb, st, f16));
        } }
        // ---- w1 / w3 backward
        TIMED("bwd.rows_lora_dgate_dup");
        if (fuse_rc) {   // the products over each column tile came out of the dh GEMM's epilogue: add the tiles, scale, round
            const size_t cone = cc_bytes(R, f) / 2 / sizeof(float);
            TRY(moe_launch_cc_reduce2(ccw, ccw + cone, (int)((f + 255) / 256), R, scaling, pqp(1, 0), pqp(2, 0), pqp(4, 0), pqp(5, 0), ldt, st, f16));
        } else
        for (int c = 0; c < C; c += 2) {   // two chunks of one adapter per launch, so that dgate and dup are each fetched once per pair of chunks
            const bool two = c + 1 < C;
            TRY(moe_launch_rows_lora2(dgate, two ? dgate : nullptr, f, bt1[c], two ? bt1[c + 1] : nullptr, pqp(1, c), two ? pqp(1, c + 1) : nullptr, pqp(4, c),
                                      two ? pqp(4, c + 1) : nullptr, ldt, nullptr, 0, offsets, off64, E, R, f, 1, 1, scaling, nullptr, st, nullptr, f16));
            TRY(moe_launch_rows_lora2(dup, two ? dup : nullptr, f, bt3[c], two ? bt3[c + 1] : nullptr, pqp(2, c), two ? pqp(2, c + 1) : nullptr, pqp(5, c),
                                      two ? pqp(5, c + 1) : nullptr, ldt, nullptr, 0, offsets, off64, E, R, f, 1, 1, scaling, nullptr, st, nullptr, f16));
        }
    }
    {
        MoeGemmParams p = {};
        p.X[0] = (const uint16_t*)dgate; p.X[1] = (const uint16_t*)dup; p.ldx = f; p.nseg = 2;
        p.W[0] = (const uint16_t*)w1; p.W[1] = (const uint16_t*)w3; p.swe = f * d; p.ldw = d; p.nn = 1;  // (E, K=f, N=d)
        if (has_lora) {   // P1 chunks, then P3 chunks; every slab feeds every column
            set_slabs(p, 2 * C, pqp(1, 0), la13, pbd);
            p.slab_mode = 0;
        }
        p.Y[0] = (uint16_t*)dx_rows; p.ldy = lddx;
        p.pos = pos; p.pos64 = pos64; p.offsets = offsets; p.off64 = off64;
        p.E = E; p.K = f; p.N = d; p.fan_out = 1; p.x_grouped = 1; p.y_grouped = dx_grouped; p.epi = MOE_EPI_STORE; p.f16 = f16;
        moe_gemm_sk_attach(p, skws, R, E, d);
        p.counters_clean = counters_clean;
        if (moe_gemm_max_split(p.epi == MOE_EPI_SWIGLU || p.epi == MOE_EPI_SWIGLU_FUSED) > 1) counters_clean = true;   // zeroed by that launch if they were not, and left zero
        TIMED("bwd.gemm_dx_w1w3");
        TRY(moe_launch_gemm_mfma(p, R, st));
    }
    if (has_lora) {
        // dA1[e][k=d][r] = sum_m x[in_row(m)][k] P1[m][r];  dB1[e][r][n=f] = sum_m Q1[m][r] dgate[m][n]
        TIMED("bwd.xtp_w1w3");
        const int64_t sa1[3] = {gs[0], gs[1], gs[2]}, sa3[3] = {gs[6], gs[7], gs[8]};
        const int64_t sb1[3] = {gs[3], gs[5], gs[4]}, sb3[3] = {gs[9], gs[11], gs[10]};
        for (int c = 0; c < C; ++c) {
            const int rk = chunk_rank(c);
            TRY(moe_launch_xtp2(x, x, ldx, pos, pos64, fan_out, pqp(4, c), pqp(5, c), ldt, nullptr, (uint16_t*)lg[0] + 16 * c * gs[2],
                                (uint16_t*)lg[2] + 16 * c * gs[8], sa1, sa3, rk, rk, offsets, off64, E, R, d, 1.f, xw, xb, st, f16));
        }
        if (!fuse_rc)
        for (int c = 0; c < C; c += 2) {   // two chunks of one adapter per launch, so that dgate and dup are each fetched once per pair of chunks
            const bool two = c + 1 < C;
            const int rk0 = chunk_rank(c), rk1 = two ? chunk_rank(c + 1) : 0;
            TRY(moe_launch_xtp2(dgate, two ? dgate : nullptr, f, nullptr, 0, 1, svp(3, c), two ? svp(3, c + 1) : nullptr, ldt, nullptr, (uint16_t*)lg[1] + 16 * c * gs[4],
                                two ? (uint16_t*)lg[1] + 16 * (c + 1) * gs[4] : nullptr, sb1, sb1, rk0, rk1, offsets, off64, E, R, f, 1.f, xw, xb, st, f16));
            TRY(moe_launch_xtp2(dup, two ? dup : nullptr, f, nullptr, 0, 1, svp(4, c), two ? svp(4, c + 1) : nullptr, ldt, nullptr, (uint16_t*)lg[3] + 16 * c * gs[10],
                                two ? (uint16_t*)lg[3] + 16 * (c + 1) * gs[10] : nullptr, sb3, sb3, rk0, rk1, offsets, off64, E, R, f, 1.f, xw, xb, st, f16));
        }
    }
    return MOE_OK;
}

}  // extern "C"
