// Router (logits GEMV, softmax/top-k/renormalise) and the integer pipeline that puts token->expert
// assignments into expert-grouped order: histogram, prefix sums, stable counting sort, padded block table.
// All integer results are exact and independent of launch geometry (no floating point, no data races:
// LDS/global atomics are only used for integer counts whose final value is order independent).
#include "common.h"
#include "kernels.h"
#include <mutex>
#include <type_traits>

namespace {

constexpr int ROUTER_TOKENS_PER_WAVE = 2;
constexpr int ROUTER_EXPERT_GROUP = 8;

__device__ __forceinline__ float wave_sum(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

// 8 consecutive elements as floats; one 16-byte (2-byte types) or two 16-byte (fp32) loads when the row is aligned
template <typename T>
__device__ __forceinline__ void load8(const T* p, float* v, int kn, bool vec_ok)
{
    if (vec_ok && kn == 8) {
        if (sizeof(T) == 2) {
            const uint4 raw = *(const uint4*)p;
            const T* e = (const T*)&raw;
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = Elem<T>::ld(e + u);
        } else {
            const float4 a = *(const float4*)p, b = *((const float4*)p + 1);
            v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
        }
    } else {
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = (u < kn) ? Elem<T>::ld(p + u) : 0.f;
    }
}

// logits[t][e] = sum_k x[t][k] * wg[e][k], fp32 accumulate.  One wave owns ROUTER_TOKENS_PER_WAVE tokens
// and walks the hidden dimension 8 elements per lane at a time; experts are processed in groups of 8.
template <typename T>
__global__ void __launch_bounds__(256) router_logits_kernel(const T* __restrict__ x, int64_t ldx,
                                                            const T* __restrict__ wg, int64_t ldw,
                                                            float* __restrict__ logits, int64_t ntok, int64_t d, int E,
                                                            bool vec_ok)
{
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const int64_t t0 = wave * ROUTER_TOKENS_PER_WAVE;
    if (t0 >= ntok) return;
    for (int e0 = 0; e0 < E; e0 += ROUTER_EXPERT_GROUP) {
        float acc[ROUTER_TOKENS_PER_WAVE][ROUTER_EXPERT_GROUP];
#pragma unroll
        for (int i = 0; i < ROUTER_TOKENS_PER_WAVE; ++i)
#pragma unroll
            for (int j = 0; j < ROUTER_EXPERT_GROUP; ++j) acc[i][j] = 0.f;
#pragma unroll 2
        for (int64_t k0 = (int64_t)lane * 8; k0 < d; k0 += 64 * 8) {
            const int kn = (d - k0 < 8) ? (int)(d - k0) : 8;
            float xv[ROUTER_TOKENS_PER_WAVE][8];
#pragma unroll
            for (int i = 0; i < ROUTER_TOKENS_PER_WAVE; ++i) {
                const int64_t t = (t0 + i < ntok) ? t0 + i : ntok - 1;
                load8<T>(x + t * ldx + k0, xv[i], kn, vec_ok);
            }
#pragma unroll
            for (int j = 0; j < ROUTER_EXPERT_GROUP; ++j) {
                const int e = (e0 + j < E) ? e0 + j : E - 1;
                float wv[8];
                load8<T>(wg + (int64_t)e * ldw + k0, wv, kn, vec_ok);
#pragma unroll
                for (int i = 0; i < ROUTER_TOKENS_PER_WAVE; ++i)
#pragma unroll
                    for (int u = 0; u < 8; ++u) acc[i][j] = fmaf(xv[i][u], wv[u], acc[i][j]);
            }
        }
#pragma unroll
        for (int i = 0; i < ROUTER_TOKENS_PER_WAVE; ++i)
#pragma unroll
            for (int j = 0; j < ROUTER_EXPERT_GROUP; ++j) {
                const float s = wave_sum(acc[i][j]);
                if (lane == 0 && t0 + i < ntok && e0 + j < E) logits[(t0 + i) * E + e0 + j] = s;
            }
    }
}

// fp32 softmax over the E logits of one token, k rounds of arg-max (strict '>' so the lowest expert index wins a
// tie), optional division by the sum of the selected scores.  s / topw / topi point at the token's output rows.
__device__ __forceinline__ void softmax_topk_token(const float* __restrict__ l, float* __restrict__ s,
                                                   float* __restrict__ topw, int32_t* __restrict__ topi, int E, int k,
                                                   int renorm)
{
    float mx = l[0];
    for (int e = 1; e < E; ++e) mx = fmaxf(mx, l[e]);
    float sum = 0.f;
    for (int e = 0; e < E; ++e) { const float v = expf(l[e] - mx); s[e] = v; sum += v; }
    for (int e = 0; e < E; ++e) s[e] = s[e] / sum;
    float wsum = 0.f;
    for (int j = 0; j < k; ++j) {
        int best = -1;
        float bv = 0.f;
        for (int e = 0; e < E; ++e) {
            bool taken = false;
            for (int jj = 0; jj < j; ++jj) taken |= (topi[jj] == e);
            if (taken) continue;
            const float v = s[e];
            if (best < 0 || v > bv) { best = e; bv = v; }
        }
        topi[j] = best;
        topw[j] = bv;
        wsum += bv;
    }
    if (renorm) for (int j = 0; j < k; ++j) topw[j] = topw[j] / wsum;
}

// One thread per token.
__global__ void router_topk_kernel(const float* __restrict__ logits, float* __restrict__ scores,
                                   float* __restrict__ topw, int32_t* __restrict__ topi, int64_t ntok, int E, int k,
                                   int renorm)
{
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= ntok) return;
    softmax_topk_token(logits + t * E, scores + t * E, topw + t * k, topi + t * k, E, k, renorm);
}

// Logits, softmax and top-k in one launch for up to ROUTER_EXPERT_GROUP experts of a 2-byte type, the logits on the
// matrix cores.  A workgroup of 8 waves handles 16 tokens; wave w takes the w-th eighth of the hidden dimension: it
// requests all of its operand fragments at once -- 16 bytes per lane straight from global memory in v_mfma_f32_16x16x32
// layout (lane i + 16 g holds row i, k = 8 g .. 8 g + 7 of a 32-wide step; rows are tokens for the activations and
// experts for the router weight, whose 64 KiB stay in L2) -- so the kernel pays one memory round trip, and then runs one
// MFMA per step.  With the weight fragment as first operand a lane ends up with 4 experts' partial logits of one
// token; the eight waves' partial sums meet in LDS and are added in wave order (fixed: the result does not depend on
// timing).  The summation order differs from router_logits_kernel's, so the two agree to fp32 rounding, not bit for bit.
constexpr int RM_WAVES = 8, RM_TOKENS = 16;
constexpr int RM_BATCH = 16;   // 32-wide K steps whose loads are in flight together (16 steps x 8 waves = 4096 columns)
template <typename T>
__global__ void __launch_bounds__(RM_WAVES * 64) router_mfma_kernel(const T* __restrict__ x, int64_t ldx,
                                                                    const T* __restrict__ wg, int64_t ldw,
                                                                    float* __restrict__ logits, float* __restrict__ scores,
                                                                    float* __restrict__ topw, int32_t* __restrict__ topi,
                                                                    int64_t ntok, int d, int E, int k, int renorm)
{
    __shared__ float s_part[RM_WAVES][RM_TOKENS][16];
    __shared__ float s_logits[RM_TOKENS][ROUTER_EXPERT_GROUP];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t t0 = (int64_t)blockIdx.x * RM_TOKENS;
    const int row = lane & 15, kc = lane >> 4;
    const int64_t tok = (t0 + row < ntok) ? t0 + row : ntok - 1;      // tokens past the end re-read the last one
    const T* xp = x + tok * ldx + kc * 8;
    const T* wp = wg + (int64_t)(row < E ? row : E - 1) * ldw + kc * 8;   // rows past the last expert enter as zeros
    const int nsteps = d / 32;
    const int s_end = nsteps * (wave + 1) / RM_WAVES;
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
    for (int s0 = nsteps * wave / RM_WAVES; s0 < s_end; s0 += RM_BATCH) {
        uint4 xa[RM_BATCH], wa[RM_BATCH];
#pragma unroll
        for (int i = 0; i < RM_BATCH; ++i) {
            const int st = (s0 + i < s_end) ? s0 + i : s_end - 1;
            xa[i] = *(const uint4*)(xp + (int64_t)st * 32);
            wa[i] = *(const uint4*)(wp + (int64_t)st * 32);
        }
#pragma unroll
        for (int i = 0; i < RM_BATCH; ++i) {
            if (s0 + i < s_end) {
                uint4 w4 = wa[i];
                if (row >= E) w4 = make_uint4(0, 0, 0, 0);
                if constexpr (sizeof(T) == 2 && std::is_same<T, __hip_bfloat16>::value) {
                    union { uint4 u; bf16x8_t v; } a, b;
                    a.u = w4; b.u = xa[i];
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, b.v, acc, 0, 0, 0);
                } else {
                    typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
                    union { uint4 u; f16x8_t v; } a, b;
                    a.u = w4; b.u = xa[i];
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a.v, b.v, acc, 0, 0, 0);
                }
            }
        }
    }
    // acc[r] = partial logit of token `row`, expert 4 * kc + r
    *(f32x4_t*)&s_part[wave][row][4 * kc] = acc;
    __syncthreads();
    if (tid < RM_TOKENS * ROUTER_EXPERT_GROUP) {
        const int t = tid / ROUTER_EXPERT_GROUP, e = tid % ROUTER_EXPERT_GROUP;
        float sum = s_part[0][t][e];
#pragma unroll
        for (int w = 1; w < RM_WAVES; ++w) sum += s_part[w][t][e];
        s_logits[t][e] = sum;
        if (e < E && t0 + t < ntok) logits[(t0 + t) * E + e] = sum;
    }
    __syncthreads();
    const int64_t t = t0 + tid;
    if (tid < RM_TOKENS && t < ntok) softmax_topk_token(s_logits[tid], scores + t * E, topw + t * k, topi + t * k, E, k, renorm);
}

// Backward of softmax -> top-k -> renormalise with respect to the logits.
// dw (T,k): gradient of the returned weights; w (T,k) the returned weights; scores (T,E) the softmax.
__global__ void router_bwd_kernel(const float* __restrict__ dw, const float* __restrict__ w,
                                  const int32_t* __restrict__ topi, const float* __restrict__ scores,
                                  float* __restrict__ dlogits, int64_t ntok, int E, int k, int renorm)
{
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= ntok) return;
    const float* s = scores + t * E;
    float* dl = dlogits + t * E;
    for (int e = 0; e < E; ++e) dl[e] = 0.f;
    // selected scores p_j = s[idx_j]; w_j = p_j / S (S = sum p) when renorm, else w_j = p_j
    float S = 1.f, dot = 0.f;
    if (renorm) {
        S = 0.f;
        for (int j = 0; j < k; ++j) S += s[topi[t * k + j]];
        for (int j = 0; j < k; ++j) dot += dw[t * k + j] * w[t * k + j];
    }
    float sdot = 0.f;  // sum_e dscore_e * s_e
    for (int j = 0; j < k; ++j) {
        const int e = topi[t * k + j];
        const float dp = renorm ? (dw[t * k + j] - dot) / S : dw[t * k + j];
        dl[e] = dp;  // holds dscore for the selected experts for now
        sdot += dp * s[e];
    }
    for (int e = 0; e < E; ++e) dl[e] = s[e] * (dl[e] - sdot);
}

// ---------------------------------------------------------------------------------------------------------
// stable counting sort by expert id
// ---------------------------------------------------------------------------------------------------------
constexpr int SORT_THREADS = 256;
constexpr int SORT_SCAN_LDS_INTS = 8192;   // chunk histograms the scan kernel keeps in LDS (32 KiB)
constexpr int SORT_CHUNK = 512;   // assignments per workgroup: small, so that a batch of a few thousand tokens still spreads over many compute units

__global__ void __launch_bounds__(SORT_THREADS) sort_hist_kernel(const void* __restrict__ expert_idx, int in64,
                                                                 int64_t R, int E, int32_t* __restrict__ block_hist)
{
    extern __shared__ int32_t sh[];
    for (int e = threadIdx.x; e < E; e += SORT_THREADS) sh[e] = 0;
    __syncthreads();
    const int64_t base = (int64_t)blockIdx.x * SORT_CHUNK;
    for (int i = threadIdx.x; i < SORT_CHUNK; i += SORT_THREADS) {
        const int64_t p = base + i;
        if (p < R) {
            const int64_t e = load_idx(expert_idx, p, in64);
            if (e >= 0 && e < E) atomicAdd(&sh[e], 1);  // ids outside [0,E) are left out of the sorted order
        }
    }
    __syncthreads();
    for (int e = threadIdx.x; e < E; e += SORT_THREADS) block_hist[(int64_t)blockIdx.x * E + e] = sh[e];
}

__device__ __forceinline__ void store_idx(void* p, int64_t i, int64_t v, int is64)
{
    if (is64) ((int64_t*)p)[i] = v; else ((int32_t*)p)[i] = (int32_t)v;
}

// Single workgroup: per-expert totals, exclusive bases per (expert, chunk) in expert-major order, inclusive
// offsets, and the table of block starts (block_m rows per block, blocks never straddle experts).
__global__ void __launch_bounds__(SORT_THREADS) sort_scan_kernel(int32_t* __restrict__ block_hist, int nblk, int E,
                                                                 int block_m, void* __restrict__ counts,
                                                                 void* __restrict__ offsets, int meta64,
                                                                 void* __restrict__ padded_blocks, int64_t padded_cap,
                                                                 int32_t* __restrict__ num_padded)
{
    extern __shared__ int32_t sh[];  // totals[E], then (when it fits) a copy of block_hist
    int32_t* hist = sh + E;
    const bool in_lds = (int64_t)nblk * E <= SORT_SCAN_LDS_INTS;
    // the running sums walk the chunks one after the other; from a copy in LDS that costs a few cycles per step
    // instead of a round trip to memory
    if (in_lds) {
        for (int i = threadIdx.x; i < nblk * E; i += SORT_THREADS) hist[i] = block_hist[i];
        __syncthreads();
    }
    for (int e = threadIdx.x; e < E; e += SORT_THREADS) {
        int32_t run = 0;
        if (in_lds) for (int b = 0; b < nblk; ++b) { const int32_t c = hist[b * E + e]; hist[b * E + e] = run; run += c; }
        else for (int b = 0; b < nblk; ++b) { const int32_t c = block_hist[(int64_t)b * E + e]; block_hist[(int64_t)b * E + e] = run; run += c; }
        sh[e] = run;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int64_t run = 0, nb = 0;
        for (int e = 0; e < E; ++e) {
            const int64_t c = sh[e];
            const int64_t start = run;
            run += c;
            if (counts) store_idx(counts, e, c, meta64);
            if (offsets) store_idx(offsets, e, run, meta64);
            sh[e] = (int32_t)start;
            if (padded_blocks)
                for (int64_t s = start; s < run; s += block_m) { if (nb < padded_cap) store_idx(padded_blocks, nb, s, meta64); ++nb; }
        }
        if (num_padded) *num_padded = (int32_t)nb;
    }
    __syncthreads();
    if (in_lds) for (int i = threadIdx.x; i < nblk * E; i += SORT_THREADS) block_hist[i] = hist[i] + sh[i % E];
    else for (int i = threadIdx.x; i < nblk * E; i += SORT_THREADS) block_hist[i] += sh[i % E];
}

// Each workgroup re-reads its chunk; wave w owns a contiguous slice of it and walks it 64 entries at a time so
// that destinations within one expert ascend with the flat position (stability).
__global__ void __launch_bounds__(SORT_THREADS) sort_scatter_kernel(const void* __restrict__ expert_idx, int in64,
                                                                    int64_t R, int E,
                                                                    const int32_t* __restrict__ block_base,
                                                                    void* __restrict__ sorted_expert,
                                                                    void* __restrict__ sorted_pos, int out64,
                                                                    int32_t* __restrict__ inv)
{
    extern __shared__ int32_t sh[];  // cursor[nwave][E]
    constexpr int NW = SORT_THREADS / 64;
    constexpr int PER_WAVE = SORT_CHUNK / NW;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    for (int i = threadIdx.x; i < NW * E; i += SORT_THREADS) sh[i] = 0;
    __syncthreads();
    const int64_t wbase = (int64_t)blockIdx.x * SORT_CHUNK + (int64_t)w * PER_WAVE;
    // pass 1: per-wave histogram
    for (int i = lane; i < PER_WAVE; i += 64) {
        const int64_t p = wbase + i;
        if (p < R) {
            const int64_t e = load_idx(expert_idx, p, in64);
            if (e >= 0 && e < E) atomicAdd(&sh[w * E + (int)e], 1);
        }
    }
    __syncthreads();
    // exclusive prefix over waves, seeded with this chunk's base
    for (int e = threadIdx.x; e < E; e += SORT_THREADS) {
        int32_t run = block_base[(int64_t)blockIdx.x * E + e];
        for (int ww = 0; ww < NW; ++ww) { const int32_t c = sh[ww * E + e]; sh[ww * E + e] = run; run += c; }
    }
    __syncthreads();
    // pass 2: ranked scatter
    volatile int32_t* cursor = sh + w * E;
    for (int i0 = 0; i0 < PER_WAVE; i0 += 64) {
        const int64_t p = wbase + i0 + lane;
        int e = -1;
        if (p < R) { const int64_t ee = load_idx(expert_idx, p, in64); e = (ee >= 0 && ee < E) ? (int)ee : -1; }
        uint64_t rem = __ballot(e >= 0);
        while (rem) {
            const int leader = __ffsll((unsigned long long)rem) - 1;
            const int e0 = __shfl(e, leader, 64);
            const uint64_t m = __ballot(e == e0);
            if (e == e0) {
                const int rank = __popcll(m & ((1ull << lane) - 1ull));
                const int32_t dst = cursor[e0] + rank;
                store_idx(sorted_expert, dst, e0, out64);
                store_idx(sorted_pos, dst, p, out64);
                if (inv) inv[p] = dst;
            }
            __builtin_amdgcn_wave_barrier();
            if (lane == leader) cursor[e0] += __popcll(m);
            __builtin_amdgcn_wave_barrier();
            rem &= ~m;
        }
    }
}

// The whole sort in one launch, for batches small enough that every workgroup can afford to read ALL assignment ids
// itself: a workgroup counts, per expert, the entries before its own chunk and the entries altogether (LDS atomics, each
// wave into its own rows), which gives it its chunk's destination bases without a histogram
// launch and a scan launch before it; then it scatters its chunk exactly as sort_scatter_kernel does.  Workgroup 0 also
// writes the per-expert counts, the inclusive offsets and the block table.  Same results as the three-launch path.
constexpr int64_t SORT_ONE_LAUNCH_MAX_ROWS = 16384;
constexpr int SORT_ONE_LAUNCH_MAX_EXPERTS = 256;
static_assert(SORT_CHUNK % 64 == 0, "a 64-entry group of the counting pass lies wholly before a chunk or not at all");
__global__ void __launch_bounds__(SORT_THREADS) sort_one_launch_kernel(const void* __restrict__ expert_idx, int in64,
                                                                       int64_t R, int E, int block_m,
                                                                       void* __restrict__ sorted_expert,
                                                                       void* __restrict__ sorted_pos, int out64,
                                                                       void* __restrict__ counts, void* __restrict__ offsets,
                                                                       void* __restrict__ padded_blocks, int64_t padded_cap,
                                                                       int32_t* __restrict__ num_padded, int32_t* __restrict__ inv)
{
    extern __shared__ int32_t sh[];  // before[NW][E], total[NW][E], then cursor[NW][E]
    constexpr int NW = SORT_THREADS / 64;
    constexpr int PER_WAVE = SORT_CHUNK / NW;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    int32_t* before = sh;
    int32_t* total = sh + NW * E;
    int32_t* cur = sh + 2 * NW * E;
    for (int i = threadIdx.x; i < 3 * NW * E; i += SORT_THREADS) sh[i] = 0;
    __syncthreads();
    const int64_t chunk_base = (int64_t)blockIdx.x * SORT_CHUNK;
    // counts over the whole array: wave w walks entries [64 (w + NW j), +64), sixteen groups' ids requested together;
    // LDS atomics into the wave's own rows (integer counts: the order of the additions does not matter)
    constexpr int SB = 16;
    for (int64_t p0 = (int64_t)w * 64; p0 < R; p0 += (int64_t)NW * 64 * SB) {
        int ev[SB];
        int64_t raw[SB];
        // (one branch on the index width around all the loads, so that they are in flight together; entries past the
        // end re-read the last one and are dropped below)
        if (in64) {
#pragma unroll
            for (int j = 0; j < SB; ++j) { const int64_t p = p0 + (int64_t)j * NW * 64 + lane; raw[j] = ((const int64_t*)expert_idx)[p < R ? p : R - 1]; }
        } else {
#pragma unroll
            for (int j = 0; j < SB; ++j) { const int64_t p = p0 + (int64_t)j * NW * 64 + lane; raw[j] = ((const int32_t*)expert_idx)[p < R ? p : R - 1]; }
        }
#pragma unroll
        for (int j = 0; j < SB; ++j) {
            const int64_t p = p0 + (int64_t)j * NW * 64 + lane;
            ev[j] = (p < R && raw[j] >= 0 && raw[j] < E) ? (int)raw[j] : -1;
        }
#pragma unroll
        for (int j = 0; j < SB; ++j) {
            if (ev[j] >= 0) {
                atomicAdd(&total[w * E + ev[j]], 1);
                // a 64-entry group lies wholly before the chunk or not at all (chunks are multiples of 64 entries)
                if (p0 + (int64_t)j * NW * 64 < chunk_base) atomicAdd(&before[w * E + ev[j]], 1);
            }
        }
    }
    // per-wave histogram of the own chunk (as in sort_scatter_kernel)
    const int64_t wbase = chunk_base + (int64_t)w * PER_WAVE;
    for (int i = lane; i < PER_WAVE; i += 64) {
        const int64_t p = wbase + i;
        if (p < R) {
            const int64_t e = load_idx(expert_idx, p, in64);
            if (e >= 0 && e < E) atomicAdd(&cur[w * E + (int)e], 1);
        }
    }
    __syncthreads();
    for (int e = threadIdx.x; e < E; e += SORT_THREADS) {
        int32_t b = 0, t = 0;
        for (int ww = 0; ww < NW; ++ww) { b += before[ww * E + e]; t += total[ww * E + e]; }
        before[e] = b;
        total[e] = t;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        // exclusive scan over the experts; workgroup 0 publishes counts, offsets and the block table
        const bool pub = blockIdx.x == 0;
        int64_t run = 0, nb = 0;
        for (int e = 0; e < E; ++e) {
            const int64_t c = total[e];
            const int64_t start = run;
            run += c;
            if (pub) {
                if (counts) store_idx(counts, e, c, out64);
                if (offsets) store_idx(offsets, e, run, out64);
                if (padded_blocks)
                    for (int64_t s_ = start; s_ < run; s_ += block_m) { if (nb < padded_cap) store_idx(padded_blocks, nb, s_, out64); ++nb; }
            }
            total[e] = (int32_t)start;
        }
        if (pub && num_padded) *num_padded = (int32_t)nb;
    }
    __syncthreads();
    // exclusive prefix over waves, seeded with this chunk's base = the expert's start + its entries before the chunk
    for (int e = threadIdx.x; e < E; e += SORT_THREADS) {
        int32_t run = total[e] + before[e];
        for (int ww = 0; ww < NW; ++ww) { const int32_t c = cur[ww * E + e]; cur[ww * E + e] = run; run += c; }
    }
    __syncthreads();
    volatile int32_t* cursor = cur + w * E;
    for (int i0 = 0; i0 < PER_WAVE; i0 += 64) {
        const int64_t p = wbase + i0 + lane;
        int e = -1;
        if (p < R) { const int64_t ee = load_idx(expert_idx, p, in64); e = (ee >= 0 && ee < E) ? (int)ee : -1; }
        uint64_t rem = __ballot(e >= 0);
        while (rem) {
            const int leader = __ffsll((unsigned long long)rem) - 1;
            const int e0 = __shfl(e, leader, 64);
            const uint64_t m = __ballot(e == e0);
            if (e == e0) {
                const int rank = __popcll(m & ((1ull << lane) - 1ull));
                const int32_t dst = cursor[e0] + rank;
                store_idx(sorted_expert, dst, e0, out64);
                store_idx(sorted_pos, dst, p, out64);
                if (inv) inv[p] = dst;
            }
            __builtin_amdgcn_wave_barrier();
            if (lane == leader) cursor[e0] += __popcll(m);
            __builtin_amdgcn_wave_barrier();
            rem &= ~m;
        }
    }
}

// offsets[e] = number of entries of the non-decreasing array sorted_expert that are <= e  (inclusive running count)
__global__ void offsets_from_sorted_kernel(const void* __restrict__ sorted_expert, int in64, int64_t R, int E,
                                           void* __restrict__ offsets, int out64)
{
    const int e = blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= E) return;
    int64_t lo = 0, hi = R;
    while (lo < hi) {
        const int64_t mid = (lo + hi) >> 1;
        if (load_idx(sorted_expert, mid, in64) <= e) lo = mid + 1; else hi = mid;
    }
    store_idx(offsets, e, lo, out64);
}

__global__ void padded_blocks_kernel(const void* __restrict__ offsets, int off64, int E, int block_m,
                                     void* __restrict__ padded_blocks, int out64, int64_t cap,
                                     int32_t* __restrict__ num_padded)
{
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    int64_t start = 0, nb = 0;
    for (int e = 0; e < E; ++e) {
        const int64_t end = load_idx(offsets, e, off64);
        for (int64_t s = start; s < end; s += block_m) { if (nb < cap) store_idx(padded_blocks, nb, s, out64); ++nb; }
        start = end;
    }
    *num_padded = (int32_t)nb;
}

}  // namespace

int moe_launch_router_logits(const void* x, int64_t ldx, const void* wg, int64_t ldw, int dtype, float* logits,
                             int64_t ntok, int64_t d, int E, hipStream_t stream)
{
    if (ntok == 0) return MOE_OK;
    const int64_t waves = (ntok + ROUTER_TOKENS_PER_WAVE - 1) / ROUTER_TOKENS_PER_WAVE;
    const unsigned grid = (unsigned)((waves + 3) / 4);
    const int64_t per16 = dtype == MOE_F32 ? 4 : 8;
    const bool vec_ok = ((uintptr_t)x % 16 == 0) && ((uintptr_t)wg % 16 == 0) && ldx % per16 == 0 && ldw % per16 == 0;
    MOE_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL((router_logits_kernel<T>), dim3(grid), dim3(256), 0, stream,
                                                 (const T*)x, ldx, (const T*)wg, ldw, logits, ntok, d, E, vec_ok));
    return moe_launch_status();
}

// logits + softmax + top-k; one launch when the router weight fits the fused kernel, otherwise the two kernels above
int moe_launch_router_forward(const void* x, int64_t ldx, const void* wg, int64_t ldw, int dtype, float* logits,
                              float* scores, float* topw, int32_t* topi, int64_t ntok, int64_t d, int E, int k,
                              int renorm, hipStream_t stream)
{
    if (ntok == 0) return MOE_OK;
    const bool fused = dtype != MOE_F32 && E <= ROUTER_EXPERT_GROUP && d % 32 == 0 && d >= 32 && d < (1 << 30) &&
                       ((uintptr_t)x % 16 == 0) && ((uintptr_t)wg % 16 == 0) && ldx % 8 == 0 && ldw % 8 == 0;
    if (!fused) {
        const int rc = moe_launch_router_logits(x, ldx, wg, ldw, dtype, logits, ntok, d, E, stream);
        return rc != MOE_OK ? rc : moe_launch_router_topk(logits, scores, topw, topi, ntok, E, k, renorm, stream);
    }
    const unsigned grid = (unsigned)((ntok + RM_TOKENS - 1) / RM_TOKENS);
    if (dtype == MOE_BF16)
        hipLaunchKernelGGL(router_mfma_kernel<__hip_bfloat16>, dim3(grid), dim3(RM_WAVES * 64), 0, stream, (const __hip_bfloat16*)x, ldx,
                           (const __hip_bfloat16*)wg, ldw, logits, scores, topw, topi, ntok, (int)d, E, k, renorm);
    else
        hipLaunchKernelGGL(router_mfma_kernel<__half>, dim3(grid), dim3(RM_WAVES * 64), 0, stream, (const __half*)x, ldx,
                           (const __half*)wg, ldw, logits, scores, topw, topi, ntok, (int)d, E, k, renorm);
    return moe_launch_status();
}

int moe_launch_router_topk(const float* logits, float* scores, float* topw, int32_t* topi, int64_t ntok, int E, int k,
                           int renorm, hipStream_t stream)
{
    if (ntok == 0) return MOE_OK;
    hipLaunchKernelGGL(router_topk_kernel, dim3((unsigned)((ntok + 255) / 256)), dim3(256), 0, stream, logits, scores,
                       topw, topi, ntok, E, k, renorm);
    return moe_launch_status();
}

int moe_launch_router_bwd(const float* dw, const float* w, const int32_t* topi, const float* scores, float* dlogits,
                          int64_t ntok, int E, int k, int renorm, hipStream_t stream)
{
    if (ntok == 0) return MOE_OK;
    hipLaunchKernelGGL(router_bwd_kernel, dim3((unsigned)((ntok + 255) / 256)), dim3(256), 0, stream, dw, w, topi,
                       scores, dlogits, ntok, E, k, renorm);
    return moe_launch_status();
}

size_t moe_sort_ws_bytes(int64_t R, int E)
{
    const int64_t nblk = (R + SORT_CHUNK - 1) / SORT_CHUNK;
    return (size_t)((nblk > 0 ? nblk : 1) * E + 4) * sizeof(int32_t);
}

int moe_launch_sort(const void* expert_idx, int in64, int64_t R, int E, int block_m, void* sorted_expert,
                    void* sorted_pos, int out64, void* counts, void* offsets, void* padded_blocks, int64_t padded_cap,
                    int32_t* num_padded, int32_t* inv, void* workspace, size_t workspace_bytes, hipStream_t stream)
{
    if (E < 1 || E > 4096 || R < 0 || block_m < 1) return MOE_ERR_BAD_ARG;
    if (workspace_bytes < moe_sort_ws_bytes(R, E)) return MOE_ERR_WORKSPACE;
    const int nblk = (int)((R + SORT_CHUNK - 1) / SORT_CHUNK);
    if (nblk > 0 && R <= SORT_ONE_LAUNCH_MAX_ROWS && E <= SORT_ONE_LAUNCH_MAX_EXPERTS) {
        hipLaunchKernelGGL(sort_one_launch_kernel, dim3(nblk), dim3(SORT_THREADS), 3 * (SORT_THREADS / 64) * E * sizeof(int32_t), stream,
                           expert_idx, in64, R, E, block_m, sorted_expert, sorted_pos, out64, counts, offsets, padded_blocks,
                           padded_cap, num_padded, inv);
        return moe_launch_status();
    }
    int32_t* hist = (int32_t*)workspace;
    if (nblk > 0)
        hipLaunchKernelGGL(sort_hist_kernel, dim3(nblk), dim3(SORT_THREADS), E * sizeof(int32_t), stream, expert_idx,
                           in64, R, E, hist);
    const size_t scan_lds = ((int64_t)nblk * E <= SORT_SCAN_LDS_INTS ? (size_t)E + (size_t)nblk * E : (size_t)E) * sizeof(int32_t);
    hipLaunchKernelGGL(sort_scan_kernel, dim3(1), dim3(SORT_THREADS), scan_lds, stream, hist, nblk, E,
                       block_m, counts, offsets, out64, padded_blocks, padded_cap, num_padded);
    if (nblk > 0)
        hipLaunchKernelGGL(sort_scatter_kernel, dim3(nblk), dim3(SORT_THREADS), (SORT_THREADS / 64) * E * sizeof(int32_t),
                           stream, expert_idx, in64, R, E, hist, sorted_expert, sorted_pos, out64, inv);
    return moe_launch_status();
}

// ---------------------------------------------------------------------------------------------------------
// The same sort for callers that cannot allocate or pass a workspace: the per-chunk histograms live in a static
// device array (each GPU the library runs on holds its own copy at its own address until the process ends).
// Every call on a GPU shares that GPU's array: calls that overlap on one GPU race.  Nothing in it has to start at
// zero -- the histogram launch writes every cell the later launches read.
// ---------------------------------------------------------------------------------------------------------
constexpr int64_t SORT_STATIC_INTS = 262144;   // 1 MiB: ceil(R / 512) * E + 4 cells at most
static __device__ __align__(256) int32_t scratch[SORT_STATIC_INTS];

constexpr int SORT_STATIC_MAX_DEVICES = 64;
static std::mutex g_scratch_mu;
static int32_t* g_scratch_ptr[SORT_STATIC_MAX_DEVICES] = {};

// Device address of `scratch` on the current device.  In host code the array's name is only a handle: the address a
// kernel may use comes from hipGetSymbolAddress, once per device with that device current.
static int sort_static_scratch(int32_t** out)
{
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= SORT_STATIC_MAX_DEVICES) return MOE_ERR_LAUNCH;
    std::lock_guard<std::mutex> lk(g_scratch_mu);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return MOE_ERR_LAUNCH;
        g_scratch_ptr[dev] = (int32_t*)p;
    }
    *out = g_scratch_ptr[dev];
    return MOE_OK;
}

size_t moe_sort_static_capacity_bytes() { return (size_t)SORT_STATIC_INTS * sizeof(int32_t); }

int moe_launch_sort_static(const void* expert_idx, int in64, int64_t R, int E, int block_m, void* sorted_expert,
                           void* sorted_pos, int out64, void* counts, void* offsets, void* padded_blocks,
                           int64_t padded_cap, int32_t* num_padded, int32_t* inv, hipStream_t stream)
{
    if (E < 1 || E > 4096 || R < 0 || block_m < 1) return MOE_ERR_BAD_ARG;
    if (moe_sort_ws_bytes(R, E) > moe_sort_static_capacity_bytes()) return MOE_ERR_WORKSPACE;
    int32_t* ptr = nullptr;
    const int rc = sort_static_scratch(&ptr);
    if (rc != MOE_OK) return rc;
    return moe_launch_sort(expert_idx, in64, R, E, block_m, sorted_expert, sorted_pos, out64, counts, offsets,
                           padded_blocks, padded_cap, num_padded, inv, ptr, moe_sort_static_capacity_bytes(), stream);
}

int moe_launch_offsets_from_sorted(const void* sorted_expert, int in64, int64_t R, int E, void* offsets, int out64,
                                   hipStream_t stream)
{
    hipLaunchKernelGGL(offsets_from_sorted_kernel, dim3((E + 63) / 64), dim3(64), 0, stream, sorted_expert, in64, R, E,
                       offsets, out64);
    return moe_launch_status();
}

int moe_launch_padded_blocks(const void* offsets, int off64, int E, int block_m, void* padded_blocks, int out64,
                             int64_t cap, int32_t* num_padded, hipStream_t stream)
{
    hipLaunchKernelGGL(padded_blocks_kernel, dim3(1), dim3(64), 0, stream, offsets, off64, E, block_m, padded_blocks,
                       out64, cap, num_padded);
    return moe_launch_status();
}
