// HBM-bound row kernels: gather rows into expert-grouped order, weighted combine of the k expert rows of a
// token (and its backward), fan-out reduction, SwiGLU.  Every output element is produced by exactly one
// thread with a fixed summation order, so results are deterministic.
#include "common.h"
#include "kernels.h"

namespace {

constexpr int ROW_THREADS = 256;

template <typename T> struct Vec8 { static constexpr int N = 16 / sizeof(T); };

template <typename T>
__device__ __forceinline__ void load_vec(const T* p, float* v, bool vec_ok, int n)
{
    constexpr int N = Vec8<T>::N;
    if (vec_ok) {
        uint4 raw = *(const uint4*)p;
        const T* e = (const T*)&raw;
#pragma unroll
        for (int i = 0; i < N; ++i) v[i] = Elem<T>::ld(e + i);
    } else {
        for (int i = 0; i < N; ++i) v[i] = (i < n) ? Elem<T>::ld(p + i) : 0.f;
    }
}
template <typename T>
__device__ __forceinline__ void store_vec(T* p, const float* v, bool vec_ok, int n)
{
    constexpr int N = Vec8<T>::N;
    if (vec_ok) {
        uint4 raw;
        T* e = (T*)&raw;
#pragma unroll
        for (int i = 0; i < N; ++i) Elem<T>::st(e + i, v[i]);
        *(uint4*)p = raw;
    } else {
        for (int i = 0; i < N && i < n; ++i) Elem<T>::st(p + i, v[i]);
    }
}

__device__ __forceinline__ float load_gate(const void* g, int64_t i, int gdtype)
{
    if (gdtype == MOE_F32) return ((const float*)g)[i];
    if (gdtype == MOE_BF16) return Elem<__hip_bfloat16>::ld((const __hip_bfloat16*)g + i);
    return Elem<__half>::ld((const __half*)g + i);
}
__device__ __forceinline__ void store_gate(void* g, int64_t i, float v, int gdtype)
{
    if (gdtype == MOE_F32) ((float*)g)[i] = v;
    else if (gdtype == MOE_BF16) Elem<__hip_bfloat16>::st((__hip_bfloat16*)g + i, v);
    else Elem<__half>::st((__half*)g + i, v);
}

// out[i][:] = src[pos[i] / fan_out][:] * coeff[pos[i]]      (one workgroup per output row)
template <typename T>
__global__ void __launch_bounds__(ROW_THREADS) group_rows_kernel(const T* __restrict__ src, int64_t lds_,
                                                                 T* __restrict__ out, int64_t ldo,
                                                                 const void* __restrict__ pos, int pos64, int fan_out,
                                                                 const void* __restrict__ coeff, int cdtype,
                                                                 int64_t nrows, int64_t ncols, int vec_ok)
{
    constexpr int N = Vec8<T>::N;
    const int64_t i = blockIdx.x;
    const int64_t p = load_idx(pos, i, pos64);
    const T* s = src + (p / fan_out) * lds_;
    T* o = out + i * ldo;
    const float c = coeff ? load_gate(coeff, p, cdtype) : 1.f;
    for (int64_t c0 = (int64_t)threadIdx.x * N; c0 < ncols; c0 += (int64_t)ROW_THREADS * N) {
        float v[N];
        const int n = (ncols - c0 < N) ? (int)(ncols - c0) : N;
        const bool vo = vec_ok && n == N;
        load_vec<T>(s + c0, v, vo, n);
        if (coeff) {
#pragma unroll
            for (int u = 0; u < N; ++u) v[u] *= c;
        }
        store_vec<T>(o + c0, v, vo, n);
    }
}

// out[t][:] = sum_j gates[t*k+j] * y[row(t,j)][:],  row(t,j) = inv ? inv[t*k+j] : t*k+j.   gates may be null (=1).
template <typename T>
__global__ void __launch_bounds__(ROW_THREADS) combine_fwd_kernel(const T* __restrict__ y, int64_t ldy,
                                                                  T* __restrict__ out, int64_t ldo,
                                                                  const void* __restrict__ gates, int gdtype,
                                                                  const int32_t* __restrict__ inv, int k,
                                                                  int64_t ncols, int vec_ok,
                                                                  const float* __restrict__ extra_coef,
                                                                  const T* __restrict__ extra_rows, int64_t lde,
                                                                  int n_extra)
{
    constexpr int N = Vec8<T>::N;
    const int64_t t = blockIdx.x;
    for (int64_t c0 = (int64_t)threadIdx.x * N; c0 < ncols; c0 += (int64_t)ROW_THREADS * N) {
        const int n = (ncols - c0 < N) ? (int)(ncols - c0) : N;
        const bool vo = vec_ok && n == N;
        float acc[N];
#pragma unroll
        for (int u = 0; u < N; ++u) acc[u] = 0.f;
        for (int j = 0; j < k; ++j) {
            const int64_t row = inv ? (int64_t)inv[t * k + j] : t * k + j;
            const float g = gates ? load_gate(gates, t * k + j, gdtype) : 1.f;
            float v[N];
            load_vec<T>(y + row * ldy + c0, v, vo, n);
#pragma unroll
            for (int u = 0; u < N; ++u) acc[u] = fmaf(g, v[u], acc[u]);
        }
        // optional dense tail: + sum_e extra_coef[t][e] * extra_rows[e][:]   (router input gradient)
        for (int e = 0; e < n_extra; ++e) {
            const float g = extra_coef[t * n_extra + e];
            float v[N];
            load_vec<T>(extra_rows + (int64_t)e * lde + c0, v, vo, n);
#pragma unroll
            for (int u = 0; u < N; ++u) acc[u] = fmaf(g, v[u], acc[u]);
        }
        store_vec<T>(out + t * ldo + c0, acc, vo, n);
    }
}

// The same sum for whole 16-byte columns and k <= KMAX: the k row numbers and weights of the token are fetched first,
// then the k rows' loads of a column chunk are all in flight before the first of them is used -- one trip to memory per
// chunk instead of one per row (rows j >= k re-read row 0 with weight 0).  The summation order is unchanged.
template <typename T, int KMAX>
__global__ void __launch_bounds__(ROW_THREADS) combine_fwd_batched_kernel(const T* __restrict__ y, int64_t ldy,
                                                                          T* __restrict__ out, int64_t ldo,
                                                                          const void* __restrict__ gates, int gdtype,
                                                                          const int32_t* __restrict__ inv, int k,
                                                                          int64_t ncols,
                                                                          const float* __restrict__ extra_coef,
                                                                          const T* __restrict__ extra_rows, int64_t lde,
                                                                          int n_extra)
{
    constexpr int N = Vec8<T>::N;
    const int64_t t = blockIdx.x;
    const T* rowp[KMAX];
    float g[KMAX];
#pragma unroll
    for (int j = 0; j < KMAX; ++j) {
        const int64_t idx = t * k + (j < k ? j : 0);
        const int64_t row = inv ? (int64_t)inv[idx] : idx;
        rowp[j] = y + row * ldy;
        g[j] = j < k ? (gates ? load_gate(gates, idx, gdtype) : 1.f) : 0.f;
    }
#pragma unroll 2
    for (int64_t c0 = (int64_t)threadIdx.x * N; c0 < ncols; c0 += (int64_t)ROW_THREADS * N) {
        uint4 raw[KMAX];
#pragma unroll
        for (int j = 0; j < KMAX; ++j) raw[j] = *(const uint4*)(rowp[j] + c0);
        float acc[N];
#pragma unroll
        for (int u = 0; u < N; ++u) acc[u] = 0.f;
#pragma unroll
        for (int j = 0; j < KMAX; ++j) {
            const T* e = (const T*)&raw[j];
#pragma unroll
            for (int u = 0; u < N; ++u) acc[u] = fmaf(g[j], Elem<T>::ld(e + u), acc[u]);
        }
        for (int e = 0; e < n_extra; ++e) {
            const float ge = extra_coef[t * n_extra + e];
            float v[N];
            load_vec<T>(extra_rows + (int64_t)e * lde + c0, v, true, N);
#pragma unroll
            for (int u = 0; u < N; ++u) acc[u] = fmaf(ge, v[u], acc[u]);
        }
        store_vec<T>(out + t * ldo + c0, acc, true, N);
    }
}

// dgates[t*k+j] = <y[row(t,j)], dout[t]>   (one wave per (t,j))
template <typename T>
__global__ void __launch_bounds__(ROW_THREADS) combine_dgates_kernel(const T* __restrict__ y, int64_t ldy,
                                                                     const T* __restrict__ dout, int64_t ldd,
                                                                     void* __restrict__ dgates, int gdtype,
                                                                     const int32_t* __restrict__ inv, int k,
                                                                     int64_t npairs, int64_t ncols, int vec_ok)
{
    constexpr int N = Vec8<T>::N;
    const int lane = threadIdx.x & 63;
    const int64_t pair = (int64_t)blockIdx.x * (ROW_THREADS / 64) + (threadIdx.x >> 6);
    if (pair >= npairs) return;
    const int64_t t = pair / k;
    const int64_t row = inv ? (int64_t)inv[pair] : pair;
    float acc = 0.f;
    for (int64_t c0 = (int64_t)lane * N; c0 < ncols; c0 += 64 * N) {
        const int n = (ncols - c0 < N) ? (int)(ncols - c0) : N;
        const bool vo = vec_ok && n == N;
        float a[N], b[N];
        load_vec<T>(y + row * ldy + c0, a, vo, n);
        load_vec<T>(dout + t * ldd + c0, b, vo, n);
#pragma unroll
        for (int u = 0; u < N; ++u) acc = fmaf(a[u], b[u], acc);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) acc += __shfl_xor(acc, o, 64);
    if (lane == 0) store_gate(dgates, pair, acc, gdtype);
}

// h = silu(g) * u   elementwise over (rows, cols)
template <typename T>
__global__ void __launch_bounds__(ROW_THREADS) swiglu_fwd_kernel(const T* __restrict__ g, const T* __restrict__ u,
                                                                 T* __restrict__ h, int64_t n)
{
    const int64_t i = (int64_t)blockIdx.x * ROW_THREADS + threadIdx.x;
    if (i >= n) return;
    const float gv = Elem<T>::ld(g + i), uv = Elem<T>::ld(u + i);
    Elem<T>::st(h + i, gv / (1.f + __expf(-gv)) * uv);
}

// dg = dh * u * sig(g) * (1 + g * (1 - sig(g))),  du = dh * silu(g)
template <typename T>
__global__ void __launch_bounds__(ROW_THREADS) swiglu_bwd_kernel(const T* __restrict__ g, const T* __restrict__ u,
                                                                 const T* __restrict__ dh, T* __restrict__ dg,
                                                                 T* __restrict__ du, int64_t n)
{
    const int64_t i = (int64_t)blockIdx.x * ROW_THREADS + threadIdx.x;
    if (i >= n) return;
    const float gv = Elem<T>::ld(g + i), uv = Elem<T>::ld(u + i), d = Elem<T>::ld(dh + i);
    const float sg = 1.f / (1.f + __expf(-gv));
    Elem<T>::st(dg + i, d * uv * sg * (1.f + gv * (1.f - sg)));
    Elem<T>::st(du + i, d * gv * sg);
}

// Router weight gradient dWg[e][c] = sum_t dlogits[t][e] * x[t][c], fp32 coefficients (no rounding of dlogits), fp32
// accumulate.  Pass 1: workgroup (chunk, column block) sums its WG_TOKENS tokens for every expert, a thread owning N
// consecutive columns (one 16-byte load per token) and EG experts at a time; partial[chunk][e][c] fp32.  Pass 2 adds the
// chunks in order (deterministic) and rounds once to the storage type.
constexpr int WG_TOKENS = 64;   // tokens per partial
constexpr int WG_EG = 8;        // experts per register block
template <typename T>
__global__ void __launch_bounds__(ROW_THREADS) router_wgrad_partial_kernel(const T* __restrict__ x, int64_t ldx,
                                                                           const float* __restrict__ dl, int64_t ntok,
                                                                           int64_t d, int E, float* __restrict__ partial,
                                                                           int vec_ok)
{
    constexpr int N = Vec8<T>::N;
    __shared__ float s_dl[WG_TOKENS * WG_EG];
    const int64_t t0 = (int64_t)blockIdx.x * WG_TOKENS;
    const int nt = (ntok - t0 < WG_TOKENS) ? (int)(ntok - t0) : WG_TOKENS;
    const int64_t c0 = ((int64_t)blockIdx.y * ROW_THREADS + threadIdx.x) * N;
    const int n = (d - c0 < N) ? (int)(d - c0) : N;
    const bool vo = vec_ok && n == N;
    for (int e0 = 0; e0 < E; e0 += WG_EG) {
        const int ne = (E - e0 < WG_EG) ? E - e0 : WG_EG;
        __syncthreads();
        for (int i = threadIdx.x; i < WG_TOKENS * WG_EG; i += ROW_THREADS) {
            const int tt = i / WG_EG, ee = i % WG_EG;
            s_dl[i] = (tt < nt && ee < ne) ? dl[(t0 + tt) * E + e0 + ee] : 0.f;
        }
        __syncthreads();
        if (c0 >= d) continue;
        float acc[WG_EG][N];
#pragma unroll
        for (int ee = 0; ee < WG_EG; ++ee)
#pragma unroll
            for (int u = 0; u < N; ++u) acc[ee][u] = 0.f;
        for (int tt = 0; tt < nt; ++tt) {
            float v[N];
            load_vec<T>(x + (t0 + tt) * ldx + c0, v, vo, n);
#pragma unroll
            for (int ee = 0; ee < WG_EG; ++ee) {
                const float g = s_dl[tt * WG_EG + ee];
#pragma unroll
                for (int u = 0; u < N; ++u) acc[ee][u] = fmaf(g, v[u], acc[ee][u]);
            }
        }
        for (int ee = 0; ee < ne; ++ee)
            for (int u = 0; u < n; ++u) partial[((int64_t)blockIdx.x * E + e0 + ee) * d + c0 + u] = acc[ee][u];
    }
}

template <typename T>
__global__ void __launch_bounds__(ROW_THREADS) router_wgrad_reduce_kernel(const float* __restrict__ partial, int nchunk,
                                                                          int64_t total, int64_t d, T* __restrict__ out,
                                                                          int64_t ldo)
{
    const int64_t i = (int64_t)blockIdx.x * ROW_THREADS + threadIdx.x;   // (e, c) flattened
    if (i >= total) return;
    float acc = 0.f;
    for (int ch = 0; ch < nchunk; ++ch) acc += partial[(int64_t)ch * total + i];
    Elem<T>::st(out + (i / d) * ldo + i % d, acc);
}

template <typename T> bool vec_aligned(const void* p, int64_t ld)
{
    return ((uintptr_t)p % 16 == 0) && (ld % (16 / sizeof(T)) == 0);
}

}  // namespace

int moe_launch_group_rows(const void* src, int64_t lds_, void* out, int64_t ldo, const void* pos, int pos64,
                          int fan_out, const void* coeff, int cdtype, int64_t nrows, int64_t ncols, int dtype,
                          hipStream_t stream)
{
    if (nrows == 0 || ncols == 0) return MOE_OK;
    if (fan_out < 1) return MOE_ERR_BAD_ARG;
    MOE_DISPATCH_DTYPE(dtype, {
        const int vo = vec_aligned<T>(src, lds_) && vec_aligned<T>(out, ldo);
        hipLaunchKernelGGL((group_rows_kernel<T>), dim3((unsigned)nrows), dim3(ROW_THREADS), 0, stream, (const T*)src,
                           lds_, (T*)out, ldo, pos, pos64, fan_out, coeff, cdtype, nrows, ncols, vo);
    });
    return moe_launch_status();
}

int moe_launch_combine_fwd(const void* y, int64_t ldy, void* out, int64_t ldo, const void* gates, int gdtype,
                           const int32_t* inv, int k, int64_t ntok, int64_t ncols, int dtype,
                           const float* extra_coef, const void* extra_rows, int64_t lde, int n_extra,
                           hipStream_t stream)
{
    if (ntok == 0 || ncols == 0) return MOE_OK;
    MOE_DISPATCH_DTYPE(dtype, {
        const int vo = vec_aligned<T>(y, ldy) && vec_aligned<T>(out, ldo) && (!extra_rows || vec_aligned<T>(extra_rows, lde));
        if (vo && k >= 1 && k <= 8 && ncols % Vec8<T>::N == 0) {
            auto kern = k <= 2 ? combine_fwd_batched_kernel<T, 2> : (k <= 4 ? combine_fwd_batched_kernel<T, 4> : combine_fwd_batched_kernel<T, 8>);
            hipLaunchKernelGGL(kern, dim3((unsigned)ntok), dim3(ROW_THREADS), 0, stream, (const T*)y, ldy, (T*)out, ldo, gates, gdtype,
                               inv, k, ncols, extra_coef, (const T*)extra_rows, lde, n_extra);
        } else
        hipLaunchKernelGGL((combine_fwd_kernel<T>), dim3((unsigned)ntok), dim3(ROW_THREADS), 0, stream, (const T*)y,
                           ldy, (T*)out, ldo, gates, gdtype, inv, k, ncols, vo, extra_coef, (const T*)extra_rows, lde,
                           n_extra);
    });
    return moe_launch_status();
}

int moe_launch_combine_dgates(const void* y, int64_t ldy, const void* dout, int64_t ldd, void* dgates, int gdtype,
                              const int32_t* inv, int k, int64_t ntok, int64_t ncols, int dtype, hipStream_t stream)
{
    if (ntok == 0) return MOE_OK;
    const int64_t npairs = ntok * k;
    MOE_DISPATCH_DTYPE(dtype, {
        const int vo = vec_aligned<T>(y, ldy) && vec_aligned<T>(dout, ldd);
        hipLaunchKernelGGL((combine_dgates_kernel<T>), dim3((unsigned)((npairs + 3) / 4)), dim3(ROW_THREADS), 0, stream,
                           (const T*)y, ldy, (const T*)dout, ldd, dgates, gdtype, inv, k, npairs, ncols, vo);
    });
    return moe_launch_status();
}

int moe_launch_swiglu_fwd(const void* g, const void* u, void* h, int64_t n, int dtype, hipStream_t stream)
{
    if (n == 0) return MOE_OK;
    MOE_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL((swiglu_fwd_kernel<T>), dim3((unsigned)((n + ROW_THREADS - 1) / ROW_THREADS)),
                                                 dim3(ROW_THREADS), 0, stream, (const T*)g, (const T*)u, (T*)h, n));
    return moe_launch_status();
}

int moe_launch_swiglu_bwd(const void* g, const void* u, const void* dh, void* dg, void* du, int64_t n, int dtype,
                          hipStream_t stream)
{
    if (n == 0) return MOE_OK;
    MOE_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL((swiglu_bwd_kernel<T>), dim3((unsigned)((n + ROW_THREADS - 1) / ROW_THREADS)),
                                                 dim3(ROW_THREADS), 0, stream, (const T*)g, (const T*)u, (const T*)dh,
                                                 (T*)dg, (T*)du, n));
    return moe_launch_status();
}

size_t moe_router_wgrad_ws_bytes(int64_t ntok, int64_t d, int E)
{
    const int64_t nchunk = (ntok + WG_TOKENS - 1) / WG_TOKENS;
    return (size_t)(nchunk > 0 ? nchunk : 1) * (size_t)E * (size_t)d * sizeof(float);
}

int moe_launch_router_wgrad(const void* x, int64_t ldx, const float* dlogits, void* dwg, int64_t ldo, int64_t ntok,
                            int64_t d, int E, int dtype, void* workspace, size_t workspace_bytes, hipStream_t stream)
{
    if (d == 0 || E == 0) return MOE_OK;
    if (workspace_bytes < moe_router_wgrad_ws_bytes(ntok, d, E)) return MOE_ERR_WORKSPACE;
    const int64_t nchunk = (ntok + WG_TOKENS - 1) / WG_TOKENS;
    const int64_t total = (int64_t)E * d;
    MOE_DISPATCH_DTYPE(dtype, {
        constexpr int N = Vec8<T>::N;
        const int vo = vec_aligned<T>(x, ldx);
        if (nchunk > 0)
            hipLaunchKernelGGL((router_wgrad_partial_kernel<T>), dim3((unsigned)nchunk, (unsigned)((d + ROW_THREADS * N - 1) / (ROW_THREADS * N))),
                               dim3(ROW_THREADS), 0, stream, (const T*)x, ldx, dlogits, ntok, d, E, (float*)workspace, vo);
        hipLaunchKernelGGL((router_wgrad_reduce_kernel<T>), dim3((unsigned)((total + ROW_THREADS - 1) / ROW_THREADS)), dim3(ROW_THREADS), 0,
                           stream, (const float*)workspace, (int)nchunk, total, d, (T*)dwg, ldo);
    });
    return moe_launch_status();
}
