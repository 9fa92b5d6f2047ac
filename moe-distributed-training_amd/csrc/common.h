// Shared definitions for the gfx950 kernels of the dropless MoE expert-MLP path.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <atomic>

// status codes returned by every C-ABI entry point (see include/moe_hip.h)
#define MOE_OK 0
#define MOE_ERR_BAD_ARG (-1)
#define MOE_ERR_UNSUPPORTED (-2)
#define MOE_ERR_WORKSPACE (-3)
#define MOE_ERR_LAUNCH (-4)

// element types
#define MOE_BF16 0
#define MOE_F16 1
#define MOE_F32 2

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;
typedef __attribute__((__vector_size__(4 * sizeof(short)))) short s16x4_t;

#define LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))
#define GLB_PTR(p) ((const __attribute__((address_space(1))) void*)(p))

__device__ __forceinline__ int64_t load_idx(const void* p, int64_t i, int is64)
{
    return is64 ? ((const int64_t*)p)[i] : (int64_t)((const int32_t*)p)[i];
}

// float <-> storage conversions (round to nearest even for bf16)
__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) { return __uint_as_float(((uint32_t)b) << 16); }
// fp32 -> bf16, round to nearest even, through the hardware's packed conversion (v_cvt_pk_bf16_f32)
typedef __bf16 moe_bf16x2_t __attribute__((ext_vector_type(2)));
typedef float moe_f32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi)
{
    const moe_f32x2_t v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, moe_bf16x2_t));
}
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) { return (uint16_t)pack_bf16x2(f, 0.f); }

// The matrix-core kernels are written once for both 16-bit storage types: a policy type says how 16 bits become a
// float, how two floats are rounded (to nearest even) into a packed pair, and which 16x16x32 MFMA takes the
// fragments.  Fragments travel as bf16x8_t whatever they hold (16 bytes per lane).
typedef _Float16 moe_f16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 moe_f16x2_t __attribute__((ext_vector_type(2)));
struct NumBf16 {
    static constexpr int dtype = MOE_BF16;
    static __device__ __forceinline__ float to_f32(uint16_t b) { return bf16_bits_to_f32(b); }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) { return pack_bf16x2(lo, hi); }
    static __device__ __forceinline__ uint16_t from_f32(float f) { return f32_to_bf16_bits(f); }
    // rounds a pair to storage precision in place
    static __device__ __forceinline__ void round2(float& a, float& b)
    {
        const uint32_t w = pack_bf16x2(a, b);
        a = __uint_as_float(w << 16);
        b = __uint_as_float(w & 0xffff0000u);
    }
    static __device__ __forceinline__ f32x4_t mfma(bf16x8_t a, bf16x8_t b, f32x4_t c) { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0); }
};
struct NumF16 {
    static constexpr int dtype = MOE_F16;
    static __device__ __forceinline__ float to_f32(uint16_t b) { return (float)__builtin_bit_cast(_Float16, b); }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi)
    {
        const moe_f32x2_t v = {lo, hi};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, moe_f16x2_t));
    }
    static __device__ __forceinline__ uint16_t from_f32(float f) { return __builtin_bit_cast(uint16_t, (_Float16)f); }
    static __device__ __forceinline__ void round2(float& a, float& b)
    {
        a = (float)(_Float16)a;
        b = (float)(_Float16)b;
    }
    static __device__ __forceinline__ f32x4_t mfma(bf16x8_t a, bf16x8_t b, f32x4_t c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(moe_f16x8_t, a), __builtin_bit_cast(moe_f16x8_t, b), c, 0, 0, 0);
    }
};

template <typename T> struct Elem;
template <> struct Elem<float> {
    static __device__ __forceinline__ float ld(const float* p) { return *p; }
    static __device__ __forceinline__ void st(float* p, float v) { *p = v; }
};
template <> struct Elem<__hip_bfloat16> {
    static __device__ __forceinline__ float ld(const __hip_bfloat16* p) { return bf16_bits_to_f32(*(const uint16_t*)p); }
    static __device__ __forceinline__ void st(__hip_bfloat16* p, float v) { *(uint16_t*)p = f32_to_bf16_bits(v); }
};
template <> struct Elem<__half> {
    static __device__ __forceinline__ float ld(const __half* p) { return __half2float(*p); }
    static __device__ __forceinline__ void st(__half* p, float v) { *p = __float2half(v); }
};

// a 64-bit value that is the same in every lane, moved to scalar registers
__device__ __forceinline__ int64_t uniform_i64(int64_t v)
{
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)((uint64_t)v >> 32));
    return (int64_t)(((uint64_t)hi << 32) | lo);
}

// Row tiles of ragged expert groups: offsets[e] is the inclusive running row count, tiles of bm rows never straddle
// two experts.  For up to 64 experts one wave looks at all groups at once -- lane e loads offsets[e], a wave-wide
// prefix sum gives every group's first tile -- so that finding a tile costs one memory round trip instead of one per
// expert.  Must be called with all 64 lanes of the wave active (one-dimensional workgroups).
struct ExpertScan {
    int64_t start, end;                   // rows of group `lane` (lanes >= E: empty)
    int64_t tiles_before, tiles_through;  // exclusive / inclusive running tile count
};
__device__ __forceinline__ ExpertScan scan_expert_tiles(const void* offsets, int off64, int E, int bm)
{
    const int lane = threadIdx.x & 63;
    const int64_t end = load_idx(offsets, lane < E ? lane : E - 1, off64);
    int64_t start = __shfl_up(end, 1);
    if (lane == 0) start = 0;
    const int64_t nt = lane < E ? (end - start + bm - 1) / bm : 0;
    int64_t incl = nt;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const int64_t t = __shfl_up(incl, d);
        if (lane >= d) incl += t;
    }
    ExpertScan s;
    s.start = start; s.end = end; s.tiles_before = incl - nt; s.tiles_through = incl;
    return s;
}

// Maps a linear row-tile id (uniform over the wave) onto (expert, first row, one-past-last row).
struct RowTile { int expert; int64_t row0; int64_t row1; };
__device__ __forceinline__ bool find_row_tile(const void* offsets, int off64, int E, int bm, int64_t tile, RowTile* out)
{
    if (E <= 64) {
        const int lane = threadIdx.x & 63;
        const ExpertScan s = scan_expert_tiles(offsets, off64, E, bm);
        const unsigned long long hit = __ballot(lane < E && tile >= s.tiles_before && tile < s.tiles_through);
        if (hit == 0) return false;
        const int e = __ffsll(hit) - 1;
        const int64_t end = __shfl(s.end, e);
        out->expert = e;
        out->row0 = __shfl(s.start, e) + (tile - __shfl(s.tiles_before, e)) * bm;
        out->row1 = (out->row0 + bm < end) ? out->row0 + bm : end;
        return true;
    }
    int64_t start = 0;
    for (int e = 0; e < E; ++e) {
        int64_t end = load_idx(offsets, e, off64);
        int64_t nt = (end - start + bm - 1) / bm;
        if (tile < nt) {
            out->expert = e;
            out->row0 = start + tile * bm;
            out->row1 = (out->row0 + bm < end) ? out->row0 + bm : end;
            return true;
        }
        tile -= nt;
        start = end;
    }
    return false;
}

#define MOE_DISPATCH_DTYPE(dtype, ...)                                                   \
    do {                                                                                 \
        if ((dtype) == MOE_BF16) { typedef __hip_bfloat16 T; __VA_ARGS__; }              \
        else if ((dtype) == MOE_F16) { typedef __half T; __VA_ARGS__; }                  \
        else if ((dtype) == MOE_F32) { typedef float T; __VA_ARGS__; }                   \
        else return MOE_ERR_BAD_ARG;                                                     \
    } while (0)

// Per-device caches (dynamic LDS opt-in done, compute-unit count) are indexed by the HIP device ordinal.
constexpr int MOE_MAX_DEVICES = 64;
static inline int moe_current_device()
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MOE_MAX_DEVICES) dev = 0;
    return dev;
}
// compute units of the current device, looked up once per device
static inline int moe_device_cus()
{
    static std::atomic<int> cus[MOE_MAX_DEVICES];
    const int dev = moe_current_device();
    int n = cus[dev];
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n < 1) n = 256;
        cus[dev] = n;
    }
    return n;
}

static inline int moe_launch_status()
{
    return hipGetLastError() == hipSuccess ? MOE_OK : MOE_ERR_LAUNCH;
}
