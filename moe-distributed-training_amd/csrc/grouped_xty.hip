// Per-expert weight gradient of the ragged grouped GEMM on the gfx950 matrix cores (bf16 in, fp32 accumulate, bf16 out):
//
//   DW[e][k][n] = sum over the rows m of expert e's group  X[m][k] * DY[m][n]
//
// (scattermoe.kernels.ops.group_bwd_W, selected by the reference at megablocks_utils/config_utils.py:124-125 when an
// expert projection carries no adapters, i.e. full fine-tuning.)  X and DY are in expert-grouped order; a group's rows
// are the contraction dimension, so the raggedness sits in the loop count of a tile, not in its shape, and an empty
// group yields a tile of zeros.
//
// Tiling: 256 (k) x 256 (n) output tile per workgroup, contraction in steps of 64 rows, 8 waves (2 x 4) of 128 x 64 =
// 8 x 4 MFMA 16x16x32 tiles.  Both operands are stored with the contraction index as the slow one, so both travel
// HBM -> LDS as [64 rows][256 columns] images (direct-to-LDS 16-byte loads, two stages) and both are read back
// transposed with ds_read_b64_tr_b16.  The loads go through buffer descriptors whose range ends at the group's last
// row: rows past it read as zeros and contribute nothing, so the last, partial step needs no special case.
#include "common.h"
#include "kernels.h"

namespace {

constexpr int BM = 256, BN = 256, BR = 64;
constexpr int NWAVES = 8, NTHREADS = NWAVES * 64;
constexpr int WAVES_N = 4;
constexpr int WTM = 128, WTN = 64;
constexpr int MB = WTM / 16, NB = WTN / 16, MBH = MB / 2;   // 16x16 blocks per wave; a wave works on half its rows at a time
constexpr int LPT = 32 / NWAVES;                 // load instructions per wave, operand and contraction step
constexpr int OP_BYTES = BM * BR * 2;            // 32 KiB (BM == BN)
constexpr int STAGE_BYTES = 2 * OP_BYTES;
constexpr int LDS_BYTES = 2 * STAGE_BYTES;
constexpr int NXCD = 8;
constexpr int PANEL = 8;                         // n tiles that consecutive work items walk before moving to the next k tile
constexpr uint32_t OUT_OF_RANGE = 0x80000000u;   // beyond any descriptor range used here

typedef int i32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

// 16 bytes per lane, global -> LDS: lane l's data lands at lds_addr + 16*l; lanes whose offset lies outside the
// descriptor's range deliver zeros.
__device__ __forceinline__ void load_to_lds_16(i32x4_t rsrc, uint32_t lane_off, uint32_t lds_addr)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds" ::"s"(lds_addr), "v"(lane_off), "s"(rsrc) : "memory", "m0");
}

template <typename Num>
__global__ void __launch_bounds__(NTHREADS) grouped_xty_mfma_kernel(const MoeXtyParams p)
{
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;

    // ---- work item -> (expert, k tile, n tile).  Every expert has the same number of tiles, but a tile costs as much
    // as its group has rows, so each expert's tiles are dealt out evenly to the 8 XCDs (blockIdx round-robins over
    // them): every XCD gets a contiguous eighth of every expert, and skewed group sizes load all XCDs alike.  Within
    // that range consecutive items walk a panel of PANEL n tiles per k tile, so the tiles that run side by side on an
    // XCD share their operand columns in its L2.
    const int mt_n = (int)((p.K + BM - 1) / BM), nt_n = (int)((p.N + BN - 1) / BN);
    const int per_e = mt_n * nt_n;
    const int per_x = (per_e + NXCD - 1) / NXCD;           // tiles of one expert on one XCD
    const int64_t q = blockIdx.x / NXCD;
    const int expert = (int)(q / per_x);
    const int local = (int)(blockIdx.x % NXCD) * per_x + (int)(q % per_x);
    if (expert >= p.E || local >= per_e) return;
    const int panel = local / (mt_n * PANEL);
    const int width = (nt_n - panel * PANEL < PANEL) ? nt_n - panel * PANEL : PANEL;
    const int in_panel = local - panel * mt_n * PANEL;
    const int mt = in_panel / width, nt = panel * PANEL + in_panel % width;
    const int64_t m0 = (int64_t)mt * BM, n0 = (int64_t)nt * BN;

    const int64_t start = expert ? load_idx(p.offsets, expert - 1, p.off64) : 0;
    const int64_t end = load_idx(p.offsets, expert, p.off64);
    const int nrows = (int)__builtin_amdgcn_readfirstlane((int)(end - start));
    const int ke = (nrows + BR - 1) / BR;

    // ---- per-lane source offsets.  Image of one operand: [64 rows][32 chunks of 8 columns]; chunk (r, c) sits at
    // slot c ^ x(r), x(r) = ((r & 3) << 2) | (((r >> 3) & 1) << 1): every row starts at the same bank, a transposing
    // fragment read touches rows 8g + 0..3 (g = 0..3), 32 bytes each, and the XOR spreads those 16 pieces over all 64
    // banks.  Load instruction (j, wave) fills rows 2*(j*NWAVES + wave) and the one after.
    uint32_t a_off[LPT], b_off[LPT];
#pragma unroll
    for (int j = 0; j < LPT; ++j) {
        const int r = (j * NWAVES + wave) * 2 + (lane >> 5);
        const int c = (lane & 31) ^ (((r & 3) << 2) | (((r >> 3) & 1) << 1));
        const int64_t kcol = m0 + c * 8, ncol = n0 + c * 8;
        a_off[j] = kcol < p.K ? (uint32_t)(((int64_t)r * p.ldx + kcol) * 2) : OUT_OF_RANGE;
        b_off[j] = ncol < p.N ? (uint32_t)(((int64_t)r * p.ldy + ncol) * 2) : OUT_OF_RANGE;
    }
    const uint64_t a_base = (uint64_t)(p.X + start * p.ldx), b_base = (uint64_t)(p.DY + start * p.ldy);
    const uint32_t a_row_bytes = (uint32_t)p.ldx * 2, b_row_bytes = (uint32_t)p.ldy * 2;
    const uint32_t smem_u = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)LDS_PTR(smem) + wave * 1024);

    // One load instruction of contraction step kt: idx < LPT the wave's idx-th DY instruction, otherwise its
    // (idx - LPT)-th X instruction.  The descriptor starts at the step's first row and ends with the group, so steps
    // at or past the end (the pipeline runs two ahead) fetch nothing and fill their stage with zeros.
    auto issue_one = [&](int kt, int idx) {
        const bool is_b = idx < LPT;
        const int j = is_b ? idx : idx - LPT;
        const int left = nrows - kt * BR;
        const uint32_t row_bytes = is_b ? b_row_bytes : a_row_bytes;
        const uint64_t base = (is_b ? b_base : a_base) + (uint64_t)(kt * BR) * row_bytes;   // 64-bit: a group may span more than 4 GiB
        i32x4_t rsrc;
        rsrc.x = __builtin_amdgcn_readfirstlane((int)(uint32_t)base);
        rsrc.y = __builtin_amdgcn_readfirstlane((int)(uint32_t)(base >> 32));
        rsrc.z = __builtin_amdgcn_readfirstlane((int)(left > 0 ? (uint32_t)(left < BR ? left : BR) * row_bytes : 0u));   // a step reads BR rows at most
        rsrc.w = 0x00020000;
        load_to_lds_16(rsrc, is_b ? b_off[j] : a_off[j], smem_u + (kt & 1) * STAGE_BYTES + (is_b ? OP_BYTES : 0) + j * (NWAVES * 1024));
    };

    // ---- per-lane LDS fragment offsets: lane 16g + i reads 4 columns at row 8g + (i>>2) (+4 for the second half) of a
    // 32-row step; the transposing read hands lane 16g + i the 8 contraction rows 8g.. of column i -- the 16x16x32 operand.
    int a_frag_off[MB], b_frag_off[NB];
    {
        const int g = lane >> 4, i = lane & 15;
        const int r = 8 * g + (i >> 2);
        const int x = ((r & 3) << 2) | (((r >> 3) & 1) << 1);
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            const int col = wm * WTM + mb * 16 + 4 * (i & 3);
            a_frag_off[mb] = (r * (BM / 8) + ((col >> 3) ^ x)) * 16 + ((col >> 2) & 1) * 8;
        }
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            const int col = wn * WTN + nb * 16 + 4 * (i & 3);
            b_frag_off[nb] = (r * (BN / 8) + ((col >> 3) ^ x)) * 16 + ((col >> 2) & 1) * 8;
        }
    }
    auto read_frag = [&](const uint8_t* img, int off, int ks) {
        const uint8_t* bp = img + off + ks * 32 * (BM / 8) * 16;
        union { struct { s16x4_t a, b; } s; bf16x8_t v; } u;
        u.s.a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)LDS_PTR(bp));
        u.s.b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)LDS_PTR(bp + 4 * (BM / 8) * 16));
        return u.v;
    };

    f32x4_t acc[MB][NB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[mb][nb][r] = 0.f;

    // ---- main loop: two LDS stages; a contraction step of 64 rows is worked through in four half steps (32-row
    // sub-step 0 or 1) x (row-block half 0 or 1) of MBH*NB MFMAs; DY fragments are double-buffered per sub-step, X
    // fragments per half step, both fetched one half step ahead and across the step boundary; one barrier per step;
    // the fragment reads and the loads that refill a freed stage are issued one at a time between the MFMAs.
    constexpr int NLOADS = 2 * LPT, MFMAS_PER_STEP = MBH * NB, LOAD_GAP = 4, READ_GAP = 2;
    static_assert((NB + MBH) * READ_GAP <= MFMAS_PER_STEP, "fragment reads are issued inside the half step");
    constexpr int LOADS_STEP0 = (MFMAS_PER_STEP + LOAD_GAP - 1) / LOAD_GAP < NLOADS ? (MFMAS_PER_STEP + LOAD_GAP - 1) / LOAD_GAP : NLOADS;
    static_assert((NLOADS - 1) * LOAD_GAP < 4 * MFMAS_PER_STEP, "all loads of a step must be issued within one step of MFMAs");
    if (ke > 0) {
#pragma unroll
        for (int i = 0; i < NLOADS; ++i) issue_one(0, i);
#pragma unroll
        for (int i = 0; i < LOADS_STEP0; ++i) issue_one(1, i);
        __builtin_amdgcn_s_waitcnt(0x0F70 | (LOADS_STEP0 & 15) | ((LOADS_STEP0 >> 4) << 14));   // step 0 has landed
        __syncthreads();
        bf16x8_t af[2][MBH], bf[2][NB];
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) bf[0][nb] = read_frag(smem + OP_BYTES, b_frag_off[nb], 0);
#pragma unroll
        for (int mb = 0; mb < MBH; ++mb) af[0][mb] = read_frag(smem, a_frag_off[mb], 0);
        for (int kt = 0; kt < ke; ++kt) {
            const uint8_t* stage = smem + (kt & 1) * STAGE_BYTES;
#pragma unroll
            for (int hs = 0; hs < 4; ++hs) {
                const int cur_a = hs & 1, cur_b = hs >> 1, mh = hs & 1;
                const int nhs = (hs + 1) & 3;
                if (hs == 3) {
                    __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): step kt+1 has landed
                    __syncthreads();                      // for every wave; and every wave is done reading this stage
                }
                const uint8_t* rstage = (hs == 3) ? smem + ((kt + 1) & 1) * STAGE_BYTES : stage;
                __builtin_amdgcn_sched_barrier(0);
                const int seq = (hs + 1) & 3;
                const int load_kt = (hs == 3) ? kt + 2 : kt + 1;
                // priority falls with progress through the step, so that the two waves of a SIMD leapfrog (see grouped_gemm.hip)
                if (hs == 3) __builtin_amdgcn_s_setprio(3);
                else if (hs == 0) __builtin_amdgcn_s_setprio(2);
                else if (hs == 1) __builtin_amdgcn_s_setprio(1);
                else __builtin_amdgcn_s_setprio(0);
#pragma unroll
                for (int m = 0; m < MFMAS_PER_STEP; ++m) {
                    const int mb = m / NB, nb = (mb & 1) ? NB - 1 - m % NB : m % NB;   // one operand fragment changes per MFMA, never both (see grouped_gemm.hip)
                    const int g = seq * MFMAS_PER_STEP + m;
                    if (m % READ_GAP == 0) {   // one fragment of the next half step; DY blocks first when it starts a sub-step
                        const int nbr = ((nhs & 1) == 0) ? NB : 0;
                        const int q = m / READ_GAP;
                        if (q < nbr) { bf[cur_b ^ 1][q] = read_frag(rstage + OP_BYTES, b_frag_off[q], nhs >> 1); __builtin_amdgcn_sched_barrier(0); }
                        else if (q - nbr < MBH) { af[cur_a ^ 1][q - nbr] = read_frag(rstage, a_frag_off[(nhs & 1) * MBH + q - nbr], nhs >> 1); __builtin_amdgcn_sched_barrier(0); }
                    }
                    if (g % LOAD_GAP == 0 && g / LOAD_GAP < NLOADS) {
                        issue_one(load_kt, g / LOAD_GAP);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                    acc[mh * MBH + mb][nb] = Num::mfma(bf[cur_b][nb], af[cur_a][mb], acc[mh * MBH + mb][nb]);
                }
                __builtin_amdgcn_s_setprio(0);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        __builtin_amdgcn_s_waitcnt(0x0F70);   // loads past the last step must not land in the staging below
        __syncthreads();
    }

    // ---- epilogue.  acc[mb][nb][r] is element (k = mb*16 + lane%16, n = nb*16 + (lane/16)*4 + r) of the wave's
    // sub-tile.  Each wave stages its sub-tile as bf16 in its own slice of the operand buffers (chunks XORed with half
    // the row number -- two 128-byte rows span the 64 banks) and writes whole 128-byte row segments with 16-byte
    // buffer stores; lanes outside the matrix get an offset the hardware drops.
    uint8_t* stg = smem + wave * (WTM * WTN * 2);
    const int mrow = lane & 15, nq = (lane >> 4) * 4;
    constexpr int CPR = WTN / 8;   // 16-byte chunks per staged row
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            const int m = mb * 16 + mrow, ncol = nb * 16 + nq;
            uint2 v;
            v.x = Num::pack2(acc[mb][nb][0], acc[mb][nb][1]);
            v.y = Num::pack2(acc[mb][nb][2], acc[mb][nb][3]);
            *(uint2*)(stg + m * (WTN * 2) + ((((ncol >> 3) ^ (m >> 1)) & (CPR - 1)) << 4) + ((ncol >> 2) & 1) * 8) = v;
        }
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): this wave's staging writes have landed
    const __amdgpu_buffer_rsrc_t obuf = __builtin_amdgcn_make_buffer_rsrc(p.DW + (int64_t)expert * p.swe, 0, (int)0x80000000u, 0x00020000);
    const int slot = lane % CPR;
    const uint32_t ldw2 = (uint32_t)p.ldw * 2;
#pragma unroll 8
    for (int it = 0; it < WTM / (64 / CPR); ++it) {
        const int m = it * (64 / CPR) + lane / CPR;
        const u32x4_t v = *(const u32x4_t*)(stg + m * (WTN * 2) + slot * 16);
        const int64_t k = m0 + wm * WTM + m;
        const int64_t n = n0 + wn * WTN + ((slot ^ (m >> 1)) & (CPR - 1)) * 8;
        const uint32_t off = (k < p.K && n < p.N) ? (uint32_t)k * ldw2 + (uint32_t)n * 2 : 0xFFFFFFF0u;
        __builtin_amdgcn_raw_buffer_store_b128(v, obuf, off, 0, 0);
    }
}

}  // namespace

bool moe_xty_mfma_supported(const MoeXtyParams& p, int64_t R)
{
    auto al16 = [](const void* q) { return q != nullptr && ((uintptr_t)q % 16) == 0; };
    if (p.K <= 0 || p.N <= 0 || p.K % 8 != 0 || p.N % 8 != 0 || p.ldx % 8 != 0 || p.ldy % 8 != 0 || p.ldw % 8 != 0 || p.swe % 8 != 0) return false;
    if (!al16(p.X) || !al16(p.DY) || !al16(p.DW)) return false;
    // operand tiles are addressed with 32-bit byte offsets from the first row of one contraction step (descriptors are
    // re-based per step), output tiles inside one expert's matrix: no limit on the number of rows
    (void)R;
    const int64_t limit = (int64_t)1 << 31;
    if ((BR * p.ldx + p.K) * 2 >= limit || (BR * p.ldy + p.N) * 2 >= limit) return false;
    if ((p.K * p.ldw + p.N) * 2 >= limit) return false;
    return true;
}

int moe_launch_xty_mfma(const MoeXtyParams& p, int64_t R, hipStream_t stream)
{
    if (p.E < 1) return MOE_ERR_BAD_ARG;
    if (!moe_xty_mfma_supported(p, R)) return MOE_ERR_UNSUPPORTED;
    static std::atomic<bool> attr_set[MOE_MAX_DEVICES];   // per device; forward and backward may call from different host threads
    const int dev = moe_current_device();
    if (!attr_set[dev]) {
        if (hipFuncSetAttribute((const void*)grouped_xty_mfma_kernel<NumBf16>, hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES) != hipSuccess ||
            hipFuncSetAttribute((const void*)grouped_xty_mfma_kernel<NumF16>, hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES) != hipSuccess)
            return MOE_ERR_LAUNCH;
        attr_set[dev] = true;
    }
    const int64_t per_e = ((p.K + BM - 1) / BM) * ((p.N + BN - 1) / BN);
    const int64_t grid = (per_e + NXCD - 1) / NXCD * p.E * NXCD;   // an eighth of every expert's tiles per XCD
    if (grid > 0x7fffffff) return MOE_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(p.f16 ? grouped_xty_mfma_kernel<NumF16> : grouped_xty_mfma_kernel<NumBf16>, dim3((unsigned)grid), dim3(NTHREADS), LDS_BYTES, stream, p);
    return moe_launch_status();
}
