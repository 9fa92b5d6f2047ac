// Ragged per-expert grouped GEMM on the gfx950 matrix cores (bf16 in, fp32 accumulate, bf16 out).
//
//   Y[out_row(m)][n] = sum_seg sum_k X_seg[in_row(m)][k] * W_seg[e(m)][k][n]  +  sum_slab Q_slab[m][0:16] . LB_slab[e(m)][n][0:16]
//
// m runs over expert-sorted positions; row tiles of BM positions never straddle two experts (derived from the
// inclusive expert offsets), rows past the end of a group are computed on clamped addresses and never stored,
// so no token is dropped and no padding is materialised.  The low-rank (LoRA) branch enters as one extra
// 16-wide K slab per adapter: Q = bf16(scaling * X A) is produced once per row by the skinny kernel in
// lora_kernels.hip, LB is the adapter's B factor packed as [expert][n][16].
//
// Tiling: 256x256x64 macro tile, 8 waves (2 along M x 4 along N), each wave 128x64 = 8x4 MFMA 16x16x32 tiles (this
// shape sustains a higher rate than 32x32x16 on the same operand traffic).
// Operand tiles are brought HBM -> LDS with direct-to-LDS 16-byte loads (no VGPR staging): two stages of activation
// tiles and three of weight tiles, 160 KiB, all of a compute unit's LDS.
// LDS images are XOR-swizzled at 16-byte granularity by choosing which global chunk each lane fetches, so the
// ds_read_b128 (K-contiguous operands) and ds_read_b64_tr_b16 (N-contiguous weights) fragment reads spread over
// the banks.  Gathered A rows are resolved once per tile into LDS row tables.
#include "common.h"
#include "kernels.h"
#include <type_traits>

#define EPI_IS_PAIR(e) ((e) == MOE_EPI_SWIGLU || (e) == MOE_EPI_SWIGLU_FUSED)
constexpr int NXCD_HOST = 8;
// compute units of the current device that the tile plan fills: a multiple of 8 (whole rounds are dealt out to the 8 XCDs)
static int moe_num_cus()
{
    const int n = moe_device_cus() / NXCD_HOST * NXCD_HOST;
    return n < NXCD_HOST ? NXCD_HOST : n;
}

namespace {

constexpr int BM = 256, BN = 256, BK = 64;
constexpr int NWAVES = 8;                 // 2 x 4 waves of 128x64
constexpr int NTHREADS = NWAVES * 64;
constexpr int WAVES_M = 2, WAVES_N = NWAVES / 2;
constexpr int WTM = BM / WAVES_M;  // 128
constexpr int WTN = BN / WAVES_N;  // 64
constexpr int MB = WTM / 16;       // 8 row blocks of 16
constexpr int NB = WTN / 16;       // 4 column blocks of 16
constexpr int NBH = NB / 2;        // column blocks per projection in the gate/up pair kernel
constexpr int MBH = MB / 2;        // row blocks per half: a wave works through its tile one half (MBH x NB blocks, 32 k) at a time
constexpr int LPT = 32 / NWAVES;   // direct-to-LDS load instructions per wave, operand and K tile
constexpr int A_STAGE_BYTES = BM * BK * 2;  // 32 KiB
constexpr int B_STAGE_BYTES = BN * BK * 2;  // 32 KiB
constexpr int NSTAGE_A = 2, NSTAGE_B = 3;   // the weight tile ring is one stage deeper: its loads miss the caches more often
constexpr int B_REGION = NSTAGE_A * A_STAGE_BYTES;                                // weight stages follow the activation stages
constexpr int LDS_BYTES = NSTAGE_A * A_STAGE_BYTES + NSTAGE_B * B_STAGE_BYTES;    // 160 KiB: all of a compute unit's LDS
// Row tables (in_row, out_row as int64) and the split tiles' arrival flag borrow the third weight stage: before the
// main loop's first tile that stage is still empty, and after the loop the epilogue staging only needs the first 128 KiB.
constexpr int TABLE_OFF = B_REGION + 2 * B_STAGE_BYTES;
static_assert(TABLE_OFF >= NWAVES * (BM / 2) * (BN / (NWAVES / 2)) * 2, "epilogue staging must not reach the tables");
// SwiGLU-backward epilogue with fused row contractions: images of three [BM][16] bf16 operands sit behind the row tables
constexpr int RC_MATS = 3;
constexpr int RC_IMG_OFF = TABLE_OFF + 2 * BM * 8 + 64;
constexpr int RC_IMG_BYTES = BM * 16 * 2;                       // 8 KiB per operand
static_assert(RC_IMG_OFF + RC_MATS * RC_IMG_BYTES <= LDS_BYTES, "row-contraction images fit behind the tables");
constexpr int NXCD = 8;
constexpr int INTERLEAVE_MIN_ROUNDS = 8;    // launches with at least this many rounds of tiles deal them to the XCDs in chunks
constexpr int CONTIGUOUS_MIN_ROUNDS = 4;    // ... and so do launches of fewer rounds than this; those in between give every XCD one contiguous range

// 16 bytes per lane, global -> LDS without passing through VGPRs: lane l's data lands at lds_addr + 16*l.  The source
// is a raw buffer (base address in a scalar resource descriptor) plus a 32-bit per-lane byte offset plus a scalar byte
// offset, so advancing along K costs no vector instructions.  Issued through inline assembly so that the compiler's
// wait-count insertion does not serialise the prefetch against the fragment reads of the other stage; completion is
// awaited with explicit s_waitcnt vmcnt(n) below.
typedef int i32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ i32x4_t make_buffer(const void* base, uint32_t num_records = 0xFFFFFFFFu)
{
    const uint64_t a = (uint64_t)base;
    i32x4_t r;
    r.x = __builtin_amdgcn_readfirstlane((int)(uint32_t)a);
    r.y = __builtin_amdgcn_readfirstlane((int)(uint32_t)(a >> 32));   // stride field (bits 16..29 of this word) = 0: raw buffer
    r.z = (int)num_records;                                           // a per-lane offset at or above this is out of range (loads return zeros); real offsets are checked on the host
    r.w = 0x00020000;                                                 // 32-bit data format
    return r;
}
__device__ __forceinline__ void load_to_lds_16(i32x4_t rsrc, uint32_t lane_off, uint32_t uniform_off, uint32_t lds_addr)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds" ::"s"(__builtin_amdgcn_readfirstlane(lds_addr)), "v"(lane_off), "s"(rsrc), "s"(__builtin_amdgcn_readfirstlane(uniform_off)) : "memory", "m0");
}

// logistic function through the hardware exponential and reciprocal (about 1 ulp each; the results are rounded to bf16)
__device__ __forceinline__ float sigmoid_f(float g) { return __builtin_amdgcn_rcpf(1.f + __expf(-g)); }

// ---- work item of a workgroup -> (expert, n tile, m tile, K part).  One workgroup per work item; the hardware dispatcher
// hands the next item to whichever compute unit of the XCD frees up first (blockIdx round-robins over the 8 XCDs), which
// balances ragged (cheaper) row tiles inside an XCD by itself; between XCDs work cannot migrate.
struct WorkItem {
    bool valid;
    int expert, nt;            // expert, n tile
    int64_t row0, row1;        // rows of the m tile
    int part, nparts;          // K part of a split tile (0 of 1: whole tile)
    int split_item;            // exchange slot of this part (the slots of a tile are consecutive, in part order)
    int split_tile;            // counter of the split tile
    int mtile;                 // number of the row tile among all row tiles (experts in order, BM rows each)
    int mt_in_group;           // number of the row tile within its expert's group (0: the group's first tile)
};

__device__ __forceinline__ WorkItem decode_work_item(const void* offsets, int off64, int E, int ntiles_n, int ktiles,
                                                     int max_split, int ncu)
{
    WorkItem w = {};
    const int lane = threadIdx.x & 63;
    ExpertScan sc = {};
    int64_t T = 0;
    if (E <= 64) {
        // every wave sees all expert groups at once: one memory round trip for the whole lookup
        sc = scan_expert_tiles(offsets, off64, E, BM);
        T = uniform_i64(__shfl(sc.tiles_through, 63)) * ntiles_n;
    } else {
        int64_t start = 0;
        for (int e = 0; e < E; ++e) { const int64_t end = load_idx(offsets, e, off64); T += (end - start + BM - 1) / BM; start = end; }
        T *= ntiles_n;
    }
    const int xcd = blockIdx.x % NXCD;
    const int64_t q = blockIdx.x / NXCD;
    const int CH = ncu / NXCD;             // compute units per XCD
    int64_t t = -1;                        // output tile in the list (expert, n tile, m tile fastest)
    {
        // The T tiles are cut into F = (T / #CU) * #CU tiles that fill whole rounds of compute units and a remainder; the
        // remainder tiles' K ranges are split 2 or 4 ways (when that many parts still fit in one round), so that the
        // last round is a half or a quarter as long instead of leaving most compute units idle.  Whole-round tiles, few
        // rounds: each XCD takes one contiguous range of the tile list (for evenly sized groups that is one expert per
        // XCD, whose row tiles it re-reads from nearby caches).  Many rounds: consecutive chunks of one XCD's worth of
        // tiles go to consecutive XCDs instead -- a chunk still runs side by side on its XCD (its tiles share weight and
        // row tiles in that L2), but every XCD sees every part of the list, which evens out the cheaper tiles of ragged
        // groups (measured: the gate/up launch, 16 rounds, 3 % faster dealt out in chunks, the 9-round launches of a
        // skewed 16384-token batch 8 %).  Launches of two or three rounds are dealt out the same way: over eight routing
        // draws of 8192 rows their two N-contiguous launches run 1-2 % faster than with contiguous ranges (0.4 % of the
        // layer's GEMM time on average, 1 % on the default draw, and no slower with evenly sized groups), while the
        // 7-round launch with the SwiGLU-backward epilogue measured 1.5 % slower dealt out and keeps its ranges.  Measured and
        // dropped for launches of few rounds: XCD ranges cut by the running cost of the tiles (32-row blocks, at
        // least half a tile) instead of by their number -- 4-7 % slower, with either way of splitting the last tiles.
        const int64_t F = (T / ncu) * ncu;
        const int rem = (int)(T - F);
        int split = 1;
        while (split * 2 <= max_split && rem * split * 2 <= ncu && ktiles / (split * 2) >= 8) split *= 2;
        const int S = rem * split;                       // items of the last round
        const int64_t Fx = F / NXCD;
        const int Sx = (S + NXCD - 1) / NXCD;
        if (q < Fx) {
            const bool deal = F >= (int64_t)INTERLEAVE_MIN_ROUNDS * ncu || F < (int64_t)CONTIGUOUS_MIN_ROUNDS * ncu;
            t = deal ? ((q / CH) * NXCD + xcd) * CH + q % CH : xcd * Fx + q;
        } else {
            const int64_t j = (int64_t)xcd * Sx + (q - Fx);
            if (q - Fx >= Sx || j >= S) return w;
            t = F + j / split;
            w.part = (int)(j % split);
            w.nparts = split;
            w.split_item = (int)j;
            w.split_tile = (int)(j / split);
        }
    }
    if (w.nparts == 0) w.nparts = 1;
    if (E <= 64) {
        const unsigned long long hit = __ballot(lane < E && t >= sc.tiles_before * ntiles_n && t < sc.tiles_through * ntiles_n);
        if (hit == 0) return w;
        int expert = __ffsll(hit) - 1;
        const int64_t start = __shfl(sc.start, expert), end = __shfl(sc.end, expert), before = __shfl(sc.tiles_before, expert);
        const int64_t mte = (end - start + BM - 1) / BM;
        const int64_t local = t - before * ntiles_n;
        const int nt = (int)(local / mte);
        const int64_t mt = local % mte;
        const int64_t row0 = start + mt * BM;
        const int64_t row1 = (row0 + BM < end) ? row0 + BM : end;
        // the shuffles return per-lane values; everything derived from the item is uniform and belongs in scalar registers
        w.expert = __builtin_amdgcn_readfirstlane(expert);
        w.nt = __builtin_amdgcn_readfirstlane(nt);
        w.row0 = uniform_i64(row0);
        w.row1 = uniform_i64(row1);
        w.mtile = __builtin_amdgcn_readfirstlane((int)(before + mt));
        w.mt_in_group = __builtin_amdgcn_readfirstlane((int)mt);
        w.valid = true;
    } else {
        int64_t start = 0, id = t, mtiles_before = 0;
        for (int e = 0; e < E; ++e) {
            const int64_t end = load_idx(offsets, e, off64);
            const int64_t mte = (end - start + BM - 1) / BM;
            const int64_t te = mte * ntiles_n;
            if (id < te) {
                w.expert = e;
                w.nt = (int)(id / mte);
                const int64_t mt = id % mte;
                w.mtile = (int)(mtiles_before + mt);
                w.mt_in_group = (int)mt;
                w.row0 = start + mt * BM;
                w.row1 = (w.row0 + BM < end) ? w.row0 + BM : end;
                w.valid = true;
                break;
            }
            id -= te;
            mtiles_before += mte;
            start = end;
        }
    }
    w.part = __builtin_amdgcn_readfirstlane(w.part);
    w.nparts = __builtin_amdgcn_readfirstlane(w.nparts);
    w.split_item = __builtin_amdgcn_readfirstlane(w.split_item);
    w.split_tile = __builtin_amdgcn_readfirstlane(w.split_tile);
    return w;
}

// Test aid: the work item of every workgroup of a launch with this geometry, 8 ints per workgroup
// (valid, expert, n tile, first row, one-past-last row, part, parts, exchange slot), the split tile's counter in the 9th.
__global__ void gemm_plan_kernel(const void* offsets, int off64, int E, int ntiles_n, int ktiles, int max_split, int ncu, int* out)
{
    const WorkItem w = decode_work_item(offsets, off64, E, ntiles_n, ktiles, max_split, ncu);
    if (threadIdx.x == 0) {
        int* o = out + (int64_t)blockIdx.x * 9;
        o[0] = w.valid; o[1] = w.expert; o[2] = w.nt; o[3] = (int)w.row0; o[4] = (int)w.row1;
        o[5] = w.part; o[6] = w.nparts; o[7] = w.split_item; o[8] = w.split_tile;
    }
}

// KTAIL, the general variant (plain epilogue only): K need not be a multiple of the 64-wide K tile (but of 8) -- the last
// tile of every K segment is then partial, and the loads that would reach past K fetch zeros instead -- and the adapter may
// have more than MOE_MAX_SLABS slabs.  A variant of its own so that the kernels of the usual shapes carry none of it.
template <bool NN, int EPI, typename Num, bool KTAIL>
__global__ void __launch_bounds__(NTHREADS) grouped_gemm_mfma_kernel(const MoeGemmParams p)
{
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
    int64_t* s_inrow = (int64_t*)(smem + TABLE_OFF);
    int64_t* s_outrow = s_inrow + BM;
    int* s_arrival = (int*)(s_outrow + BM);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;

    // ---- work item -> (expert, n tile, m tile, K part)
    const int ntiles_n = (EPI_IS_PAIR(EPI)) ? (int)((p.N + BN / 2 - 1) / (BN / 2)) : (int)((p.N + BN - 1) / BN);
    const int ktiles_seg = KTAIL ? (int)((p.K + BK - 1) / BK) : (int)(p.K / BK);
    const int ktiles = ktiles_seg * p.nseg;
    const WorkItem item = decode_work_item(p.offsets, p.off64, p.E, ntiles_n, ktiles, p.max_split, p.num_cus);
    if (!item.valid) return;
    const int expert = item.expert, nt = item.nt, part = item.part, nparts = item.nparts, split_item = item.split_item;
    const int64_t row0 = item.row0, row1 = item.row1;
    const int nrows = (int)(row1 - row0);
    const int64_t n0 = (int64_t)nt * ((EPI_IS_PAIR(EPI)) ? BN / 2 : BN);

    // ---- row tables
    for (int r = tid; r < BM; r += NTHREADS) {
        const int64_t m = row0 + ((r < nrows) ? r : nrows - 1);  // clamp: rows past the group re-read its last row
        int64_t in_row = m, out_row = m;
        if (!p.x_grouped || !p.y_grouped) {
            const int64_t pp = load_idx(p.pos, m, p.pos64);
            if (!p.x_grouped) in_row = pp / p.fan_out;
            if (!p.y_grouped) out_row = pp;
        }
        s_inrow[r] = in_row;
        s_outrow[r] = out_row;
    }
    __syncthreads();

    // ---- per-thread global source pointers for the direct-to-LDS loads (k offset added per tile)
    // A image: row r at r*128 B, logical 16-byte chunk c of that row at slot c ^ ((r >> 1) & 7): two rows span the
    // 64 LDS banks, so 16 consecutive rows of one chunk column hit 16 different bank groups.
    // Wave w issues load instructions j = 0..3; instruction (j, w) fills rows [(j*8 + w)*8, +8).
    // Grouped rows are addressed from the tile's first row (the descriptor is re-based there, so the 32-bit offsets
    // only span one tile whatever the number of rows); gathered rows from the start of X.
    const int64_t a_row_base = p.x_grouped ? row0 : 0;
    uint32_t a_off[LPT];   // byte offsets into X[0] / X[1] (the same for both K segments)
#pragma unroll
    for (int j = 0; j < LPT; ++j) {
        const int r = (j * NWAVES + wave) * 8 + (lane >> 3);
        const int c = (lane & 7) ^ ((r >> 1) & 7);
        a_off[j] = (uint32_t)(((s_inrow[r] - a_row_base) * p.ldx + c * 8) * 2);
    }
    // (KTAIL: the masked loads of a partial K tile use the offset OUT_OF_RANGE, which must lie at or above the descriptors'
    // range -- with the full 32-bit range it would be a valid offset and the load would touch memory 4 GiB past the base)
    constexpr uint32_t LOAD_RANGE = KTAIL ? 0x80000000u : 0xFFFFFFFFu;
    const i32x4_t a_buf0 = make_buffer(p.X[0] + a_row_base * p.ldx, LOAD_RANGE), a_buf1 = make_buffer((p.X[1] ? p.X[1] : p.X[0]) + a_row_base * p.ldx, LOAD_RANGE);
    // B: offsets within this expert's matrix.  For the SwiGLU pair image rows [0,128) come from W[0] and [128,256)
    // from W[1], which are whole load instructions (the first and second half of a wave's LPT); otherwise W[0] / W[1]
    // are the two K segments.
    uint32_t b_off[LPT];
    const i32x4_t b_buf0 = make_buffer(p.W[0] + (int64_t)expert * p.swe, LOAD_RANGE), b_buf1 = make_buffer((p.W[1] ? p.W[1] : p.W[0]) + (int64_t)expert * p.swe, LOAD_RANGE);
    if (!NN) {
        // B image as A: row = n (BN rows of 64 k)
#pragma unroll
        for (int j = 0; j < LPT; ++j) {
            const int r = (j * NWAVES + wave) * 8 + (lane >> 3);
            const int c = (lane & 7) ^ ((r >> 1) & 7);
            int64_t n = (EPI_IS_PAIR(EPI)) ? n0 + (r & (BN / 2 - 1)) : n0 + r;
            if (n >= p.N) n = p.N - 1;
            b_off[j] = (uint32_t)((n * p.ldw + c * 8) * 2);
        }
    } else {
        // B image: [64 k][BN n], 32 chunks per k row; chunk (k, c) at slot c ^ x(k), x(k) = ((k&3) << 2) | (((k>>3)&1) << 1):
        // all k rows start at the same bank, and a transposing fragment read touches rows 8g + 0..3 (g = 0..3), 32
        // bytes each -- the XOR spreads those 16 pieces over all 64 banks, each bank used twice by the 512-byte read.
        // Instruction (j, w) fills LDS chunks [(j*NWAVES + w)*64, +64) = k rows 2*(j*NWAVES+w), +1.
#pragma unroll
        for (int j = 0; j < LPT; ++j) {
            const int k = (j * NWAVES + wave) * 2 + (lane >> 5);
            const int c = (lane & 31) ^ (((k & 3) << 2) | (((k >> 3) & 1) << 1));
            int64_t n = n0 + c * 8;
            if (n >= p.N) n = 0;
            b_off[j] = (uint32_t)(((int64_t)k * p.ldw + n) * 2);
        }
    }

    // ---- low-rank slabs (up to two) ride in as the activation image of the K tile after the last: that tile's four
    // load instructions per wave fetch, instead of a re-read nobody uses, 32 rows x 16 k of Q[0], of Q[1], and 32
    // columns x 16 k of LB[0], of LB[1] (8 KiB each over the 8 waves; for the gate/up pair the two halves of a column
    // image hold the same 128 columns; with one slab both images of a kind hold that slab).  The slab step after the
    // loop then reads its fragments from LDS instead of waiting for a round trip to memory.
    static_assert(LPT == 4, "slab image: one load instruction per wave for each of Q[0], Q[1], LB[0], LB[1]");
    const bool lds_slabs = p.nslab >= 1 && p.nslab <= 2;
    uint32_t slab_off_q = 0, slab_off_l = 0;
    const bool two_slabs = p.nslab > 1;   // (static indices below: a dynamic one would move the parameter block to scratch memory)
    const uint16_t* const q1 = two_slabs ? p.Q[1] : p.Q[0];
    const uint16_t* const l1 = two_slabs ? p.LB[1] : p.LB[0];
    const i32x4_t q_buf0 = make_buffer(lds_slabs ? p.Q[0] : p.X[0]), q_buf1 = make_buffer(lds_slabs ? q1 : p.X[0]);
    const i32x4_t l_buf0 = make_buffer(lds_slabs ? p.LB[0] + (int64_t)expert * p.N * 16 : p.X[0]);
    const i32x4_t l_buf1 = make_buffer(lds_slabs ? l1 + (int64_t)expert * p.N * 16 : p.X[0]);
    {
        if (lds_slabs) {
            const int i = wave * 32 + (lane >> 1);
            const int r = i < nrows ? i : nrows - 1;
            slab_off_q = (uint32_t)((r * 16 + (lane & 1) * 8) * 2);             // + row0 * 32 as the scalar offset
            int64_t n = (EPI_IS_PAIR(EPI)) ? n0 + (i & (BN / 2 - 1)) : n0 + i;
            if (n >= p.N) n = p.N - 1;
            slab_off_l = (uint32_t)(((n - n0) * 16 + (lane & 1) * 8) * 2);      // + n0 * 32
        }
    }

    // ---- per-lane LDS fragment offsets.  A 16x16x32 operand fragment: lane l holds row (l & 15), k = 8*(l >> 4) .. +7 of
    // a 32-wide K step, i.e. 16-byte chunk (l >> 4) of that step.
    int a_frag_off[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks)
        a_frag_off[ks] = (wm * WTM + (lane & 15)) * 128 + (((ks * 4 + (lane >> 4)) ^ ((lane >> 1) & 7)) << 4);
    int b_frag_off[NN ? NB : 2];
    if (!NN) {
#pragma unroll
        for (int ks = 0; ks < 2; ++ks)
            b_frag_off[ks] = (lane & 15) * 128 + (((ks * 4 + (lane >> 4)) ^ ((lane >> 1) & 7)) << 4);
    } else {
        // transposing reads: lane 16g + i fetches 4 columns at k row 8g + (i >> 2) (a second read 4 rows further down);
        // the hardware hands lane 16g + i the 8 k values 8g .. 8g+7 of column i
        const int g = lane >> 4, i = lane & 15;
        const int krow = 8 * g + (i >> 2);  // + ks*32 + 4*t
        const int x = ((krow & 3) << 2) | (((krow >> 3) & 1) << 1);   // the same for the second read and for both K steps
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            const int ncol = wn * WTN + nb * 16 + 4 * (i & 3);
            const int c = ncol >> 3, half = (ncol >> 2) & 1;
            b_frag_off[nb] = (krow * (BN / 8) + (c ^ x)) * 16 + half * 8;
        }
    }

    f32x4_t acc[MB][NB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[mb][nb][r] = 0.f;

    // number of 16-row MFMA blocks of this wave that hold at least one real row
    int mb_cnt = (nrows - wm * WTM + 15) / 16;
    mb_cnt = mb_cnt < 0 ? 0 : (mb_cnt > MB ? MB : mb_cnt);
    // the same in every lane: as a scalar it selects the wave's copy of the K loop with one branch, and the checks in
    // the slab step are scalar branches (under a vector condition the compiler masks single MFMAs instead of branching
    // around them, and the matrix cores ignore the mask)
    mb_cnt = __builtin_amdgcn_readfirstlane(mb_cnt);

    const int kb = ktiles * part / nparts;
    const int ke = ktiles * (part + 1) / nparts;

    const uint32_t smem_u = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)LDS_PTR(smem) + wave * 1024);   // this wave's 1 KiB slot in the NWAVES KiB that one round of load instructions fills
    // One direct-to-LDS load instruction of a K tile's activation (issue_a) or weight (issue_b) image, into the given
    // stage.  K tiles past the end re-read the last one (into the stage such a tile would use, which nobody reads any
    // more), which keeps the main loop free of branches around the loads.  Activation instructions whose 8 rows lie
    // past the tile's last 32-row block are dropped when `ragged` is set (what MFMAs compute from such rows is never
    // stored or summed); the wait counts of the main loop only ever leave weight instructions in flight, which are never dropped,
    // so they do not depend on how many activation instructions were.
    const int live_rows = (nrows + 31) / 32 * 32;
    // Partial last K tile (KTAIL): a load whose 8 k (K-contiguous images) or whose k row (N-contiguous image) lies at or past
    // K gets a per-lane offset beyond the descriptor's range (LOAD_RANGE, 2 GiB in this variant) -- the hardware then writes
    // zeros to LDS and touches no memory.
    // The range check looks at the per-lane offset, so the K advance moves from the scalar offset into it for that tile.
    // The 16-byte chunk a lane fetches of a K-contiguous row is (lane & 7) ^ ((row >> 1) & 7), the same in all of a wave's
    // load instructions (their rows differ by multiples of 64).
    constexpr uint32_t OUT_OF_RANGE = 0xFFFFFFF0u;
    const uint32_t ktail_kq = (uint32_t)(((lane & 7) ^ (((lane >> 4) + 4 * (wave & 1)) & 7)) * 8);
    auto issue_a = [&](int kt, int jj, int stage, bool ragged) {
        kt = __builtin_amdgcn_readfirstlane(kt < ke ? kt : ke - 1);
        const int seg = (kt >= ktiles_seg) ? 1 : 0;
        const uint32_t k0 = (uint32_t)(kt - seg * ktiles_seg) * BK;
        if constexpr (KTAIL) {
            uint32_t voff = a_off[jj], soff = k0 * 2;
            if (k0 + BK > (uint32_t)p.K) { voff = (k0 + ktail_kq < (uint32_t)p.K) ? voff + soff : OUT_OF_RANGE; soff = 0; }
            if (!ragged || (jj * NWAVES + wave) * 8 < live_rows)
                load_to_lds_16(seg ? a_buf1 : a_buf0, voff, soff, smem_u + stage * A_STAGE_BYTES + jj * (NWAVES * 1024));
        } else {
        if (!ragged || (jj * NWAVES + wave) * 8 < live_rows)
            load_to_lds_16(seg ? a_buf1 : a_buf0, a_off[jj], k0 * 2, smem_u + stage * A_STAGE_BYTES + jj * (NWAVES * 1024));
        }
    };
    // the same instruction slot for the slab image (the activation image of tile ke)
    auto issue_slab = [&](int jj, int stage) {
        const uint32_t dst = smem_u + stage * A_STAGE_BYTES + jj * (NWAVES * 1024);
        const i32x4_t d = jj == 0 ? q_buf0 : (jj == 1 ? q_buf1 : (jj == 2 ? l_buf0 : l_buf1));
        load_to_lds_16(d, jj < 2 ? slab_off_q : slab_off_l, (uint32_t)(jj < 2 ? row0 : n0) * 32u, dst);
    };
    auto issue_b = [&](int kt, int idx, int stage) {
        kt = __builtin_amdgcn_readfirstlane(kt < ke ? kt : ke - 1);
        const int seg = (kt >= ktiles_seg) ? 1 : 0;
        const uint32_t k0 = (uint32_t)(kt - seg * ktiles_seg) * BK;
        const bool second = (EPI_IS_PAIR(EPI)) ? (idx >= LPT / 2) : (seg != 0);
        if constexpr (KTAIL) {
            uint32_t voff = b_off[idx], soff = NN ? k0 * (uint32_t)p.ldw * 2 : k0 * 2;
            if (k0 + BK > (uint32_t)p.K) {
                // K-contiguous image: this lane's 8 k as for the activation image; N-contiguous image: the lane's whole k row
                const bool in = NN ? k0 + (uint32_t)((idx * NWAVES + wave) * 2 + (lane >> 5)) < (uint32_t)p.K : k0 + ktail_kq < (uint32_t)p.K;
                voff = in ? voff + soff : OUT_OF_RANGE;
                soff = 0;
            }
            load_to_lds_16(second ? b_buf1 : b_buf0, voff, soff, smem_u + B_REGION + stage * B_STAGE_BYTES + idx * (NWAVES * 1024));
        } else {
        load_to_lds_16(second ? b_buf1 : b_buf0, b_off[idx], NN ? k0 * (uint32_t)p.ldw * 2 : k0 * 2, smem_u + B_REGION + stage * B_STAGE_BYTES + idx * (NWAVES * 1024));
        }
    };

    // fragment readers (LDS -> registers), one 16-wide block each.  Accumulator tiles are kept transposed -- the weight fragment is the
    // MFMA's first operand -- so that a lane ends up with 4 consecutive output columns of one row (8-byte packs).
    auto read_b1 = [&](const uint8_t* b_lds, int ks, int nb, bf16x8_t* bfrag) {
        if (!NN) {
            const int brow = (EPI_IS_PAIR(EPI)) ? (nb / NBH) * (BN / 2) + wn * (WTN / 2) + (nb % NBH) * 16 : wn * WTN + nb * 16;
            bfrag[nb] = *(const bf16x8_t*)(b_lds + brow * 128 + b_frag_off[ks]);
        } else {
            const uint8_t* bp = b_lds + b_frag_off[nb] + ks * 32 * (BN / 8) * 16;
            s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)LDS_PTR(bp));
            s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)LDS_PTR(bp + 4 * (BN / 8) * 16));
            union { struct { s16x4_t a, b; } s; bf16x8_t v; } u;
            u.s.a = lo; u.s.b = hi;
            bfrag[nb] = u.v;
        }
    };
    auto read_a1 = [&](const uint8_t* a_lds, int ks, int mh, int mb, bf16x8_t* afrag) {
        afrag[mb] = *(const bf16x8_t*)(a_lds + (mh * MBH + mb) * 16 * 128 + a_frag_off[ks]);
    };
    // Software pipeline.  A K tile is worked through in four half steps (k step 0 or 1) x (row half 0 or 1) of MBH*NB
    // MFMAs each; the weight fragments of a k step and the activation fragments of a half step are double-buffered in
    // registers and fetched one half step ahead, also across the tile boundary: the MFMAs of a tile's last half step
    // run after the barrier that hands over the next tile, so they cover the LDS latency of that tile's first fragment
    // reads.  That barrier also frees the stages the finished tile occupied.  Neither the fragment reads nor the loads
    // that refill the stages are issued in one burst -- a burst keeps the wave's instruction stream and the LDS / load
    // unit's queue busy while the matrix pipe idles -- but one at a time between the MFMAs: a fragment read before every
    // second MFMA of a half step (weight blocks first, when the next half step starts a k step), the loads as below.
    constexpr int MFMAS_PER_STEP = MBH * NB;
    constexpr int READ_GAP = 2;     // MFMAs between two fragment reads
    static_assert((NB + MBH) * READ_GAP <= MFMAS_PER_STEP, "fragment reads are issued inside the half step");
    constexpr int A_LOAD_GAP = 4;   // MFMAs between two activation loads (the half step after the barrier)
    constexpr int B_LOAD_GAP = 8;   // ... between two weight loads (the two half steps after that)
    static_assert(LPT * A_LOAD_GAP <= MFMAS_PER_STEP && LPT * B_LOAD_GAP <= 3 * MFMAS_PER_STEP, "loads are issued inside their half steps");
    // Stages: activation tile kt lives in A stage (kt - kb) % 2, weight tile kt in B stage (kt - kb) % 3.  The barrier
    // that ends tile kt frees both of its stages; the half step after it requests activation tile kt+2 (into the A
    // stage just freed), the two after that weight tile kt+3 (into the B stage just freed).  The next barrier then only
    // has to see the activation loads -- requested first, mostly cache hits -- and the weight tile requested a whole
    // tile earlier: the youngest LPT loads, weight loads that may well be waiting for HBM, stay in flight across it.
    // NBLK: how many of the wave's MB 16-row blocks take part -- MB for every wave of a full tile; in a ragged tile each
    // wave runs the copy of the loop that fits its own rows, the count of its live blocks rounded up to 0, 1, 2, MBH or MB
    // (0: no MFMAs, no fragment reads, the wave only issues its loads and meets the barriers).  A compile-time count, not a
    // check per block: a check is a scalar branch per MFMA, and a tail tile of a few rows spent more time on those branches
    // than on its MFMAs.  Blocks inside the count that lie past the group work on whatever their LDS rows hold (rows past
    // the last 32-row block are never loaded); every consumer of the accumulators masks rows past the group.
    auto mainloop = [&](auto nblk_tag, auto full_tag) {
        constexpr int NBLK = decltype(nblk_tag)::value;
        constexpr bool FULL = decltype(full_tag)::value;
#pragma unroll
        for (int i = 0; i < LPT; ++i) issue_a(kb, i, 0, !FULL);
#pragma unroll
        for (int i = 0; i < LPT; ++i) issue_b(kb, i, 0);
        if (lds_slabs && kb + 1 == ke) {
#pragma unroll
            for (int i = 0; i < LPT; ++i) issue_slab(i, 1);
        } else {
#pragma unroll
            for (int i = 0; i < LPT; ++i) issue_a(kb + 1, i, 1, !FULL);
        }
#pragma unroll
        for (int i = 0; i < LPT; ++i) issue_b(kb + 1, i, 1);
        __builtin_amdgcn_s_waitcnt(0x0F70 | LPT);   // everything but weight tile kb+1 has landed
        __syncthreads();                            // (also: every wave has read the row tables that share B stage 2)
        bf16x8_t af[2][MBH], bf[2][NB];
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) read_b1(smem + B_REGION, 0, nb, bf[0]);
#pragma unroll
        for (int mb = 0; mb < MBH; ++mb) read_a1(smem, 0, 0, mb, af[0]);
        int bs = 0;   // B stage of tile kt
        // A tail tile of at most two row blocks has next to no MFMA work and would run through K several times faster than
        // the full row tiles that share its weight tiles: the weight tiles it fetches are then gone from L2 again before
        // those arrive (measured on the gate/up launch: 0.8 GB more fetched from memory with three such tails), and its
        // requests compete with theirs.  The waves of such a tile therefore take at least PACE_CYCLES per K tile (a full tile
        // cannot take less: 2048 cycles are its MFMAs alone), which keeps it just ahead of them -- close enough to act as their
        // prefetcher.  Measured over eight routing draws of 8192 rows: the launches of few rounds 1-2 % faster; the gate/up
        // launch, whose sixteen rounds are bound by the sum of the tiles' times, 2 % slower than with unpaced tails --
        // the price of not fetching those weight tiles twice.  The copy of the loop is chosen per wave (its live blocks);
        // whether it paces is decided per tile: only a tail that follows full row tiles of its group shares weight tiles
        // with anybody -- a group's first tile (small batches, many experts with a few rows each) runs unpaced.
        constexpr bool PACED = !FULL && NBLK <= 2;
        const bool pace = PACED && item.mt_in_group > 0;
        constexpr int64_t PACE_CYCLES = 2048;
        int64_t pace_t0 = pace ? (int64_t)__builtin_readcyclecounter() : 0;
        // one K tile; SLAB: the activation loads it requests (for tile kt+2) fetch the slab image instead
        auto tile = [&](int kt, auto slab_tag) {
            constexpr bool SLAB = decltype(slab_tag)::value;
            const int as = (kt - kb) & 1;
            const int bs1 = bs == 2 ? 0 : bs + 1;     // B stage of tile kt+1
            const int bs2 = bs1 == 2 ? 0 : bs1 + 1;   // B stage of tile kt+2 (= of tile kt-1, free since the last barrier)
            const uint8_t* a_lds = smem + as * A_STAGE_BYTES;
            const uint8_t* b_lds = smem + B_REGION + bs * B_STAGE_BYTES;
#pragma unroll
            for (int hs = 0; hs < 4; ++hs) {
                const int cur_a = hs & 1, cur_b = hs >> 1, mh = hs & 1;
                const int nhs = (hs + 1) & 3;
                // ra / rb: where the fragments of the next half step come from; for the last one of a tile, the first of
                // the next tile.  (After the last tile this fetches fragments nobody uses.)
                if (hs == 3) {
                    if (pace) {   // (see PACE_CYCLES; a sleep is 128 cycles, so the count bounds the wait whatever the counter's rate)
                        for (int n = 0; n < 24 && (int64_t)__builtin_readcyclecounter() - pace_t0 < PACE_CYCLES; ++n) __builtin_amdgcn_s_sleep(2);
                        pace_t0 = (int64_t)__builtin_readcyclecounter();
                    }
                    __builtin_amdgcn_s_waitcnt(0x0F70 | LPT);   // all but the youngest LPT loads: tile kt+1 has landed
                    __syncthreads();                            // for every wave; and every wave is done reading tile kt
                }
                const uint8_t* ra = (hs == 3) ? smem + (as ^ 1) * A_STAGE_BYTES : a_lds;
                const uint8_t* rb = (hs == 3) ? smem + B_REGION + bs1 * B_STAGE_BYTES : b_lds;
                __builtin_amdgcn_sched_barrier(0);
                // Wave priority falls as the wave advances through the period between two barriers (one level per half
                // step), so of the two waves of a SIMD the one that is behind issues first.  With equal priorities the
                // older wave of each SIMD wins every tie, runs a whole K tile ahead and then sits at the barrier while
                // the younger one works through its MFMAs alone, with nobody to fill its stalls (measured: the older
                // waves spent 34 % of the loop waiting at the barrier, the younger ones 5 %; with the levels 14 % and
                // 5 %, and the layer's GEMM launches run 3-4 % faster).  Levels that change inside a half step are slower.
                auto prio_at = [&](int g) {
                    if (g < MFMAS_PER_STEP) __builtin_amdgcn_s_setprio(3);
                    else if (g < 2 * MFMAS_PER_STEP) __builtin_amdgcn_s_setprio(2);
                    else if (g < 3 * MFMAS_PER_STEP) __builtin_amdgcn_s_setprio(1);
                    else __builtin_amdgcn_s_setprio(0);
                };
                const int g0 = ((hs + 1) & 3) * MFMAS_PER_STEP;   // MFMAs since the barrier
                prio_at(g0);
#pragma unroll
                for (int m = 0; m < MFMAS_PER_STEP; ++m) {
                    // boustrophedon order over the half step's MBH x NB blocks: from one MFMA to the next only one of the two
                    // operand fragments changes, never both (the matrix cores draw less power when an operand is repeated:
                    // on this clock-limited part that is 0.5 % of the GEMM launches; the accumulation order does not change)
                    const int mb = m / NB, nb = (mb & 1) ? NB - 1 - m % NB : m % NB;
                    if (m % READ_GAP == 0) {
                        const int nbr = ((nhs & 1) == 0) ? NB : 0;   // weight fragments first, when a new k step starts
                        const int q = m / READ_GAP;
                        if (q < nbr) { if (NBLK > 0) read_b1(rb, nhs >> 1, q, bf[cur_b ^ 1]); __builtin_amdgcn_sched_barrier(0); }
                        // (a wave does not fetch the fragments of row blocks beyond its count: its MFMAs on them are skipped too)
                        else if (q - nbr < MBH) { if ((nhs & 1) * MBH + (q - nbr) < NBLK) read_a1(ra, nhs >> 1, nhs & 1, q - nbr, af[cur_a ^ 1]); __builtin_amdgcn_sched_barrier(0); }
                    }
                    if (hs == 3 && m % A_LOAD_GAP == 0 && m / A_LOAD_GAP < LPT) {
                        if (SLAB) issue_slab(m / A_LOAD_GAP, as); else issue_a(kt + 2, m / A_LOAD_GAP, as, !FULL);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                    const int gb = hs * MFMAS_PER_STEP + m;   // MFMAs since the tile's first
                    if (hs < 3 && gb % B_LOAD_GAP == 0 && gb / B_LOAD_GAP < LPT) {
                        issue_b(kt + 2, gb / B_LOAD_GAP, bs2);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                    if (mh * MBH + mb < NBLK)
                        acc[mh * MBH + mb][nb] = Num::mfma(bf[cur_b][nb], af[cur_a][mb], acc[mh * MBH + mb][nb]);
                }
                __builtin_amdgcn_s_setprio(0);
                __builtin_amdgcn_sched_barrier(0);
            }
            bs = bs1;
        };
        // The tile before the last requests "tile ke": with slabs to fetch it runs a copy of the loop body whose
        // activation loads are the slab image's (selecting the operands inside the one loop body instead costs every
        // iteration some twenty scalar instructions, and the launch 1.7 %).
        int kt = kb;
        for (; kt < ke - 2; ++kt) tile(kt, std::false_type{});
        if (lds_slabs && kt == ke - 2) { tile(kt, std::true_type{}); ++kt; }
        for (; kt < ke; ++kt) tile(kt, std::false_type{});
        __builtin_amdgcn_s_waitcnt(0x0F70);   // loads past the last tile must not land in the epilogue's staging
        __syncthreads();   // operand buffers are free for the epilogue staging
    };
    // full tiles run a loop body without any checks; in a ragged tile the activation loads of dead row blocks are dropped
    // and every wave takes the loop for the number of its live blocks (a scalar: the same in all lanes of the wave)
    if (live_rows == BM) mainloop(std::integral_constant<int, MB>{}, std::true_type{});
    else if (mb_cnt > MBH) mainloop(std::integral_constant<int, MB>{}, std::false_type{});
    else if (mb_cnt > 2) mainloop(std::integral_constant<int, MBH>{}, std::false_type{});
    else if (mb_cnt == 2) mainloop(std::integral_constant<int, 2>{}, std::false_type{});
    else if (mb_cnt == 1) mainloop(std::integral_constant<int, 1>{}, std::false_type{});
    else mainloop(std::integral_constant<int, 0>{}, std::false_type{});
    if (!p.y_grouped) {   // the output row table again: weight tiles have passed through its place
        for (int r = tid; r < BM; r += NTHREADS) s_outrow[r] = load_idx(p.pos, row0 + ((r < nrows) ? r : nrows - 1), p.pos64);
        __syncthreads();
    }

    // ---- K parts of a split tile: every part publishes its fp32 partial tile and then bumps the tile's counter; the
    // part that finds all others already counted sums the partials in part order (so the result does not depend on who
    // arrives last) and finishes the tile.  Nobody waits for anybody.  The partials travel through device-coherent
    // (agent scope) stores and loads, which are visible across the XCDs' separate L2 caches without flushing or
    // invalidating those caches.
    if (nparts > 1) {
        const int ti = item.split_tile;   // number of the split tile, < #CU
        // 16 bytes per lane and access, device scope (the cache-policy bit that the compiler's agent-scope atomics set):
        // partial element (mb, nb, r) of thread tid sits at float ((mb*NB + nb) * NTHREADS + tid) * 4 + r of the slot
        constexpr int DEVICE_SCOPE = 16;
        const __amdgpu_buffer_rsrc_t xbuf = __builtin_amdgcn_make_buffer_rsrc(p.sk_partials, 0, (int)0x80000000u, 0x00020000);
        const uint32_t slot_bytes = (uint32_t)split_item * (uint32_t)(BM * BN * sizeof(float));
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                u32x4_t v;
#pragma unroll
                for (int r = 0; r < 4; ++r) v[r] = __float_as_uint(acc[mb][nb][r]);
                __builtin_amdgcn_raw_buffer_store_b128(v, xbuf, slot_bytes + (uint32_t)(((mb * NB + nb) * NTHREADS + tid) * 16), 0, DEVICE_SCOPE);
            }
        __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): this wave's stores are acknowledged
        __syncthreads();                      // ... and every wave's: the partial is visible
        // release + acquire at agent scope: the parts of a tile run on different XCDs with separate L2 caches, and the part that
        // counts last must find every earlier part's partial (a relaxed increment lets it read stale lines)
        if (tid == 0) *s_arrival = __hip_atomic_fetch_add(&p.sk_counters[ti], 1, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        if (*s_arrival != nparts - 1) return;
        if (tid == 0) __hip_atomic_store(&p.sk_counters[ti], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // clean for the next launch
        const uint32_t first_bytes = (uint32_t)(split_item - part) * (uint32_t)(BM * BN * sizeof(float));
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                const uint32_t o = first_bytes + (uint32_t)(((mb * NB + nb) * NTHREADS + tid) * 16);
                u32x4_t v = __builtin_amdgcn_raw_buffer_load_b128(xbuf, o, 0, DEVICE_SCOPE);
                float sum[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) sum[r] = __uint_as_float(v[r]);
                for (int x = 1; x < nparts; ++x) {
                    v = __builtin_amdgcn_raw_buffer_load_b128(xbuf, o + (uint32_t)x * (uint32_t)(BM * BN * sizeof(float)), 0, DEVICE_SCOPE);
#pragma unroll
                    for (int r = 0; r < 4; ++r) sum[r] += __uint_as_float(v[r]);
                }
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[mb][nb][r] = sum[r];
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }

    // ---- low-rank slabs: 16 k each.  The MFMA step is 32 k wide: lanes 0..31 carry k 0..15, lanes 32..63 k 16..31, so a
    // step takes two slabs (or one, with zeros in the upper lanes).  With slab_mode 0 all slabs feed every column and
    // pair up in order; with slab_mode 1 (gate/up pair) the first half of the slabs feeds the gate columns and the
    // second half the up columns, pairing within each half.  Up to four slabs make at most two steps.  One or two slabs
    // are read from the LDS image that the main loop fetched as "the tile after the last" (the gate/up launch 1.5 %
    // faster than with the round trip to memory here); three or four come straight from global memory, all fragments
    // requested before the first of them is used, so that the tile pays one memory round trip, not one per fragment.
    // More than MOE_MAX_SLABS slabs (an adapter rank above 64, above 32 for the gate/up pair; general variant): the slabs
    // are slab_stride-spaced copies of Q[0] / LB[0] and are worked through two per MFMA step in a loop, each step's
    // fragments straight from global memory -- one round trip per 32 rank columns, paid only by such ranks.
    if constexpr (KTAIL) {
        if (p.nslab > MOE_MAX_SLABS) {
            const int kc = (lane >> 4) & 1;
            const bool upper = lane >= 32;
            const int ngroups = p.slab_mode == 0 ? 1 : 2;   // slab_mode 1: gate slabs, then up slabs
            const int per_group = p.nslab / ngroups;
#pragma unroll 1
            for (int grp = 0; grp < ngroups; ++grp) {
#pragma unroll 1
                for (int l = 0; l < per_group; l += 2) {
                    const bool has_hi = l + 1 < per_group;
                    const int src = grp * per_group + ((upper && has_hi) ? l + 1 : l);
                    const bool live = !upper || has_hi;
                    const uint16_t* Q = p.Q[0] + (int64_t)src * p.q_slab_stride;
                    const uint16_t* LB = p.LB[0] + (int64_t)src * p.lb_slab_stride + (int64_t)expert * p.N * 16;
                    bf16x8_t ta[MB], tb[NB];
#pragma unroll
                    for (int nb = 0; nb < NB; ++nb) {
                        int64_t n = (EPI_IS_PAIR(EPI)) ? n0 + wn * (WTN / 2) + (nb % NBH) * 16 + (lane & 15) : n0 + wn * WTN + nb * 16 + (lane & 15);
                        if (n >= p.N) n = p.N - 1;
                        bf16x8_t v = {};
                        if (live) v = *(const bf16x8_t*)(LB + n * 16 + 8 * kc);
                        tb[nb] = v;
                    }
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb) {
                        int r = wm * WTM + mb * 16 + (lane & 15);
                        if (r >= nrows) r = nrows - 1;
                        bf16x8_t v = {};
                        if (live) v = *(const bf16x8_t*)(Q + (row0 + r) * 16 + 8 * kc);
                        ta[mb] = v;
                    }
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb)
                        if (mb < mb_cnt) {
#pragma unroll
                            for (int nb = 0; nb < NB; ++nb)
                                if (p.slab_mode == 0 || nb / NBH == grp) acc[mb][nb] = Num::mfma(tb[nb], ta[mb], acc[mb][nb]);
                        }
                }
            }
        }
    }
    if (!KTAIL || p.nslab <= MOE_MAX_SLABS) {
        const int kc = (lane >> 4) & 1;          // which 8 of a slab's 16 k this lane holds
        const bool upper = lane >= 32;
        const int per_group = p.slab_mode == 0 ? p.nslab : p.nslab / 2;   // slabs per column group
        const int steps_per_group = (per_group + 1) / 2;
        const int nsteps = p.slab_mode == 0 ? steps_per_group : 2 * steps_per_group;
        bf16x8_t sa[2][MB], sb[2][NB];
        int group_of[2] = {-1, -1};              // column group a step feeds (-1: all columns)
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            if (s < nsteps) {
                const int grp = p.slab_mode == 0 ? 0 : s / steps_per_group;
                const int lo = grp * per_group + 2 * (s % steps_per_group);
                const bool has_hi = 2 * (s % steps_per_group) + 1 < per_group;
                group_of[s] = p.slab_mode == 0 ? -1 : grp;
                const int src = (upper && has_hi) ? lo + 1 : lo;
                const bool live = !upper || has_hi;
                if (lds_slabs) {
                    // image of the tile after the last: Q[src] rows at src * 8 KiB, LB[src] columns 16 KiB further up
                    const uint8_t* img = smem + ((ke - kb) & 1) * A_STAGE_BYTES + src * (BM * 32) + 16 * kc;
#pragma unroll
                    for (int nb = 0; nb < NB; ++nb) {
                        const int c = (EPI_IS_PAIR(EPI)) ? wn * (WTN / 2) + (nb % NBH) * 16 + (lane & 15) : wn * WTN + nb * 16 + (lane & 15);
                        bf16x8_t v = {};
                        if (live) v = *(const bf16x8_t*)(img + 2 * (BM * 32) + c * 32);
                        sb[s][nb] = v;
                    }
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb) {
                        bf16x8_t v = {};
                        if (live) v = *(const bf16x8_t*)(img + (wm * WTM + mb * 16 + (lane & 15)) * 32);
                        sa[s][mb] = v;
                    }
                    continue;
                }
                const uint16_t* Q = p.Q[src];
                const uint16_t* LB = p.LB[src] + (int64_t)expert * p.N * 16;
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) {
                    int64_t n = (EPI_IS_PAIR(EPI)) ? n0 + wn * (WTN / 2) + (nb % NBH) * 16 + (lane & 15) : n0 + wn * WTN + nb * 16 + (lane & 15);
                    if (n >= p.N) n = p.N - 1;
                    bf16x8_t v = {};
                    if (live) v = *(const bf16x8_t*)(LB + n * 16 + 8 * kc);
                    sb[s][nb] = v;
                }
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) {
                    int r = wm * WTM + mb * 16 + (lane & 15);
                    if (r >= nrows) r = nrows - 1;
                    bf16x8_t v = {};
                    if (live) v = *(const bf16x8_t*)(Q + (row0 + r) * 16 + 8 * kc);
                    sa[s][mb] = v;
                }
            }
        }
        if (lds_slabs) {
            __builtin_amdgcn_s_waitcnt(0xC07F);   // lgkmcnt(0): this wave holds its fragments ...
            __syncthreads();                      // ... and so does every other, before anybody's epilogue staging overwrites the image
        }
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            if (s < nsteps) {
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
                    if (mb < mb_cnt) {
#pragma unroll
                        for (int nb = 0; nb < NB; ++nb)
                            if (group_of[s] < 0 || nb / NBH == group_of[s])
                                acc[mb][nb] = Num::mfma(sb[s][nb], sa[s][mb], acc[mb][nb]);
                    }
            }
        }
    }

    // ---- epilogue.  acc[mb][nb][r] is element (row m = mb*16 + lane%16, column n = nb*16 + (lane/16)*4 + r) of the
    // wave's sub-tile: 4 consecutive columns per lane and block.  Each wave stages its sub-tile as bf16 in its own
    // slice of the (now idle) operand buffers and writes it out with 16-byte stores, whole row segments at a time.
    uint8_t* stg = smem + wave * (WTM * WTN * 2);   // WTM x WTN bf16 per wave
    const int mrow = lane & 15, nq = (lane >> 4) * 4;
    float rs[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        const int rl = wm * WTM + mb * 16 + mrow;
        rs[mb] = (p.row_scale && rl < nrows) ? p.row_scale[row0 + rl] : 1.f;
    }
    auto pack4 = [](float a, float b, float c, float d) {
        uint2 v;
        v.x = Num::pack2(a, b);
        v.y = Num::pack2(c, d);
        return v;
    };
    // Staging image of SW columns per row (SW*2 bytes, SW/8 chunks of 16 bytes).  256 bytes span the 64 LDS banks, so
    // the chunk index is XORed with the row number counted in units of 256 bytes: the 32 rows a store instruction
    // touches then spread over the banks.  A lane writes 8 bytes: columns [ncol, ncol+4) of row m.
    auto swz = [](int sw, int m, int c) { return c ^ ((m / (sw >= 128 ? 1 : 128 / sw)) & (sw / 8 - 1)); };
    auto stage_put = [&](int sw, int m, int ncol, uint2 v) {
        const int c = ncol >> 3, half = (ncol >> 2) & 1;
        *(uint2*)(stg + m * (sw * 2) + (swz(sw, m, c) << 4) + half * 8) = v;
    };
    // write the staged sub-tile to Y (grouped rows or rows from the table), columns [ncol0, ncol0 + sw).  The stores go
    // through a buffer descriptor with 32-bit byte offsets; lanes outside the tile's rows or the matrix's columns
    // get an offset past the descriptor's range, which the hardware drops, so the loop has no branches.
    auto stage_flush = [&](int sw, uint16_t* Y, int64_t ld, bool scattered, int64_t ncol0) {
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): this wave's staging writes have landed
        // grouped rows: the descriptor starts at the tile's first row, so offsets stay within one tile
        const __amdgpu_buffer_rsrc_t ybuf = __builtin_amdgcn_make_buffer_rsrc(scattered ? Y : Y + row0 * ld, 0, (int)0x80000000u, 0x00020000);
        const int lpr = sw / 8, rows_per_it = 64 / lpr, iters = WTM / rows_per_it;
        const int slot = lane % lpr;
        const uint32_t ld2 = (uint32_t)ld * 2;
        if (scattered && p.y_wide) {
            // scattered rows of an output beyond the 2 GiB a descriptor offset spans: 64-bit addresses, a branch per lane
            for (int it = 0; it < iters; ++it) {
                const int m = it * rows_per_it + lane / lpr;
                const u32x4_t v = *(const u32x4_t*)(stg + m * (sw * 2) + slot * 16);
                const int rl = wm * WTM + m;
                const int64_t n = ncol0 + swz(sw, m, slot) * 8;
                if (rl < nrows && n < p.N) *(u32x4_t*)(Y + s_outrow[rl] * ld + n) = v;
            }
        } else {
#pragma unroll 8
            for (int it = 0; it < iters; ++it) {
                const int m = it * rows_per_it + lane / lpr;
                const u32x4_t v = *(const u32x4_t*)(stg + m * (sw * 2) + slot * 16);
                const int rl = wm * WTM + m;
                const int64_t n = ncol0 + swz(sw, m, slot) * 8;
                const uint32_t orow = scattered ? (uint32_t)s_outrow[rl] : (uint32_t)rl;
                const uint32_t off = (rl < nrows && n < p.N) ? orow * ld2 + (uint32_t)n * 2 : 0xFFFFFFF0u;
                __builtin_amdgcn_raw_buffer_store_b128(v, ybuf, off, 0, 0);
            }
        }
        __builtin_amdgcn_s_waitcnt(0xC07F);  // reads done before the slice is reused
    };

    if (EPI == MOE_EPI_STORE) {
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                const float s_ = rs[mb];
                stage_put(WTN, mb * 16 + mrow, nb * 16 + nq, pack4(acc[mb][nb][0] * s_, acc[mb][nb][1] * s_, acc[mb][nb][2] * s_, acc[mb][nb][3] * s_));
            }
        stage_flush(WTN, p.Y[0], p.ldy, !p.y_grouped, n0 + wn * WTN);
    } else if (EPI_IS_PAIR(EPI)) {
        // gate = acc[mb][j], up = acc[mb][NBH + j] at identical (row, column) positions.  Outputs: Y0 = h = silu(gate) * up,
        // computed from the fp32 accumulators, and optionally Y1 = gate, Y2 = up for the backward pass.  One sweep produces
        // all three; gate and up wait for their passes already rounded and packed, in half of the accumulators' registers.
        const int64_t ncol0 = n0 + wn * (WTN / 2);
#pragma unroll
        for (int pass = 0; pass < 3; ++pass) {
            uint16_t* Y = p.Y[pass];
            if (!Y) continue;
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int nj = 0; nj < NBH; ++nj) {
                    if (pass == 0) {
                        float o[4], g[4], u[4];
#pragma unroll
                        for (int t = 0; t < 4; ++t) {
                            g[t] = acc[mb][nj][t];
                            u[t] = acc[mb][NBH + nj][t];
                            o[t] = g[t] * sigmoid_f(g[t]) * u[t];
                        }
                        stage_put(WTN / 2, mb * 16 + mrow, nj * 16 + nq, pack4(o[0], o[1], o[2], o[3]));
                        const uint2 pg = pack4(g[0], g[1], g[2], g[3]), pu = pack4(u[0], u[1], u[2], u[3]);
                        acc[mb][nj][0] = __uint_as_float(pg.x); acc[mb][nj][1] = __uint_as_float(pg.y);
                        acc[mb][NBH + nj][0] = __uint_as_float(pu.x); acc[mb][NBH + nj][1] = __uint_as_float(pu.y);
                    } else {
                        const int src = pass == 1 ? nj : NBH + nj;
                        uint2 v;
                        v.x = __float_as_uint(acc[mb][src][0]);
                        v.y = __float_as_uint(acc[mb][src][1]);
                        stage_put(WTN / 2, mb * 16 + mrow, nj * 16 + nq, v);
                    }
                }
            if (EPI == MOE_EPI_SWIGLU_FUSED && pass == 0) {
                // Fused column contraction (the low-rank interim of the next GEMM): CCP[0][nt][m][r] = sum_n h[m][n] CB[0][e][n][r]
                // over this tile's 128 columns of h, from the staged image of h (read row-major: the contraction index is the
                // column; this wave's 32 columns are one MFMA step), so that h is not read from memory again for it.  CB is the
                // adapter factor in MFMA fragment order.  The wave parks its sums in the free half of its staging slot.
                const int64_t hcol = n0 + wn * (WTN / 2);
                bf16x8_t cb = {};
                if (hcol < p.N) cb = *(const bf16x8_t*)(p.CB[0] + ((int64_t)expert * p.N + hcol) * 16 + lane * 8);
                float* park = (float*)(stg + WTM * (WTN / 2) * 2);
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) {
                    const bf16x8_t hf = *(const bf16x8_t*)(stg + (mb * 16 + (lane & 15)) * (WTN / 2 * 2) + (((lane >> 4) ^ ((lane >> 2) & 3)) << 4));
                    const f32x4_t z = {0.f, 0.f, 0.f, 0.f};
                    const f32x4_t d_ = Num::mfma(hf, cb, z);
                    *(f32x4_t*)(park + (mb * 64 + lane) * 4) = d_;
                }
            }
            stage_flush(WTN / 2, Y, p.ldy, false, ncol0);
        }
        if (EPI == MOE_EPI_SWIGLU_FUSED) {
            // element (row = mb*16 + 4*(lane/16) + reg, rank column lane%16) of every column wave's sums is parked in its slot;
            // wave (wm, wn) adds the four column waves' sums (in wave order) of row blocks 2 wn, 2 wn + 1 and stores them
            __builtin_amdgcn_s_waitcnt(0xC07F);
            __syncthreads();
            const int tg = lane >> 4, ti = lane & 15;
#pragma unroll
            for (int h2 = 0; h2 < 2; ++h2) {
                const int mb = 2 * wn + h2;
                f32x4_t sum = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int w2 = 0; w2 < WAVES_N; ++w2) {
                    const float* src = (const float*)(smem + (wm * WAVES_N + w2) * (WTM * WTN * 2) + WTM * (WTN / 2) * 2);
                    const f32x4_t v = *(const f32x4_t*)(src + (mb * 64 + lane) * 4);
#pragma unroll
                    for (int reg = 0; reg < 4; ++reg) sum[reg] += v[reg];
                }
                const int rl0 = wm * WTM + mb * 16 + 4 * tg;
                float* dst = p.CCP[0] + ((int64_t)nt * p.cc_rows + row0 + rl0) * 16 + ti;
#pragma unroll
                for (int reg = 0; reg < 4; ++reg)
                    if (rl0 + reg < nrows) dst[reg * 16] = sum[reg];
            }
        }
    } else {  // MOE_EPI_SWIGLU_BWD: acc = dh; dgate = dh * up * sig(g) * (1 + g (1 - sig(g))), dup = dh * silu(g)
        // dh (scaled by the row's routing weight) is staged as bf16 -- the precision a stored dh would have -- and
        // then revisited row segment by row segment: 8 lanes cover 128 bytes of a row, so the matching gate / up
        // values are fetched, and dgate / dup written, with full-width coalesced accesses.
        // (all four are grouped rows: descriptors start at the tile's first row)
        const __amdgpu_buffer_rsrc_t gbuf = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(p.H1) + row0 * p.ldh, 0, (int)0x80000000u, 0x00020000);
        const __amdgpu_buffer_rsrc_t ubuf = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(p.H3) + row0 * p.ldh, 0, (int)0x80000000u, 0x00020000);
        const __amdgpu_buffer_rsrc_t dgbuf = __builtin_amdgcn_make_buffer_rsrc(p.Y[0] + row0 * p.ldy, 0, (int)0x80000000u, 0x00020000);
        const __amdgpu_buffer_rsrc_t dubuf = __builtin_amdgcn_make_buffer_rsrc(p.Y[1] + row0 * p.ldy, 0, (int)0x80000000u, 0x00020000);
        // gate / up are read once and dgate / dup written once per launch: the non-temporal hint keeps them from
        // displacing operand tiles in L2 (measured: this kernel 2 % faster; on the plain output stores it is slower)
        constexpr int STREAMING = 2;
        constexpr int LPR = WTN / 8, ROWS_PER_IT = 64 / LPR;
        const int slot = lane % LPR;
        const uint32_t ldh2 = (uint32_t)p.ldh * 2, ldy2 = (uint32_t)p.ldy * 2;
        // The gate / up fetches run PD row segments ahead of the arithmetic -- the first ones are requested before dh is
        // staged -- so their latency is paid once per tile and not once per batch of segments (this launch 3-4 % faster).
        constexpr int NIT = WTM / ROWS_PER_IT, PD = 4;   // (8 or 16 segments ahead measured no faster: the segment arithmetic, not the fetch, bounds this epilogue)
        u32x4_t g8[PD], u8[PD];
        auto seg_addr = [&](int it, uint32_t& hoff, uint32_t& yoff) {
            const int m = it * ROWS_PER_IT + lane / LPR;
            const int rl = wm * WTM + m;
            const int64_t n = n0 + wn * WTN + swz(WTN, m, slot) * 8;
            const bool valid = rl < nrows && n < p.N;
            const uint32_t row = (uint32_t)rl;
            hoff = valid ? row * ldh2 + (uint32_t)n * 2 : 0xFFFFFFF0u;   // out of range: reads zeros, writes nothing
            yoff = valid ? row * ldy2 + (uint32_t)n * 2 : 0xFFFFFFF0u;
        };
        auto fetch = [&](int it, int b) {
            uint32_t hoff, yoff;
            seg_addr(it, hoff, yoff);
            g8[b] = __builtin_amdgcn_raw_buffer_load_b128(gbuf, hoff, 0, STREAMING);
            u8[b] = __builtin_amdgcn_raw_buffer_load_b128(ubuf, hoff, 0, STREAMING);
        };
#pragma unroll
        for (int it = 0; it < PD; ++it) fetch(it, it);
        // ---- fused low-rank products (EPI = MOE_EPI_SWIGLU_BWD_FUSED): while dgate, dup and h = silu(gate) * up (recomputed
        // here from the stored gate / up; the forward's own h came from the unrounded accumulators and differs from it in
        // the last bit or two) pass through LDS, the tile also produces
        //   row contractions (adapter gradients that sum over the tile's rows m):
        //     RCP[0][mtile][n][r] = sum_m dgate[m][n] RC[0][m][r],  RCP[1] likewise with dup and RC[1],  RCP[2] with h and RC[2]
        //   column contractions (the low-rank interims of the next GEMM, sums over the tile's columns n):
        //     CCP[0][nt][m][r] = sum_n dgate[m][n] CB[0][e][n][r],  CCP[1] likewise with dup and CB[1]
        // so that none of the three (R, N) tensors is read from memory again for them.  Small reduction kernels add the
        // row tiles per expert / the column tiles (in order), scale and round.  RC: bf16 [R][16] in grouped order, brought
        // into LDS once per tile; CB: adapter factor in MFMA fragment order (lane i + 16 g of fragment kb holds
        // factor[32 kb + 8 g .. + 7][i]).
        constexpr bool FUSED = EPI == MOE_EPI_SWIGLU_BWD_FUSED;
        uint8_t* rc_img = smem + RC_IMG_OFF;
        u32x4_t rc_in[RC_MATS];
        if (FUSED) {
            const int r_ = tid >> 1;                                   // tile row of this thread's 16 bytes
            const int64_t m_ = row0 + (r_ < nrows ? r_ : nrows - 1);   // rows past the group re-read its last row (they meet zeros)
#pragma unroll
            for (int mat = 0; mat < RC_MATS; ++mat) rc_in[mat] = *(const u32x4_t*)(p.RC[mat] + m_ * 16 + (tid & 1) * 8);
        }
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                const float s_ = rs[mb];
                stage_put(WTN, mb * 16 + mrow, nb * 16 + nq, pack4(acc[mb][nb][0] * s_, acc[mb][nb][1] * s_, acc[mb][nb][2] * s_, acc[mb][nb][3] * s_));
            }
        if (FUSED) {
            static_assert(NTHREADS * 16 == RC_IMG_BYTES, "one 16-byte piece of every operand image per thread");
#pragma unroll
            for (int mat = 0; mat < RC_MATS; ++mat) *(u32x4_t*)(rc_img + mat * RC_IMG_BYTES + tid * 16) = rc_in[mat];
            __syncthreads();   // the images are complete (and, for this wave, its dh staging)
        }
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): this wave's staging writes have landed
        // transposing reads (see the N-contiguous weight fragments): lane 16g + i fetches 4 columns at row 8g + (i >> 2)
        // and 4 rows further down, and receives rows 8g .. 8g+7 of column i -- a 16x16x32 operand whose contraction
        // index is the row.  Offsets within a block of 32 rows of this wave's staging slice / of an operand image.
        const int tg = lane >> 4, ti = lane & 15;
        const int trow = 8 * tg + (ti >> 2);
        constexpr int IBLK = WTN / 16;   // 16-column blocks of the wave's sub-tile
        constexpr int CC_MATS = 2, CC_KS = WTN / 32;
        f32x4_t rcd[RC_MATS][IBLK];      // row contractions, accumulated over the wave's 128 rows
        bf16x8_t cbf[CC_MATS][CC_KS];    // this wave's fragments of the two adapter factors
        if (FUSED) {
#pragma unroll
            for (int mat = 0; mat < RC_MATS; ++mat)
#pragma unroll
                for (int ib = 0; ib < IBLK; ++ib) rcd[mat][ib] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int mat = 0; mat < CC_MATS; ++mat)
#pragma unroll
                for (int ks = 0; ks < CC_KS; ++ks) {
                    const int64_t ncol = n0 + wn * WTN + ks * 32;
                    bf16x8_t v = {};
                    if (ncol < p.N) v = *(const bf16x8_t*)(p.CB[mat] + ((int64_t)expert * p.N + ncol) * 16 + lane * 8);
                    cbf[mat][ks] = v;
                }
        }
        auto tr_read = [&](const uint8_t* p0, const uint8_t* p1) {
            s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)LDS_PTR(p0));
            s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)LDS_PTR(p1));
            union { struct { s16x4_t a, b; } s; bf16x8_t v; } u;
            u.s.a = lo; u.s.b = hi;
            return u.v;
        };
        const int cc_frag_off = (lane & 15) * (WTN * 2);   // + (chunk ^ swizzle) * 16 per read
        constexpr int BLK_ITS = 32 / ROWS_PER_IT;   // row segments per block of 32 rows
        static_assert(NIT % BLK_ITS == 0 && PD <= BLK_ITS, "whole blocks of 32 rows");
#pragma unroll
        for (int blk = 0; blk < NIT / BLK_ITS; ++blk) {
            u32x4_t og8[BLK_ITS], ou8[BLK_ITS], hh8[BLK_ITS];
#pragma unroll
            for (int q = 0; q < BLK_ITS; ++q) {
                const int it = blk * BLK_ITS + q;
                const int m = it * ROWS_PER_IT + lane / LPR;
                const u32x4_t dh8 = *(const u32x4_t*)(stg + m * (WTN * 2) + slot * 16);
                uint32_t hoff, yoff;
                seg_addr(it, hoff, yoff);
                const u32x4_t gg = g8[it % PD], uu = u8[it % PD];
#pragma unroll
                for (int w2 = 0; w2 < 4; ++w2) {
                    float og[2], ou[2], hh[2];
#pragma unroll
                    for (int t = 0; t < 2; ++t) {
                        const float g = Num::to_f32((uint16_t)(gg[w2] >> (t * 16)));
                        const float u = Num::to_f32((uint16_t)(uu[w2] >> (t * 16)));
                        const float dh = Num::to_f32((uint16_t)(dh8[w2] >> (t * 16)));
                        const float sg = sigmoid_f(g);
                        og[t] = dh * u * sg * (1.f + g * (1.f - sg));
                        ou[t] = dh * g * sg;
                        hh[t] = g * sg * u;
                    }
                    og8[q][w2] = Num::pack2(og[0], og[1]);
                    ou8[q][w2] = Num::pack2(ou[0], ou[1]);
                    if (FUSED) hh8[q][w2] = Num::pack2(hh[0], hh[1]);
                    // Rows past the group must enter the contractions as exact zeros.  Their gate / up read as zeros, but
                    // their dh need not be finite: the accumulators of row blocks without real rows can hold anything (an
                    // MFMA that the compiler left under an execution mask instead of a branch runs all the same -- the
                    // matrix cores ignore the mask -- on fragments of rows that were never loaded), and 0 * inf is not 0.
                    if (FUSED && wm * WTM + m >= nrows) og8[q][w2] = ou8[q][w2] = 0u;
                }
                if (it + PD < NIT) fetch(it + PD, it % PD);
                __builtin_amdgcn_raw_buffer_store_b128(og8[q], dgbuf, yoff, 0, STREAMING);
                __builtin_amdgcn_raw_buffer_store_b128(ou8[q], dubuf, yoff, 0, STREAMING);
            }
            if (FUSED) {
                // The block's 32 rows of this wave's slice have been consumed: dgate, dup and h take their place in turn
                // (same swizzled positions); each is read back transposed for its row contraction and, dgate and dup,
                // row-major for the column contractions.  LDS serves a wave's requests in order, so the next operand's
                // writes and reads are queued behind the current one's reads before its MFMAs start.
                uint8_t* blk_img = stg + blk * 32 * (WTN * 2);
                bf16x8_t pf[2], vf[2][IBLK], cf[2][2][CC_KS];   // two generations of fragments
                f32x4_t ccd[CC_MATS][2];                          // column contractions of the block's two 16-row blocks
#pragma unroll
                for (int mat = 0; mat < CC_MATS; ++mat)
#pragma unroll
                    for (int rb = 0; rb < 2; ++rb) ccd[mat][rb] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
                auto queue = [&](int mat) {
                    const int gen = mat & 1;
#pragma unroll
                    for (int q = 0; q < BLK_ITS; ++q) {
                        const int m = (blk * BLK_ITS + q) * ROWS_PER_IT + lane / LPR;
                        *(u32x4_t*)(stg + m * (WTN * 2) + slot * 16) = mat == 0 ? og8[q] : (mat == 1 ? ou8[q] : hh8[q]);
                    }
                    asm volatile("" ::: "memory");   // the reads below follow the writes above in program order
                    const uint8_t* pim = rc_img + mat * RC_IMG_BYTES + (wm * WTM + blk * 32 + trow) * 32 + (ti & 3) * 8;
                    pf[gen] = tr_read(pim, pim + 4 * 32);
#pragma unroll
                    for (int ib = 0; ib < IBLK; ++ib) {
                        const int c = 2 * ib + ((ti & 3) >> 1), half = ti & 1;
                        const int r0_ = blk * 32 + trow, r1_ = r0_ + 4;   // rows within the slice (their swizzle term is (row >> 1) & 7)
                        const uint8_t* a0 = blk_img + trow * (WTN * 2) + ((c ^ ((r0_ >> 1) & 7)) << 4) + half * 8;
                        const uint8_t* a1 = blk_img + (trow + 4) * (WTN * 2) + ((c ^ ((r1_ >> 1) & 7)) << 4) + half * 8;
                        vf[gen][ib] = tr_read(a0, a1);
                    }
                    if (mat < CC_MATS) {
#pragma unroll
                        for (int rb = 0; rb < 2; ++rb)
#pragma unroll
                            for (int ks = 0; ks < CC_KS; ++ks)
                                cf[gen][rb][ks] = *(const bf16x8_t*)(blk_img + rb * 16 * (WTN * 2) + cc_frag_off + (((ks * 4 + (lane >> 4)) ^ ((lane >> 1) & 7)) << 4));
                    }
                    asm volatile("" ::: "memory");   // ... and the next operand's writes follow these reads
                };
                auto consume = [&](int mat) {
                    const int gen = mat & 1;
#pragma unroll
                    for (int ib = 0; ib < IBLK; ++ib)
                        rcd[mat][ib] = Num::mfma(vf[gen][ib], pf[gen], rcd[mat][ib]);
                    if (mat < CC_MATS) {
#pragma unroll
                        for (int rb = 0; rb < 2; ++rb)
#pragma unroll
                            for (int ks = 0; ks < CC_KS; ++ks)
                                ccd[mat][rb] = Num::mfma(cf[gen][rb][ks], cbf[mat][ks], ccd[mat][rb]);
                    }
                };
                queue(0);
                queue(1);
                consume(0);
                queue(2);
                consume(1);
                consume(2);
                // the block's column contractions are complete (they only sum over this wave's 64 columns): they take the
                // block's place in the slice -- 4 KiB, [product][16-row block][lane] -- until the waves exchange them below
#pragma unroll
                for (int mat = 0; mat < CC_MATS; ++mat)
#pragma unroll
                    for (int rb = 0; rb < 2; ++rb)
                        *(f32x4_t*)(blk_img + ((mat * 2 + rb) * 64 + lane) * 16) = ccd[mat][rb];
            }
        }
        if (FUSED) {
            // column contractions: element (row = 16-row block * 16 + 4 * (lane / 16) + reg, rank column lane % 16) summed
            // over one wave's 64 columns sits in that wave's slice; wave (wm, wn) adds the four column waves' sums (in wave
            // order) for the 32-row block wn of its row half and stores them
            __builtin_amdgcn_s_waitcnt(0xC07F);
            __syncthreads();
#pragma unroll
            for (int mat = 0; mat < CC_MATS; ++mat)
#pragma unroll
                for (int rb = 0; rb < 2; ++rb) {
                    f32x4_t sum = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int w2 = 0; w2 < WAVES_N; ++w2) {
                        const uint8_t* src = smem + (wm * WAVES_N + w2) * (WTM * WTN * 2) + wn * 32 * (WTN * 2);
                        const f32x4_t v = *(const f32x4_t*)(src + ((mat * 2 + rb) * 64 + lane) * 16);
#pragma unroll
                        for (int reg = 0; reg < 4; ++reg) sum[reg] += v[reg];
                    }
                    const int rl0 = wm * WTM + wn * 32 + rb * 16 + 4 * tg;
                    float* dst = p.CCP[mat] + ((int64_t)nt * p.cc_rows + row0 + rl0) * 16 + ti;
#pragma unroll
                    for (int reg = 0; reg < 4; ++reg)
                        if (rl0 + reg < nrows) dst[reg * 16] = sum[reg];
                }
            __builtin_amdgcn_s_waitcnt(0xC07F);
            __syncthreads();   // the slices are free again for the exchange below
            // row contractions: rcd[mat][ib][reg] = element (column ib*16 + 4*(lane/16) + reg, rank column lane%16) summed
            // over this wave's 128 rows: the lower row of waves parks its sums in its own slices, the upper one adds them
            // to its own (a fixed order) and stores the tile's partial
            float* xch = (float*)(smem + ((wave % WAVES_N) + WAVES_N) * (WTM * WTN * 2));
            if (wm == 1) {
#pragma unroll
                for (int mat = 0; mat < RC_MATS; ++mat)
#pragma unroll
                    for (int ib = 0; ib < IBLK; ++ib)
                        *(f32x4_t*)(xch + ((mat * IBLK + ib) * 64 + lane) * 4) = rcd[mat][ib];
            }
            __syncthreads();
            if (wm == 0) {
#pragma unroll
                for (int mat = 0; mat < RC_MATS; ++mat)
#pragma unroll
                    for (int ib = 0; ib < IBLK; ++ib) {
                        const f32x4_t o = *(const f32x4_t*)(xch + ((mat * IBLK + ib) * 64 + lane) * 4);
                        float* dst = p.RCP[mat] + ((int64_t)item.mtile * p.N + n0 + wn * WTN + ib * 16 + 4 * tg) * 16 + ti;
#pragma unroll
                        for (int reg = 0; reg < 4; ++reg)
                            if (n0 + wn * WTN + ib * 16 + 4 * tg + reg < p.N) dst[reg * 16] = rcd[mat][ib][reg] + o[reg];
                    }
            }
        }
    }
}

__global__ void zero_i32_kernel(int* p, int64_t n)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0;
}

// Workgroups of a launch: an upper bound on the output tiles plus one round for the split items.  Surplus workgroups
// leave at once.  (The cost-balanced ranges of a launch of few rounds differ in tile count; a plan whose largest range
// does not fit this grid falls back to ranges of equal counts.)
int64_t plan_grid(int64_t R, int E, int ntiles_n, int ncu)
{
    const int64_t grid = (R / BM + E) * ntiles_n + ncu;
    return (grid + NXCD - 1) / NXCD * NXCD;
}

template <bool NN, int EPI, typename Num, bool KTAIL> int launch_typed(const MoeGemmParams& p, int64_t R, hipStream_t stream)
{
    static std::atomic<bool> attr_set[MOE_MAX_DEVICES];   // per device; forward and backward may call from different host threads
    auto kern = grouped_gemm_mfma_kernel<NN, EPI, Num, KTAIL>;
    const int dev = moe_current_device();
    if (!attr_set[dev]) {
        if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES) != hipSuccess)
            return MOE_ERR_LAUNCH;
        attr_set[dev] = true;
    }
    const int ntiles_n = (EPI_IS_PAIR(EPI)) ? (int)((p.N + BN / 2 - 1) / (BN / 2)) : (int)((p.N + BN - 1) / BN);
    MoeGemmParams q = p;
    q.num_cus = moe_num_cus();
    q.y_wide = (!p.y_grouped && (R * p.ldy + p.N) * 2 >= ((int64_t)1 << 31)) ? 1 : 0;
    q.max_split = moe_gemm_max_split(EPI_IS_PAIR(EPI));
    if (q.max_split > 1) {
        if (!p.sk_partials || !p.sk_counters) return MOE_ERR_WORKSPACE;
        if (!p.counters_clean) hipLaunchKernelGGL(zero_i32_kernel, dim3((unsigned)((q.num_cus + 255) / 256)), dim3(256), 0, stream, p.sk_counters, (int64_t)q.num_cus);
    }
    const int64_t grid = plan_grid(R, p.E, ntiles_n, q.num_cus);
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(NTHREADS), LDS_BYTES, stream, q);
    return moe_launch_status();
}

// the kernel variant for the launch's 16-bit storage type
template <bool NN, int EPI> int launch_variant(const MoeGemmParams& p, int64_t R, hipStream_t stream)
{
    if (p.K % BK != 0 || p.nslab > MOE_MAX_SLABS) {   // a partial last K tile, many slabs: the plain epilogue, and the two SwiGLU epilogues without fused adapter products
        if constexpr (EPI == MOE_EPI_STORE || (!NN && (EPI == MOE_EPI_SWIGLU || EPI == MOE_EPI_SWIGLU_BWD)))
            return p.f16 ? launch_typed<NN, EPI, NumF16, true>(p, R, stream) : launch_typed<NN, EPI, NumBf16, true>(p, R, stream);
        else
            return MOE_ERR_UNSUPPORTED;
    }
    return p.f16 ? launch_typed<NN, EPI, NumF16, false>(p, R, stream) : launch_typed<NN, EPI, NumBf16, false>(p, R, stream);
}

}  // namespace


// The gate/up pair kernel never splits K (its launches have many more tiles than compute units); the others may cut
// the tiles of the last, partial round of compute units 2 or 4 ways.
int moe_gemm_max_split(bool pair) { return pair ? 1 : 4; }
int moe_gemm_num_counters() { return moe_num_cus(); }

static int plan_ntiles_n(int64_t N, int pair) { return pair ? (int)((N + BN / 2 - 1) / (BN / 2)) : (int)((N + BN - 1) / BN); }
int64_t moe_gemm_plan_blocks(int64_t R, int E, int64_t N, int pair) { return plan_grid(R, E, plan_ntiles_n(N, pair), moe_num_cus()); }
int moe_launch_gemm_plan(const void* offsets, int off64, int E, int64_t R, int64_t K, int64_t N, int pair, int nseg, int* out,
                         hipStream_t stream)
{
    if (K < BK || nseg < 1 || nseg > 2) return MOE_ERR_UNSUPPORTED;
    const int ntiles_n = plan_ntiles_n(N, pair);
    const int64_t grid = plan_grid(R, E, ntiles_n, moe_num_cus());
    hipLaunchKernelGGL(gemm_plan_kernel, dim3((unsigned)grid), dim3(64), 0, stream, offsets, off64, E, ntiles_n,
                       (int)((K + BK - 1) / BK) * nseg, moe_gemm_max_split(pair != 0), moe_num_cus(), out);
    return moe_launch_status();
}

// exchange area of a launch: one counter per split tile and one fp32 partial tile per split item; at most one round
// of compute units' worth of either
size_t moe_gemm_sk_bytes(int64_t R, int E, int64_t N)
{
    const int64_t tiles = (R / BM + E) * ((N + BN - 1) / BN);
    const int64_t slots = 4 * tiles < moe_num_cus() ? 4 * tiles : moe_num_cus();
    return (size_t)moe_gemm_num_counters() * sizeof(int) + 256 + (size_t)slots * BM * BN * sizeof(float);
}

void moe_gemm_sk_attach(MoeGemmParams& p, void* ws, int64_t, int, int64_t)
{
    p.sk_counters = (int*)ws;
    p.sk_partials = (float*)((uint8_t*)ws + (((size_t)moe_gemm_num_counters() * sizeof(int) + 255) & ~(size_t)255));
}

bool moe_gemm_mfma_supported(const MoeGemmParams& p, int64_t R)
{
    auto al16 = [](const void* q) { return q == nullptr || ((uintptr_t)q % 16) == 0; };
    // whole 64-wide K tiles run through the main loop (at least one), a remainder (multiple of 8) through the tail step
    if (p.K < BK || p.K % 8 != 0 || p.N % 8 != 0 || p.ldx % 8 != 0 || p.ldw % 8 != 0 || p.swe % 8 != 0) return false;
    if (!al16(p.X[0]) || !al16(p.X[1]) || !al16(p.W[0]) || !al16(p.W[1])) return false;
    for (int i = 0; i < MOE_MAX_SLABS; ++i)
        if (!al16(p.Q[i]) || !al16(p.LB[i])) return false;   // (slabs beyond these: multiples of 16 bytes from Q[0] / LB[0], checked below)
    if (p.nseg < 1 || p.nseg > 2 || p.nslab < 0 || (p.slab_mode == 1 && p.nslab % 2 != 0)) return false;
    if (p.K % BK != 0 && p.epi != MOE_EPI_STORE) return false;   // a partial last K tile: the plain epilogue only
    if (p.nslab > MOE_MAX_SLABS) {
        const bool epi_ok = p.epi == MOE_EPI_STORE || (!p.nn && (p.epi == MOE_EPI_SWIGLU || p.epi == MOE_EPI_SWIGLU_BWD));
        if (!epi_ok || (p.slab_mode == 1) != (p.epi == MOE_EPI_SWIGLU) || p.nslab > MOE_MAX_STRIDED_SLABS || p.q_slab_stride % 8 != 0 || p.lb_slab_stride % 8 != 0) return false;
    }
    // 32-bit byte offsets: gathered A rows from the start of X (grouped ones from the tile's first row), weights from
    // the start of one expert's matrix, grouped outputs and the saved gate / up from the tile's first row; scattered
    // output rows from the start of Y while Y spans less than 2 GiB, 64-bit addresses beyond (y_wide, set at launch)
    (void)R;
    const int fo = p.fan_out > 0 ? p.fan_out : 1;
    const int64_t x_rows = p.x_grouped ? BM : (R + fo - 1) / fo;
    // (a partial last K tile masks its loads through the descriptor's range, which that kernel variant sets to 2 GiB)
    const int64_t limit = (p.K % BK != 0) ? (int64_t)1 << 31 : (int64_t)1 << 32;
    if ((x_rows * p.ldx + p.K) * 2 >= limit) return false;
    if (((p.nn ? p.K : p.N) * p.ldw + (p.nn ? p.N : p.K)) * 2 >= limit) return false;
    if ((BM * p.ldy + p.N) * 2 >= ((int64_t)1 << 31)) return false;
    if ((p.epi == MOE_EPI_SWIGLU_BWD || p.epi == MOE_EPI_SWIGLU_BWD_FUSED) && (BM * p.ldh + p.N) * 2 >= ((int64_t)1 << 31)) return false;
    return true;
}

static std::atomic<int64_t> g_mfma_launches{0};
int64_t moe_gemm_mfma_launch_count() { return g_mfma_launches; }

int moe_launch_gemm_mfma(const MoeGemmParams& p, int64_t R, hipStream_t stream)
{
    if (R == 0 || p.N == 0) return MOE_OK;
    if (!moe_gemm_mfma_supported(p, R)) return MOE_ERR_UNSUPPORTED;
    ++g_mfma_launches;
    if (p.epi == MOE_EPI_STORE) return p.nn ? launch_variant<true, MOE_EPI_STORE>(p, R, stream) : launch_variant<false, MOE_EPI_STORE>(p, R, stream);
    if (p.epi == MOE_EPI_SWIGLU) return p.nn ? MOE_ERR_UNSUPPORTED : launch_variant<false, MOE_EPI_SWIGLU>(p, R, stream);
    if (p.epi == MOE_EPI_SWIGLU_FUSED) {
        if (p.nn || p.ncc != 1) return MOE_ERR_UNSUPPORTED;
        if (!p.CB[0] || !p.CCP[0] || !p.Y[0]) return MOE_ERR_BAD_ARG;
        return launch_variant<false, MOE_EPI_SWIGLU_FUSED>(p, R, stream);
    }
    if (p.epi == MOE_EPI_SWIGLU_BWD) return p.nn ? launch_variant<true, MOE_EPI_SWIGLU_BWD>(p, R, stream) : launch_variant<false, MOE_EPI_SWIGLU_BWD>(p, R, stream);
    if (p.epi == MOE_EPI_SWIGLU_BWD_FUSED) {
        if (p.nn || p.nrc != 3 || p.ncc != 2) return MOE_ERR_UNSUPPORTED;
        for (int i = 0; i < 3; ++i) if (!p.RC[i] || !p.RCP[i] || (i < 2 && (!p.CB[i] || !p.CCP[i]))) return MOE_ERR_BAD_ARG;
        return launch_variant<false, MOE_EPI_SWIGLU_BWD_FUSED>(p, R, stream);
    }
    return MOE_ERR_BAD_ARG;
}

