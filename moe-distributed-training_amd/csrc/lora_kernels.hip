// Low-rank (LoRA, rank <= 16) side kernels on the matrix cores, all HBM-bound:
//   pack_lora : strided adapter factor -> bf16 [E][K][16] (rank contiguous), or MFMA fragment order
//               [E][K/32][64 lanes][8]: lane i + 16 g of fragment kb holds A[32 kb + 8 g + 0..7][i]
//   rows_lora : Q[m][0:16] = bf16(scaling * X[in_row(m)][:] . A[e(m)][:][0:16]) for every sorted position m,
//               plus the transposed copy Qt[r][m]
//   xtp       : out[e][k][r] = scale * sum_{m in group e} X[m][k] * P[m][r]   (adapter gradients dA / dB)
// Summation order is fixed by the launch geometry only, so results are reproducible run to run.
#include "common.h"
#include "kernels.h"

namespace {

// Two jobs of a launch that read the same rows (x A1 and x A3, say) should run side by side on one XCD, so that the rows
// the first fetches serve the second from that XCD's L2: workgroups are dispatched to the 8 XCDs in turn by their linear
// number, so a one-dimensional grid deals units out in groups of 8 -- unit 8g + i of job j is workgroup (g * jobs + j) * 8 + i,
// eight workgroups behind its twin of the other job and on the same XCD.
constexpr int JOB_GROUP = 8;
__device__ __forceinline__ void unit_and_job(int njobs, int64_t* unit, int* job)
{
    const int64_t id = blockIdx.x;
    const int64_t group = id / (JOB_GROUP * njobs);
    const int within = (int)(id % (JOB_GROUP * njobs));
    *job = within / JOB_GROUP;
    *unit = group * JOB_GROUP + within % JOB_GROUP;
}
inline unsigned job_grid(int64_t units, int njobs) { return (unsigned)((units + JOB_GROUP - 1) / JOB_GROUP * JOB_GROUP * njobs); }

// (fragment order covers K rounded up to whole 32-wide fragments; positions at or past K hold zeros, so a consumer may
// feed them anything finite)
__global__ void pack_lora_kernel(const uint16_t* __restrict__ src, int64_t se, int64_t sk, int64_t sr,
                                 uint16_t* __restrict__ dst, int64_t K, int64_t Kimg, int rank, int transpose, int64_t total)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const int64_t e = i / (Kimg * 16), rem = i % (Kimg * 16);
    int64_t k;
    int r;
    if (transpose) {   // fragment order: one 16x16x32 operand fragment is 1 KiB of consecutive memory
        const int64_t kb = rem / 512;
        const int lane = (int)(rem % 512) / 8, t = (int)(rem % 8);
        r = lane & 15;
        k = kb * 32 + 8 * (lane >> 4) + t;
    } else { k = rem / 16; r = (int)(rem % 16); }           // dst[e][k][r]
    dst[i] = (r < rank && k < K) ? src[e * se + k * sk + r * sr] : (uint16_t)0;
}

// several pack jobs in one launch (blockIdx.y selects the job): the six factors of an MLP block are a few MB in total,
// so separate launches would cost more in launch latency than in data movement.  A thread produces 16 bytes: the 8
// consecutive output elements of a chunk walk the source with one stride (rank stride in [K][16] order, k stride in
// fragment order).  The launch also clears a small int array for its caller (the grouped GEMM's K-split counters),
// which saves that caller a launch of its own.
__global__ void pack_lora_batch_kernel(const MoePackBatch jobs)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (blockIdx.y == 0)
        for (int z = i; z < jobs.zero_n; z += gridDim.x * blockDim.x) jobs.zero_ptr[z] = 0;
    const MoePackJob& j = jobs.job[blockIdx.y];
    const int K = (int)j.K, rank = j.rank;
    const int per_e = K * 2;                 // chunks per expert
    if (i >= jobs.E * per_e) return;
    const int e = i / per_e, rem = i % per_e;
    int k, r;
    int64_t stride;
    if (j.transpose) {                        // chunk = (fragment kb, lane): r fixed, 8 consecutive k
        const int kb = rem >> 6, lane = rem & 63;
        r = lane & 15;
        k = kb * 32 + 8 * (lane >> 4);
        stride = j.sk;
    } else {                                  // chunk = (k, half): k fixed, 8 consecutive r
        k = rem >> 1;
        r = (rem & 1) * 8;
        stride = j.sr;
    }
    const uint16_t* sp = j.src + (int64_t)e * j.se + (int64_t)k * j.sk + (int64_t)r * j.sr;
    uint4 out;
    if (j.transpose ? (r >= rank) : false) {
        out = make_uint4(0, 0, 0, 0);
    } else if (stride == 1 && (((uintptr_t)sp) & 15) == 0 && (j.transpose || r + 8 <= rank)) {
        out = *(const uint4*)sp;
    } else {
        uint16_t v[8];
#pragma unroll
        for (int t = 0; t < 8; ++t) v[t] = (j.transpose || r + t < rank) ? sp[t * stride] : (uint16_t)0;
        out.x = v[0] | ((uint32_t)v[1] << 16); out.y = v[2] | ((uint32_t)v[3] << 16);
        out.z = v[4] | ((uint32_t)v[5] << 16); out.w = v[6] | ((uint32_t)v[7] << 16);
    }
    ((uint4*)j.dst)[i] = out;
}

// ---------------------------------------------------------------------------------------------------------
constexpr int RL_ROWS = 32;      // rows per workgroup at most: two 16-row MFMA blocks share every adapter fragment
constexpr int RL_WAVES = 8;
constexpr int RL_THREADS = RL_WAVES * 64;
constexpr int RL_KC = 256;                     // K elements per stage: one direct-to-LDS load instruction per two rows
constexpr int RL_PAIRP = 2 * RL_KC * 2 + 16;   // LDS pitch of a row pair: 8 pairs at one column fall into different bank groups
constexpr int RL_KSTEPS = RL_KC / 32;          // adapter fragments (1 KiB each) per stage
constexpr int RL_NSTAGE = 3;
constexpr int rl_xbytes(int rows) { return (rows / 2) * RL_PAIRP; }
constexpr int rl_stage(int rows) { return rl_xbytes(rows) + RL_KSTEPS * 1024; }
constexpr int rl_lds(int rows) { return RL_NSTAGE * rl_stage(rows); }
static_assert(RL_KSTEPS == RL_WAVES, "one K step per wave and stage");

// Everything is streamed through LDS with direct-to-LDS loads, three stages deep: a load instruction moves 1 KiB (two
// activation rows' 512 bytes, perfectly coalesced, or one adapter fragment), the MFMA operand fragments (16 rows x 8 K
// values per lane) are then read from LDS.  Loading the fragments straight from global memory would make adjacent
// lanes touch different rows, which the memory pipeline handles one lane at a time.  All global loads of the loop are
// inline assembly with explicit s_waitcnt: compiler-managed loads would wait for the prefetches queued behind them.
// one or two jobs per launch (see unit_and_job): same rows, shapes and scaling, different operand / output pointers
struct RowsLoraJob { const uint16_t* X; const uint16_t* Af; uint16_t* Q; uint16_t* Qt; uint16_t* Qs; };   // Qs: optional row-major copy scaled like Qt
// ROWS = 32 rows per workgroup, or 16 when a launch of 32-row tiles would leave most compute units with a single
// workgroup (and so with too few loads in flight)
template <int ROWS, typename Num>
__global__ void __launch_bounds__(RL_THREADS) rows_lora_kernel(const RowsLoraJob job0, const RowsLoraJob job1, int64_t ldx,
                                                               int64_t ldqt, const void* __restrict__ pos, int pos64,
                                                               const void* __restrict__ offsets, int off64, int E,
                                                               int64_t K, int fan_out, int x_grouped, float scaling,
                                                               const float* __restrict__ qt_row_scale, int njobs)
{
    int64_t tile_id;
    int job_id;
    unit_and_job(njobs, &tile_id, &job_id);
    const RowsLoraJob& job = job_id ? job1 : job0;
    const uint16_t* __restrict__ X = job.X;
    const uint16_t* __restrict__ Af = job.Af;
    uint16_t* __restrict__ Q = job.Q;
    uint16_t* __restrict__ Qt = job.Qt;
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
    RowTile rt;
    if (!find_row_tile(offsets, off64, E, ROWS, tile_id, &rt)) return;
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int i = lane & 15, g = lane >> 4;
    const int expert = __builtin_amdgcn_readfirstlane(rt.expert);
    const int64_t row0 = uniform_i64(rt.row0), row1 = uniform_i64(rt.row1);

    // this wave's row pairs of every stage: lanes 0..31 fetch the first row of a pair, lanes 32..63 the second
    constexpr int RL_XBYTES = rl_xbytes(ROWS), RL_STAGE = rl_stage(ROWS), NBLK = ROWS / 16;
    static_assert((ROWS / 2) % RL_WAVES == 0 && RL_WAVES * ROWS * 16 * 4 <= rl_lds(ROWS), "row pairs are dealt out evenly to the waves; the reduction reuses the stage buffers");
    constexpr int PPW = (ROWS / 2) / RL_WAVES;
    const uint16_t* rowptr[PPW];
#pragma unroll
    for (int q = 0; q < PPW; ++q) {
        int64_t m = row0 + (wave * PPW + q) * 2 + (lane >> 5);
        if (m >= row1) m = row1 - 1;   // rows past the group re-read its last row
        const int64_t in_row = x_grouped ? m : load_idx(pos, m, pos64) / fan_out;
        rowptr[q] = X + in_row * ldx;
    }
    const uint32_t lds0 = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)LDS_PTR(smem));
    const int64_t nksteps = (K + 31) / 32;   // the adapter image is zero beyond K: a partial last step takes whatever x the lanes past the row's end re-read
    const uint16_t* abase = Af + (int64_t)expert * nksteps * 512;
    const int nstages = (int)((K + RL_KC - 1) / RL_KC);
    auto issue_stage = [&](int t) {
        const uint32_t sbase = lds0 + (t % RL_NSTAGE) * RL_STAGE;
        // lanes past the end of the row (last stage of a K that is not a multiple of RL_KC) re-read its start;
        // the K steps they would feed are skipped below
        const int64_t k = (int64_t)t * RL_KC + (lane & 31) * 8;
        const int64_t koff = (k + 8 <= K) ? k : 0;
#pragma unroll
        for (int q = 0; q < PPW; ++q) {
            const uint32_t dst = sbase + (wave * PPW + q) * RL_PAIRP;
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(dst), "v"(rowptr[q] + koff) : "memory", "m0");
        }
        // this wave's adapter fragment of the stage (a fragment past the end is replaced by fragment 0 and not used)
        int64_t kstep = (int64_t)t * RL_KSTEPS + wave;
        if (kstep >= nksteps) kstep = 0;
        const uint32_t adst = sbase + RL_XBYTES + wave * 1024;
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(adst), "v"(abase + kstep * 512 + lane * 8) : "memory", "m0");
    };
    constexpr int LOADS_PER_STAGE = PPW + 1;

    f32x4_t acc[NBLK];
#pragma unroll
    for (int h = 0; h < NBLK; ++h) acc[h] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
    issue_stage(0);
    if (nstages > 1) issue_stage(1);
    for (int t = 0; t < nstages; ++t) {
        // stage t has landed once at most the loads of stage t+1 are still in flight
        if (t + 1 < nstages) __builtin_amdgcn_s_waitcnt(0x0F70 | LOADS_PER_STAGE);
        else __builtin_amdgcn_s_waitcnt(0x0F70);
        __syncthreads();                      // ... for every wave; and stage t-1 has been consumed by all waves
        if (t + 2 < nstages) issue_stage(t + 2);
        const uint8_t* st = smem + (t % RL_NSTAGE) * RL_STAGE;
        const int64_t kstep = (int64_t)t * RL_KSTEPS + wave;
        if (kstep < nksteps) {
            const bf16x8_t a = *(const bf16x8_t*)(st + RL_XBYTES + wave * 1024 + lane * 16);
            // row r of the tile: pair r/2, half r%2; this wave's K step starts at byte wave*64 of the row's 512
#pragma unroll
            for (int h = 0; h < NBLK; ++h) {
                const bf16x8_t x = *(const bf16x8_t*)(st + (h * 8 + (i >> 1)) * RL_PAIRP + (i & 1) * (RL_KC * 2) + wave * 64 + g * 16);
                acc[h] = Num::mfma(x, a, acc[h]);
            }
        }
    }
    __syncthreads();   // all fragment reads done: the stage buffers become the reduction buffer
    float (*red)[ROWS][16] = (float (*)[ROWS][16])smem;
    // acc[h][r] = element (row = h*16 + g*4 + r, col = i)
#pragma unroll
    for (int h = 0; h < NBLK; ++h)
#pragma unroll
        for (int r = 0; r < 4; ++r) red[wave][h * 16 + g * 4 + r][i] = acc[h][r];
    __syncthreads();
    for (int t = threadIdx.x; t < ROWS * 16; t += RL_THREADS) {
        const int row = t >> 4, col = t & 15;
        const int64_t mo = row0 + row;
        if (mo < row1) {
            float v = 0.f;
#pragma unroll
            for (int w = 0; w < RL_WAVES; ++w) v += red[w][row][col];
            v *= scaling;
            Q[mo * 16 + col] = Num::from_f32(v);
            const float vs = qt_row_scale ? v * qt_row_scale[mo] : v;
            if (Qt) Qt[(int64_t)col * ldqt + mo] = Num::from_f32(vs);
            if (job.Qs) job.Qs[mo * 16 + col] = Num::from_f32(vs);
        }
    }
}

// ---------------------------------------------------------------------------------------------------------
constexpr int XTP_THREADS = 256;
constexpr int XTP_RC = 256;    // rows per partial
constexpr int XTP_WCOLS = 128; // columns per wave (16 lanes x 8)
constexpr int XTP_COLS = 4 * XTP_WCOLS;  // columns per workgroup

// partial[tile][k][16] (fp32) = sum over the tile's rows of X[m][k] * P[m][r].
// MFMA 16x16x32: the contraction runs over 32 rows; a lane owns 8 consecutive columns of X for 8 rows
// (8 x 16-byte loads) and transposes them in registers into 8 column fragments; the P fragment is one 16-byte
// load from the transposed copy Pt.  Each wave owns 128 columns and walks the tile's rows 32 at a time with the
// next block's loads in flight, so there is no cross-wave reduction.
// one or two jobs per launch (see unit_and_job): same rows and shapes, different operands / outputs; job j's partials start
// at partial + j * partial_stride
struct XtpJob { const uint16_t* X; const uint16_t* Pt; uint16_t* out; int64_t soe, sok, sor; int rank; };   // rank: columns written (<= 16)
template <typename Num>
__global__ void __launch_bounds__(XTP_THREADS) xtp_partial_kernel(const XtpJob job0, const XtpJob job1, int64_t ldx,
                                                                  const void* __restrict__ pos, int pos64, int fan_out,
                                                                  int64_t ldpt,
                                                                  const float* __restrict__ p_row_scale,
                                                                  float* __restrict__ partial, int64_t partial_stride,
                                                                  const void* __restrict__ offsets, int off64, int E,
                                                                  int64_t R, int64_t K, int njobs)
{
    // unit = (row tile, column block), column block fastest
    int64_t unit;
    int job_id;
    unit_and_job(njobs, &unit, &job_id);
    const int64_t kblocks = (K + XTP_COLS - 1) / XTP_COLS;
    const int64_t tile_id = unit / kblocks, kblock = unit % kblocks;
    const XtpJob& job = job_id ? job1 : job0;
    const uint16_t* __restrict__ X = job.X;
    const uint16_t* __restrict__ Pt = job.Pt;
    partial += (int64_t)job_id * partial_stride;
    RowTile rt;
    if (!find_row_tile(offsets, off64, E, XTP_RC, tile_id, &rt)) return;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int i = lane & 15, g = lane >> 4;
    const int64_t kcol = kblock * XTP_COLS + wave * XTP_WCOLS + 8 * i;
    const bool col_ok = kcol < K;  // K % 8 == 0: a lane's 8 columns are all in or all out
    f32x4_t acc[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
    // 32-row blocks on absolute multiples of 32 so that the Pt loads are 16-byte aligned; rows outside the tile
    // are cancelled by zeroing their P values
    const int64_t b0 = rt.row0 / 32, b1 = (rt.row1 + 31) / 32;
    // source row and P scale of every row the blocks touch, fetched once: the row gather would otherwise put a
    // dependent index load in front of every block's X loads
    __shared__ int64_t s_src[XTP_RC + 64];
    __shared__ float s_scale[XTP_RC + 64];
    for (int t = threadIdx.x; t < (int)(b1 - b0) * 32; t += XTP_THREADS) {
        int64_t m = b0 * 32 + t;
        const bool inside = m >= rt.row0 && m < rt.row1;
        if (m >= R) m = R - 1;
        s_scale[t] = !inside ? 0.f : (p_row_scale ? p_row_scale[m] : 1.f);
        s_src[t] = pos ? load_idx(pos, m, pos64) / fan_out : m;
    }
    __syncthreads();
    auto load_block = [&](int64_t b, uint4* dst) {
        const int t0 = (int)(b - b0) * 32 + 8 * g;
#pragma unroll
        for (int rr = 0; rr < 8; ++rr)
            dst[rr] = col_ok ? *(const uint4*)(X + s_src[t0 + rr] * ldx + kcol) : make_uint4(0, 0, 0, 0);
    };
    auto process = [&](int64_t b, const uint4* src) {
        const int64_t mbase = b * 32 + 8 * g;
        union { bf16x8_t v; uint16_t h[8]; } pb;
        pb.v = *(const bf16x8_t*)(Pt + (int64_t)i * ldpt + mbase);
        const int t0 = (int)(b - b0) * 32 + 8 * g;
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            const float sc = s_scale[t0 + t];   // 0 outside the tile (where Pt may hold anything)
            if (sc == 0.f) pb.h[t] = 0;
            else if (sc != 1.f) pb.h[t] = Num::from_f32(Num::to_f32(pb.h[t]) * sc);
        }
        uint32_t w[8][4];   // w[rr][c]: row rr, column pair c
#pragma unroll
        for (int rr = 0; rr < 8; ++rr) { w[rr][0] = src[rr].x; w[rr][1] = src[rr].y; w[rr][2] = src[rr].z; w[rr][3] = src[rr].w; }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            union { bf16x8_t v; uint32_t u[4]; } a;
#pragma unroll
            for (int qd = 0; qd < 4; ++qd) {
                const uint32_t lo = w[2 * qd][j >> 1], hi = w[2 * qd + 1][j >> 1];
                a.u[qd] = (j & 1) ? ((lo >> 16) | (hi & 0xffff0000u)) : ((lo & 0xffffu) | (hi << 16));
            }
            acc[j] = Num::mfma(a.v, pb.v, acc[j]);
        }
    };
    uint4 in0[8], in1[8];
    if (b0 < b1) load_block(b0, in0);
    for (int64_t b = b0; b < b1; b += 2) {
        if (b + 1 < b1) load_block(b + 1, in1);
        process(b, in0);
        if (b + 1 < b1) {
            if (b + 2 < b1) load_block(b + 2, in0);
            process(b + 1, in1);
        }
    }
    // acc[j][reg]: X column kcol0 + 8*(g*4 + reg) + j (MFMA row g*4+reg), P column i
    float* out = partial + (tile_id * K + kblock * XTP_COLS + wave * XTP_WCOLS) * 16;
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
        for (int reg = 0; reg < 4; ++reg) {
            const int c = 8 * (g * 4 + reg) + j;
            if (kblock * XTP_COLS + wave * XTP_WCOLS + c < K) out[c * 16 + i] = acc[j][reg];
        }
}

// out[e][k][r] = scale * sum over the expert's partial tiles (ascending), zero for an empty expert.  A thread owns four
// consecutive rank columns of one k (one 16-byte load per tile, several tiles in flight).
template <typename Num>
__global__ void xtp_reduce_kernel(const float* __restrict__ partial, int64_t partial_stride, const XtpJob job0,
                                  const XtpJob job1, const void* __restrict__ offsets, int off64,
                                  int E, int64_t K, float scale)
{
    const XtpJob& job = blockIdx.z ? job1 : job0;
    uint16_t* __restrict__ out = job.out;
    const int64_t soe = job.soe, sok = job.sok, sor = job.sor;
    const int rank = job.rank;
    partial += (int64_t)blockIdx.z * partial_stride;
    const int e = blockIdx.y;
    int64_t tile0 = 0, start = 0, end = 0;
    for (int ee = 0; ee <= e; ++ee) {
        start = end;
        end = load_idx(offsets, ee, off64);
        if (ee < e) tile0 += (end - start + XTP_RC - 1) / XTP_RC;
    }
    const int64_t ntile = (end - start + XTP_RC - 1) / XTP_RC;
    const int64_t idx = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (idx >= K * 16) return;
    const int64_t k = idx >> 4;
    const int r = (int)(idx & 15);
    const float* __restrict__ src = partial + tile0 * K * 16 + idx;
    f32x4_t s = (f32x4_t){0.f, 0.f, 0.f, 0.f};
    int64_t t = 0;
    for (; t + 4 <= ntile; t += 4) {   // four loads in flight; the additions keep the ascending order
        const f32x4_t a = *(const f32x4_t*)(src + (t + 0) * K * 16), b = *(const f32x4_t*)(src + (t + 1) * K * 16);
        const f32x4_t c = *(const f32x4_t*)(src + (t + 2) * K * 16), d = *(const f32x4_t*)(src + (t + 3) * K * 16);
#pragma unroll
        for (int q = 0; q < 4; ++q) s[q] = (((s[q] + a[q]) + b[q]) + c[q]) + d[q];
    }
    for (; t < ntile; ++t) {
        const f32x4_t a = *(const f32x4_t*)(src + t * K * 16);
#pragma unroll
        for (int q = 0; q < 4; ++q) s[q] += a[q];
    }
#pragma unroll
    for (int q = 0; q < 4; ++q)
        if (r + q < rank) out[(int64_t)e * soe + k * sok + (r + q) * sor] = Num::from_f32(s[q] * scale);
}

// Q[m][r] = bf16(scaling * sum_t partial[t][m][r]) (t ascending: a fixed order) and Qt[r][m] likewise.  A thread owns
// four consecutive rank columns of one row and keeps eight loads in flight.
template <typename Num>
__global__ void cc_reduce_kernel(const float* __restrict__ partial0, const float* __restrict__ partial1, int ntiles, int64_t R,
                                 float scaling, uint16_t* __restrict__ Q0, uint16_t* __restrict__ Q1, uint16_t* __restrict__ Qt0,
                                 uint16_t* __restrict__ Qt1, int64_t ldqt)
{
    const float* __restrict__ partial = blockIdx.y ? partial1 : partial0;
    uint16_t* __restrict__ Q = blockIdx.y ? Q1 : Q0;
    uint16_t* __restrict__ Qt = blockIdx.y ? Qt1 : Qt0;
    const int64_t idx = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;   // (m, r) flattened, r a multiple of 4
    if (idx >= R * 16) return;
    const float* __restrict__ src = partial + idx;
    const int64_t step = R * 16;
    f32x4_t s = (f32x4_t){0.f, 0.f, 0.f, 0.f};
    int t = 0;
    for (; t + 8 <= ntiles; t += 8) {
        f32x4_t v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = *(const f32x4_t*)(src + (int64_t)(t + u) * step);
#pragma unroll
        for (int u = 0; u < 8; ++u)
#pragma unroll
            for (int q = 0; q < 4; ++q) s[q] += v[u][q];
    }
    for (; t < ntiles; ++t) {
        const f32x4_t a = *(const f32x4_t*)(src + (int64_t)t * step);
#pragma unroll
        for (int q = 0; q < 4; ++q) s[q] += a[q];
    }
    uint16_t o[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) o[q] = Num::from_f32(s[q] * scaling);
    *(uint2*)(Q + idx) = make_uint2(o[0] | ((uint32_t)o[1] << 16), o[2] | ((uint32_t)o[3] << 16));
    if (Qt) {
        const int64_t m = idx >> 4;
        const int r = (int)(idx & 15);
#pragma unroll
        for (int q = 0; q < 4; ++q) Qt[(int64_t)(r + q) * ldqt + m] = o[q];
    }
}

}  // namespace

int moe_launch_cc_reduce2(const float* partial, const float* partial2, int ntiles, int64_t R, float scaling, void* Q, void* Q2,
                          void* Qt, void* Qt2, int64_t ldqt, hipStream_t stream, int f16)
{
    if (R == 0) return MOE_OK;
    const bool two = partial2 != nullptr;
    hipLaunchKernelGGL(f16 ? cc_reduce_kernel<NumF16> : cc_reduce_kernel<NumBf16>, dim3((unsigned)((R * 4 + 255) / 256), two ? 2u : 1u), dim3(256), 0, stream, partial, partial2,
                       ntiles, R, scaling, (uint16_t*)Q, (uint16_t*)Q2, (uint16_t*)Qt, (uint16_t*)Qt2, ldqt);
    return moe_launch_status();
}

int moe_launch_pack_lora(const void* src, int64_t se, int64_t sk, int64_t sr, void* dst, int E, int64_t K, int rank,
                         int transpose, hipStream_t stream)
{
    if (rank < 1 || rank > 16) return MOE_ERR_UNSUPPORTED;
    const int64_t Kimg = transpose ? (K + 31) / 32 * 32 : K;
    const int64_t total = (int64_t)E * Kimg * 16;
    if (total == 0) return MOE_OK;
    hipLaunchKernelGGL(pack_lora_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream,
                       (const uint16_t*)src, se, sk, sr, (uint16_t*)dst, K, Kimg, rank, transpose, total);
    return moe_launch_status();
}

int moe_launch_pack_lora_batch(const MoePackBatch& jobs, hipStream_t stream)
{
    if (jobs.njobs < 1 || jobs.njobs > MOE_PACK_MAX_JOBS) return MOE_ERR_UNSUPPORTED;
    for (int j = 0; j < jobs.njobs; ++j)
        if (jobs.job[j].rank < 1 || jobs.job[j].rank > 16) return MOE_ERR_UNSUPPORTED;
    int64_t kmax = 0;
    for (int j = 0; j < jobs.njobs; ++j) kmax = jobs.job[j].K > kmax ? jobs.job[j].K : kmax;
    const int64_t total = (int64_t)jobs.E * kmax * 2;   // 16-byte chunks of the largest job
    if (total == 0 && jobs.zero_n == 0) return MOE_OK;
    if (total > 0x7fffffff || jobs.zero_n < 0 || (jobs.zero_n > 0 && !jobs.zero_ptr)) return MOE_ERR_UNSUPPORTED;
    for (int j = 0; j < jobs.njobs; ++j)
        if (((uintptr_t)jobs.job[j].dst % 16) != 0 || (jobs.job[j].transpose && jobs.job[j].K % 32 != 0)) return MOE_ERR_UNSUPPORTED;
    const unsigned gx = (unsigned)((total + 255) / 256);
    hipLaunchKernelGGL(pack_lora_batch_kernel, dim3(gx ? gx : 1u, (unsigned)jobs.njobs), dim3(256), 0, stream, jobs);
    return moe_launch_status();
}

int moe_launch_rows_lora2(const void* X, const void* X2, int64_t ldx, const void* At, const void* At2, void* Q, void* Q2,
                          void* Qt, void* Qt2, int64_t ldqt, const void* pos, int pos64, const void* offsets, int off64,
                          int E, int64_t R, int64_t K, int fan_out, int x_grouped, float scaling,
                          const float* qt_row_scale, hipStream_t stream, void* q_scaled, int f16)
{
    if (R == 0) return MOE_OK;
    const bool two = X2 != nullptr;
    if (K % 8 != 0 || ldx % 8 != 0 || ((uintptr_t)X % 16) != 0 || ((uintptr_t)At % 16) != 0 ||
        (two && (((uintptr_t)X2 % 16) != 0 || ((uintptr_t)At2 % 16) != 0)))
        return MOE_ERR_UNSUPPORTED;
    static std::atomic<bool> attr_set[MOE_MAX_DEVICES];   // per device; forward and backward may call from different host threads
    const int dev = moe_current_device();
    if (!attr_set[dev]) {
        if (hipFuncSetAttribute((const void*)rows_lora_kernel<32, NumBf16>, hipFuncAttributeMaxDynamicSharedMemorySize, rl_lds(32)) != hipSuccess ||
            hipFuncSetAttribute((const void*)rows_lora_kernel<16, NumBf16>, hipFuncAttributeMaxDynamicSharedMemorySize, rl_lds(16)) != hipSuccess ||
            hipFuncSetAttribute((const void*)rows_lora_kernel<32, NumF16>, hipFuncAttributeMaxDynamicSharedMemorySize, rl_lds(32)) != hipSuccess ||
            hipFuncSetAttribute((const void*)rows_lora_kernel<16, NumF16>, hipFuncAttributeMaxDynamicSharedMemorySize, rl_lds(16)) != hipSuccess)
            return MOE_ERR_LAUNCH;
        attr_set[dev] = true;
    }
    const RowsLoraJob j0 = {(const uint16_t*)X, (const uint16_t*)At, (uint16_t*)Q, (uint16_t*)Qt, (uint16_t*)q_scaled};
    const RowsLoraJob j1 = {(const uint16_t*)X2, (const uint16_t*)At2, (uint16_t*)Q2, (uint16_t*)Qt2, nullptr};
    // 32-row tiles halve the adapter traffic, but two workgroups fit a compute unit: use them when the launch has
    // about that many, otherwise 16-row tiles (three fit)
    if ((R / 16 + E) * 2 + 16 >= ((int64_t)1 << 31)) return MOE_ERR_UNSUPPORTED;   // workgroups of the launch, as a 32-bit grid size
    const int cus = moe_device_cus();
    const int64_t tiles32 = (R / 32 + E) * (two ? 2 : 1);
    if (tiles32 >= 3 * (int64_t)cus / 2) {
        hipLaunchKernelGGL((f16 ? rows_lora_kernel<32, NumF16> : rows_lora_kernel<32, NumBf16>), dim3(job_grid(R / 32 + E, two ? 2 : 1)), dim3(RL_THREADS), rl_lds(32), stream, j0, j1,
                           ldx, ldqt, pos, pos64, offsets, off64, E, K, fan_out, x_grouped, scaling, qt_row_scale, two ? 2 : 1);
    } else {
        hipLaunchKernelGGL((f16 ? rows_lora_kernel<16, NumF16> : rows_lora_kernel<16, NumBf16>), dim3(job_grid(R / 16 + E, two ? 2 : 1)), dim3(RL_THREADS), rl_lds(16), stream, j0, j1,
                           ldx, ldqt, pos, pos64, offsets, off64, E, K, fan_out, x_grouped, scaling, qt_row_scale, two ? 2 : 1);
    }
    return moe_launch_status();
}

int moe_launch_rows_lora(const void* X, int64_t ldx, const void* At, void* Q, void* Qt, int64_t ldqt, const void* pos,
                         int pos64, const void* offsets, int off64, int E, int64_t R, int64_t K, int fan_out,
                         int x_grouped, float scaling, const float* qt_row_scale, hipStream_t stream, int f16)
{
    return moe_launch_rows_lora2(X, nullptr, ldx, At, nullptr, Q, nullptr, Qt, nullptr, ldqt, pos, pos64, offsets, off64, E, R,
                                 K, fan_out, x_grouped, scaling, qt_row_scale, stream, nullptr, f16);
}

size_t moe_xtp_workspace_bytes(int64_t R, int E, int64_t K)
{
    return (size_t)(R / XTP_RC + E) * (size_t)K * 16 * sizeof(float);
}

int moe_launch_xtp2(const void* X, const void* X2, int64_t ldx, const void* pos, int pos64, int fan_out, const void* Pt,
                    const void* Pt2, int64_t ldpt, const float* p_row_scale, void* out, void* out2, const int64_t* so,
                    const int64_t* so2, int rank, int rank2, const void* offsets, int off64, int E, int64_t R, int64_t K,
                    float scale, void* workspace, size_t workspace_bytes, hipStream_t stream, int f16)
{
    if (E == 0 || K == 0) return MOE_OK;
    const bool two = X2 != nullptr;
    if (rank < 1 || rank > 16 || (two && (rank2 < 1 || rank2 > 16))) return MOE_ERR_UNSUPPORTED;
    if (K % 8 != 0 || ldx % 8 != 0 || ldpt % 16 != 0 || ldpt < (R + 31) / 32 * 32 || ((uintptr_t)X % 16) != 0 ||
        ((uintptr_t)Pt % 16) != 0 || (two && (((uintptr_t)X2 % 16) != 0 || ((uintptr_t)Pt2 % 16) != 0)))
        return MOE_ERR_UNSUPPORTED;
    const size_t one = moe_xtp_workspace_bytes(R, E, K);
    if (workspace_bytes < one * (two ? 2 : 1)) return MOE_ERR_WORKSPACE;
    const int64_t tiles = R / XTP_RC + E;
    const XtpJob j0 = {(const uint16_t*)X, (const uint16_t*)Pt, (uint16_t*)out, so[0], so[1], so[2], rank};
    const XtpJob j1 = two ? XtpJob{(const uint16_t*)X2, (const uint16_t*)Pt2, (uint16_t*)out2, so2[0], so2[1], so2[2], rank2} : j0;
    const int64_t pstride = (int64_t)(one / sizeof(float));
    if (R > 0) {
        const int64_t units = ((K + XTP_COLS - 1) / XTP_COLS) * tiles;
        if (units * 2 + 16 >= ((int64_t)1 << 31)) return MOE_ERR_UNSUPPORTED;
        hipLaunchKernelGGL(f16 ? xtp_partial_kernel<NumF16> : xtp_partial_kernel<NumBf16>, dim3(job_grid(units, two ? 2 : 1)), dim3(XTP_THREADS), 0, stream, j0, j1, ldx, pos, pos64, fan_out, ldpt,
                           p_row_scale, (float*)workspace, pstride, offsets, off64, E, R, K, two ? 2 : 1);
    }
    dim3 rgrid((unsigned)((K * 4 + 255) / 256), (unsigned)E, two ? 2u : 1u);
    hipLaunchKernelGGL(f16 ? xtp_reduce_kernel<NumF16> : xtp_reduce_kernel<NumBf16>, rgrid, dim3(256), 0, stream, (const float*)workspace, pstride, j0, j1, offsets,
                       off64, E, K, scale);
    return moe_launch_status();
}

int moe_launch_xtp_reduce2(const float* partial, const float* partial2, void* out, void* out2, const int64_t* so,
                           const int64_t* so2, int rank, int rank2, const void* offsets, int off64, int E, int64_t K,
                           float scale, hipStream_t stream, int f16)
{
    if (E == 0 || K == 0) return MOE_OK;
    const bool two = partial2 != nullptr;
    if (rank < 1 || rank > 16 || (two && (rank2 < 1 || rank2 > 16))) return MOE_ERR_UNSUPPORTED;
    const XtpJob j0 = {nullptr, nullptr, (uint16_t*)out, so[0], so[1], so[2], rank};
    const XtpJob j1 = two ? XtpJob{nullptr, nullptr, (uint16_t*)out2, so2[0], so2[1], so2[2], rank2} : j0;
    dim3 rgrid((unsigned)((K * 4 + 255) / 256), (unsigned)E, two ? 2u : 1u);
    hipLaunchKernelGGL(f16 ? xtp_reduce_kernel<NumF16> : xtp_reduce_kernel<NumBf16>, rgrid, dim3(256), 0, stream, partial, two ? (int64_t)(partial2 - partial) : 0, j0, j1,
                       offsets, off64, E, K, scale);
    return moe_launch_status();
}

int moe_launch_xtp(const void* X, int64_t ldx, const void* pos, int pos64, int fan_out, const void* Pt, int64_t ldpt,
                   const float* p_row_scale, void* out, int64_t soe, int64_t sok, int64_t sor, int rank,
                   const void* offsets, int off64, int E, int64_t R, int64_t K, float scale, void* workspace,
                   size_t workspace_bytes, hipStream_t stream, int f16)
{
    const int64_t so[3] = {soe, sok, sor};
    return moe_launch_xtp2(X, nullptr, ldx, pos, pos64, fan_out, Pt, nullptr, ldpt, p_row_scale, out, nullptr, so, nullptr, rank,
                           0, offsets, off64, E, R, K, scale, workspace, workspace_bytes, stream, f16);
}
