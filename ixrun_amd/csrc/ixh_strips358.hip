// (3,5,8) fused decode + GEMV for gfx950, strip variant: every lane walks a strip of 128 consecutive weights of one
// row by itself, and the products are taken on the matrix pipe, so that up to 16 activation rows share one decode.
//
// Work split.  A workgroup owns whole rows (a run of row quads), as in ixh_rows358.hip, so the result leaves as bf16
// from one launch with no workspace.  The unit of work is a task: one 512-wide column block x one row quad.  A task
// belongs to one 16-lane DPP row of a wave ("worker"): lane (q, j) of the row, q = strip 0..3 of the column block,
// j = row 0..3 of the quad, decodes the 128 weights of strip q of row j.  The four DPP rows of a wave run four tasks
// side by side; tasks are dealt round-robin to the workers.
//
// Decode.  A lane loads the four words of bitmap 0 that cover its strip straight into registers (16 bytes), counts
// them, and gets the rank of its strip's first element from the unit's table entry and two DPP additions over the
// strips of its unit.  From there it is on its own: for each of its four words it loads the 16 bytes of the 3-bit
// stream that hold the word's codes (address = 3 x rank), aligns them (three v_alignbit), splices the elements that
// are not level 1 out of the 96-bit window (their field becomes the code of 0; they go to the wave's record queue)
// and looks sixteen code pairs up in the LDS table of dequantised pairs.  No scan over the lanes of a row, no staging
// ring, no hand-counted waits.  Three steps run one task apart: table entry + bitmap words, ranks + code requests,
// decode; two register stages take turns.
//
// Products.  v_mfma_f32_4x4x4_16b_bf16: each of the 16 blocks of four lanes multiplies a 4 x 4 tile of activations
// (activation row i in lane i of the block: four rows cost what one costs) with the 4 weights of each of its four
// lanes' rows and adds into four accumulators per lane, which stay with the lane for its whole strip.  More than
// four activation rows (MG = 2 or 4 groups of four) repeat the instruction per group on the same weights.  The
// activations sit in LDS once per workgroup, in strips padded so that the 16 strips a wave reads at a time fall into
// different banks.
//
// Elements above level 1.  The waves' records are resolved together after the main loop: the elements are listed in
// one shared task list (in wave and record order) and taken 64 at a time by the waves in turn, each adding into its
// own row sums, so that every wave's additions and their order are fixed; when the list would overflow (dense mixes)
// every wave resolves its own queue as in ixh_rows358.hip.
//
// Reduction.  Strips over the four q lanes (DPP), tasks into the wave's row sums in LDS (one DPP row after the
// other), waves in wave order after one barrier.  Fixed summation order apart from the order in which the LDS adds
// the lanes of one instruction that hit the same row sum.
#include <math.h>

#include "ixh_rows_common.h"

namespace ixh {

typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kSMaxWaves = 16;
constexpr uint32_t kSQueue = 256;    // records per wave at most (128 where LDS is short)
constexpr uint32_t kSMaxRows = 128;  // rows per workgroup at most
constexpr int kSMaxM = 16;           // activation rows: four per matrix instruction, up to four instructions per step

constexpr size_t kSLdsLimit = 160 * 1024;
constexpr uint32_t kSPool = 2048;  // tasks the workgroup resolves together; more: every wave resolves its own

struct StripsLds {
    uint32_t tq1, tq2, side, xs, xs_row, zero, pool, counts, waves, wave_bytes, rowacc_off, tasks_off, total;
};

__host__ __device__ inline StripsLds strips_layout(uint32_t rows_cap, uint32_t n_chunks, uint32_t n_waves, int m,
                                                   uint32_t qcap) {
    StripsLds L;
    const uint32_t tbl = ((rows_cap * n_chunks + 1u + 3u) & ~3u) * 4u;  // one entry past the slice: its end ranks
    L.tq1 = kRLutBytes + kRSpliceBytes;
    L.tq2 = L.tq1 + tbl;
    L.side = L.tq2 + tbl;
    L.xs = L.side + kRSideBytes;
    // bytes between activation rows: the padded strips, rounded up so that consecutive rows start 8 banks apart
    L.xs_row = ((n_chunks * 4u * kStripBytes + 127u) & ~127u) + 32u;
    L.zero = L.xs + (uint32_t)m * L.xs_row;  // a strip of zeros: what the lanes of absent activation rows read
    L.pool = (L.zero + kStripBytes + 15u) & ~15u;  // the shared task list, then one task count per wave
    L.counts = L.pool + kSPool * 4u;
    L.waves = L.counts + kSMaxWaves * 4u;
    L.rowacc_off = qcap * 16u;  // behind the queue: [rows_cap][m activation rows] fp32
    L.tasks_off = (L.rowacc_off + rows_cap * (uint32_t)m * 4u + 15u) & ~15u;
    L.wave_bytes = (L.tasks_off + kRTasks * 2u + 15u) & ~15u;
    L.total = L.waves + n_waves * L.wave_bytes;
    return L;
}

// waves a workgroup may have with MG groups of four activation rows: what leaves its lanes the registers they need
__host__ __device__ constexpr int strips_max_waves(int mg) { return mg <= 1 ? kSMaxWaves : 12; }

// MG: groups of four activation rows (1, 2 or 4): every step of four columns is multiplied with each of them
template <int MG, bool ANY>
__global__ void __launch_bounds__(strips_max_waves(MG) * kWave)
k_gemv358_strips(Dev P, const int32_t *__restrict__ prefix, uint32_t n_chunks, uint32_t quads_per_wg, uint32_t qcap,
                 uint32_t flags,
                 const uint16_t *__restrict__ x, int m, int64_t ldx, uint16_t *__restrict__ y, int64_t ldy,
                 float *__restrict__ y32) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    constexpr int R = 1;        // chains per lane
    constexpr int MT = 4 * MG;  // activation rows at most

    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const uint32_t n_waves = blockDim.x >> 6;
    const uint32_t drow = lane >> 4, q = (lane >> 2) & 3u, j = lane & 3u;

    const uint32_t n_quads = P.out_f >> 2;  // out_f is a multiple of four here
    const uint32_t quad0 = blockIdx.x * quads_per_wg;
    const uint32_t n_q = min(quads_per_wg, n_quads - quad0);
    const uint32_t row0 = quad0 * 4, rows_here = n_q * 4, rows_cap = quads_per_wg * 4;
    const StripsLds L = strips_layout(rows_cap, n_chunks, n_waves, m, qcap);

    // the pair table is addressed with (index bits | lane bits): it must sit at LDS address 0
    if ((uint32_t)(uintptr_t)(lds_ptr_t)smem != 0) {
        for (uint32_t t = tid; t < rows_here * (uint32_t)m; t += blockDim.x) {
            if (y32) y32[(size_t)(t % m) * P.out_f + row0 + t / m] = __uint_as_float(0x7FC00000u);  // NaN
            else y[(int64_t)(t % m) * ldy + row0 + t / m] = 0x7FC0;
        }
        return;
    }
    uint32_t *const lut = reinterpret_cast<uint32_t *>(smem);            // [64][32]
    uint4 *const splice = reinterpret_cast<uint4 *>(smem + kRLutBytes);  // [33][2]
    uint32_t *const tq1 = reinterpret_cast<uint32_t *>(smem + L.tq1);
    uint32_t *const tq2 = reinterpret_cast<uint32_t *>(smem + L.tq2);
    uint8_t *const wave_base = smem + L.waves + wave * L.wave_bytes;
    uint4 *const queue = reinterpret_cast<uint4 *>(wave_base);
    float *const rowacc = reinterpret_cast<float *>(wave_base + L.rowacc_off);
    uint16_t *const tasks = reinterpret_cast<uint16_t *>(wave_base + L.tasks_off);

    const uint32_t unit0 = row0 * n_chunks;
    const uint32_t entries = P.out_f * n_chunks + 1;
    const uint32_t n_local = rows_here * n_chunks;

    const __amdgpu_buffer_rsrc_t b1_rsrc =
        __builtin_amdgcn_make_buffer_rsrc((void *)P.bm[0], 0, (int)(P.bm_words[0] * 4u), 0x00020000);
    const __amdgpu_buffer_rsrc_t l1_rsrc =
        __builtin_amdgcn_make_buffer_rsrc((void *)P.st[0], 0, (int)(P.st_words[0] * 4u), 0x00020000);
    const __amdgpu_buffer_rsrc_t tb_rsrc =
        __builtin_amdgcn_make_buffer_rsrc((void *)prefix, 0, (int)(entries * 4u), 0x00020000);

    // ---- tasks: t = column block + n_chunks * group; worker = one DPP row of one wave ----
    const uint32_t n_groups = (n_q + R - 1) / R;
    const uint32_t n_tasks = n_chunks * n_groups;
    const uint32_t n_workers = n_waves * 4;
    const uint32_t worker = wave * 4 + drow;
    const uint32_t wave_iters = wave * 4 < n_tasks ? (n_tasks - wave * 4 + n_workers - 1) / n_workers : 0u;
    const bool quads_fastest = m > 4 && n_groups >= 4;

    // what a lane needs for one task: requested first, so that it travels while the workgroup sets up
    struct TaskIn {
        bool valid;       // the DPP row has a task
        uint32_t col;     // first column of the lane's strip
        uint32_t strip;   // strip index in the activation rows
        uint32_t lrow[R];  // local row of chain r (clamped)
        bool live[R];      // chain r has a row
        uint32_t q1u[R];   // rank table entry of the chain's unit
        u32x4 bm[R];       // the four bitmap words of the lane's strip
    };
    auto request = [&](uint32_t it, TaskIn &T) {
        const uint32_t t = worker + it * n_workers;
        T.valid = t < n_tasks;
        const uint32_t tt = T.valid ? t : 0u;
        // Column blocks run fastest for up to four activation rows: the wave's four tasks then read neighbouring
        // pieces of the same rows (fewer cache lines per load).  Beyond that row quads run fastest: the four tasks are
        // four different row quads, their row sums never meet in one LDS addition, and what that saves per
        // activation row is worth more.
        uint32_t g, c;
        if (quads_fastest) {
            c = tt / n_groups;
            g = tt - c * n_groups;
        } else {
            g = tt / n_chunks;
            c = tt - g * n_chunks;
        }
        T.col = c * kFastChunk + q * 128u;
        T.strip = c * 4u + q;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const uint32_t quad = g * R + r;
            T.live[r] = T.valid && quad < n_q;
            T.lrow[r] = min(quad, n_q - 1) * 4u + j;
            const uint32_t unit_l = T.lrow[r] * n_chunks + c;
            T.q1u[r] = __builtin_amdgcn_raw_buffer_load_b32(tb_rsrc, (int)((unit0 + unit_l) * 4u), 0, 0);
            T.bm[r] = __builtin_amdgcn_raw_buffer_load_b128(
                b1_rsrc, (int)((((row0 + T.lrow[r]) * P.in_f + T.col) >> 5) * 4u), 0, 0);
        }
    };

    TaskIn T;
    if (wave_iters > 0) request(0, T);

    // ---- workgroup set-up: activations, table slices, side streams, pair table, splice masks ----
    {
        // activation rows into padded strips: 16-byte piece p of row i holds columns 8p .. 8p+7
        const uint32_t pieces = P.in_f >> 3;
        for (uint32_t t = tid; t < (uint32_t)m * pieces; t += blockDim.x) {
            const uint32_t i = t / pieces, p = t - i * pieces;
            const uint4 v = *reinterpret_cast<const uint4 *>(x + (int64_t)i * ldx + p * 8u);
            uint2 *dst = reinterpret_cast<uint2 *>(smem + L.xs + i * L.xs_row + (p >> 4) * kStripBytes + (p & 15u) * 16u);
            dst[0] = make_uint2(v.x, v.y);
            dst[1] = make_uint2(v.z, v.w);
        }
        for (uint32_t t = tid; t < kStripBytes / 4; t += blockDim.x) reinterpret_cast<uint32_t *>(smem + L.zero)[t] = 0u;
    }
    for (uint32_t i = tid; i <= n_local; i += blockDim.x) {
        tq1[i] = (uint32_t)prefix[unit0 + i];
        if (!ANY) tq2[i] = (uint32_t)prefix[entries + unit0 + i];
    }
    // this workgroup's share of bitmap 1 and of the 5-bit / 8-bit streams: small when few elements are above level 1,
    // then it is staged in LDS and resolving them touches no global memory
    constexpr uint32_t kSideRegs = 4;  // side-stream words a thread carries: 1024 words, at least 4 waves
    uint32_t side_reg[kSideRegs] = {0, 0, 0, 0};
    SideView sv;
    sv.staged = false;
    sv.base = L.side;
    sv.b2w0 = sv.l2w0 = sv.l3w0 = 0;
    if (!ANY) {
        const uint32_t q1b = (uint32_t)prefix[unit0], q2b = (uint32_t)prefix[entries + unit0];
        const uint32_t q1e = (uint32_t)prefix[unit0 + n_local], q2e = (uint32_t)prefix[entries + unit0 + n_local];
        const uint32_t nl1b = row0 * P.in_f - q1b, nl1e = (row0 + rows_here) * P.in_f - q1e;
        sv.b2w0 = nl1b >> 5;
        sv.l2w0 = (uint32_t)(((uint64_t)q2b * 5u) >> 5);
        sv.l3w0 = (nl1b - q2b) >> 2;
        const uint32_t n_b2 = ((nl1e + 31) >> 5) - sv.b2w0;
        const uint32_t n_l2 = (uint32_t)((((uint64_t)q2e * 5u) + 31) >> 5) - sv.l2w0;
        const uint32_t n_l3 = ((nl1e - q2e + 3) >> 2) - sv.l3w0;
        // one word of slack each: the resolver reads the word after a code's first word unconditionally
        sv.staged = (flags & kFlagStageSide) && n_b2 < 256 && n_l2 < 511 && n_l3 <= 256 &&
                    blockDim.x * kSideRegs >= kRSideBytes / 4;
        if (sv.staged) {  // asked for now, put into LDS after the main loop: nothing before that waits for them
            const uint32_t *last32 = reinterpret_cast<const uint32_t *>(P.last);
            const uint32_t last_words = (P.last_bytes + 3u) >> 2;  // whole dwords (allocations are 256-byte granular)
#pragma unroll
            for (uint32_t n = 0; n < kSideRegs; ++n) {
                const uint32_t t = tid + n * blockDim.x;
                uint32_t v = 0;
                if (t < 256) {
                    const uint32_t w = sv.b2w0 + t;
                    if (w < P.bm_words[1]) v = P.bm[1][w];
                } else if (t < 768) {
                    const uint32_t w = sv.l2w0 + (t - 256);
                    if (w < P.st_words[1]) v = P.st[1][w];
                } else if (t < kRSideBytes / 4) {
                    const uint32_t w = sv.l3w0 + (t - 768);
                    if (w < last_words) v = last32[w];
                }
                side_reg[n] = v;
            }
        }
    }
    const float scale = bf16_bits_to_f32(*P.scale);
    for (uint32_t i = tid; i < 64 * 32; i += blockDim.x) {
        const int c0 = (i >> 5) & 7, c1 = i >> 8;
        const uint32_t w0 = c0 < 7 ? f32_to_bf16_bits((float)(c0 - 3) * scale) : 0u;
        const uint32_t w1 = c1 < 7 ? f32_to_bf16_bits((float)(c1 - 3) * scale) : 0u;
        lut[i] = w0 | (w1 << 16);
    }
    if (tid <= 32) {
        // entry e < 32: masks for a zero at element e (code bits 3e..3e+2): the bits below it, and its field;
        // entry 32: the identity (nothing to splice)
        const uint32_t pos = 3 * tid;
        uint32_t lm[3], f[3];
#pragma unroll
        for (int dd = 0; dd < 3; ++dd) {
            const uint32_t base = 32u * dd;
            lm[dd] = pos <= base ? 0u : (pos >= base + 32 ? ~0u : (1u << (pos - base)) - 1u);
            f[dd] = (pos + 3 <= base || pos >= base + 32) ? 0u : (pos >= base ? 7u << (pos - base) : 7u >> (base - pos));
        }
        splice[2 * tid] = make_uint4(lm[0], lm[1], lm[2], 0u);
        splice[2 * tid + 1] = make_uint4(f[0], f[1], f[2], 0u);
    }
    for (uint32_t t = lane; t < rows_cap * (uint32_t)m; t += kWave) rowacc[t] = 0.0f;

    const uint32_t lut_lane = (lane & 31u) << 2;
    const uint32_t splice_addr = kRLutBytes;
    const uint32_t tq1_addr = L.tq1, tq2_addr = L.tq2;
    const uint32_t rowacc_addr = (uint32_t)(uintptr_t)(lds_ptr_t)rowacc;
    const uint32_t xs_addr = L.xs;
    // where this lane's activation row sits (lane j of a block feeds activation row j; absent rows read zeros)
    uint32_t x_lane[MG];
    bool x_real[MG];
#pragma unroll
    for (int g = 0; g < MG; ++g) {
        x_real[g] = 4u * g + j < (uint32_t)m;
        x_lane[g] = x_real[g] ? L.xs + (4u * g + j) * L.xs_row : L.zero;
    }

    uint32_t qcount = 0;  // wave-uniform
    // this wave's own queue, when it fills up or the workgroup's elements do not fit the shared list (dense mixes);
    // from global memory: the staged side streams are not in LDS before the main loop is over
    auto resolve = [&]() {
        if (ANY)
            resolve_rows<MT, false, true, 2>(P, sv, tq1_addr, tq2_addr, unit0, queue, qcount, rowacc_addr, tasks,
                                                xs_addr, L.xs_row, 0, m, scale, lane, prefix, entries);
        else
            resolve_rows<MT, false, false, 2>(P, sv, tq1_addr, tq2_addr, unit0, queue, qcount, rowacc_addr, tasks,
                                                 xs_addr, L.xs_row, 0, m, scale, lane);
        qcount = 0;
    };

    auto splice_once = [&](uint32_t &w0, uint32_t &w1, uint32_t &w2, uint32_t &zrem) {
        const uint32_t e = zrem != 0 ? (uint32_t)__builtin_ctz(zrem) : 32u;
        zrem &= zrem - 1;
        const u32x4 lm = lds_u128(splice_addr + e * 32), fm = lds_u128(splice_addr + e * 32 + 16);
        const uint32_t s0 = w0 << 3;
        const uint32_t s1 = __builtin_amdgcn_alignbit(w1, w0, 29);
        const uint32_t s2 = __builtin_amdgcn_alignbit(w2, w1, 29);
        w0 = (w0 & lm.x) | (s0 & ~lm.x);
        w1 = (w1 & lm.y) | (s1 & ~lm.y);
        w2 = (w2 & lm.z) | (s2 & ~lm.z);
        w0 = (w0 & ~fm.x) | (kZeroCodes0 & fm.x);
        w1 = (w1 & ~fm.y) | (kZeroCodes1 & fm.y);
        w2 = (w2 & ~fm.z) | (kZeroCodes2 & fm.z);
    };

    __syncthreads();

    // A task in flight: the ranks at which its words start and the stream bytes asked for with them.
    struct Stage {
        uint32_t word[R][4];  // bitmap words
        uint32_t rank[R][4];  // level-1 elements before each word (global rank)
        u32x4 code[R][4];     // the 16 stream bytes that hold each word's codes (address = 3 x rank)
        uint32_t col, x_strip[MG], lrow[R];
        bool live[R];
    };
    // second step of a task: from table entry and bitmap words to the ranks, and the requests for the codes
    auto launch_codes = [&](const TaskIn &T, Stage &S) {
        S.col = T.col;
#pragma unroll
        for (int g = 0; g < MG; ++g) S.x_strip[g] = x_lane[g] + (x_real[g] ? T.strip * kStripBytes : 0u);
#pragma unroll
        for (int r = 0; r < R; ++r) {
            u32x4 b = T.bm[r];
            if (!T.live[r]) b = u32x4{~0u, ~0u, ~0u, ~0u};  // a chain without a row decodes what it finds and is dropped
            S.word[r][0] = b.x; S.word[r][1] = b.y; S.word[r][2] = b.z; S.word[r][3] = b.w;
            const uint32_t p1 = __popc(b.x), p2 = p1 + __popc(b.y), p3 = p2 + __popc(b.z), p4 = p3 + __popc(b.w);
            uint32_t incl = p4 + dpp_shr(p4, 4);  // over the strips of the unit: lanes four apart in the DPP row
            incl += dpp_shr(incl, 8);
            const uint32_t first = T.q1u[r] + incl - p4;
            S.rank[r][0] = first; S.rank[r][1] = first + p1; S.rank[r][2] = first + p2; S.rank[r][3] = first + p3;
            S.lrow[r] = T.lrow[r];
            S.live[r] = T.live[r];
#pragma unroll
            for (int k = 0; k < 4; ++k)
                S.code[r][k] = __builtin_amdgcn_raw_buffer_load_b128(l1_rsrc, (int)(((S.rank[r][k] * 3u) >> 5) * 4u), 0, 0);
        }
    };
    // third step: decode and multiply the task's words
    auto compute = [&](Stage &S) {
        f32x4 acc[R][MG];
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int g = 0; g < MG; ++g) acc[r][g] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const u32x4 dq = S.code[r][k];
                const uint32_t rk = S.rank[r][k];
                const uint32_t off = rk * 3u;  // v_alignbit takes the low five bits
                uint32_t w0 = __builtin_amdgcn_alignbit(dq.y, dq.x, off);
                uint32_t w1 = __builtin_amdgcn_alignbit(dq.z, dq.y, off);
                uint32_t w2 = __builtin_amdgcn_alignbit(dq.w, dq.z, off);
                uint32_t zrem = ~S.word[r][k];
                const uint64_t any = __ballot(zrem != 0);
                if (any != 0) {  // lanes with elements above level 1 leave a record
                    if (qcount > qcap - kWave) resolve();
                    if (zrem != 0) {
                        const uint32_t kcol = S.col + 32u * (uint32_t)k;
                        const uint32_t unit = unit0 + S.lrow[r] * n_chunks + (S.col >> 9);
                        const uint32_t r0 = (row0 + S.lrow[r]) * P.in_f + kcol - rk;
                        push_record(queue, qcount + lanes_below(any), make_uint4(zrem, r0, unit, (S.lrow[r] << 16) | kcol));
                    }
                    qcount += (uint32_t)__popcll(any);
                    do splice_once(w0, w1, w2, zrem);
                    while (__ballot(zrem != 0) != 0);
                }
                // sixteen code pairs through the pair table, four weights per matrix instruction; in two halves, so
                // that eight table words and four activation words are held at a time
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    uint32_t wp[8];
#pragma unroll
                    for (int tt = 0; tt < 8; ++tt) {
                        const int t = 8 * h + tt;
                        const int bit = 6 * t, ob = bit & 31, dd = bit >> 5;
                        const uint32_t lo = dd == 0 ? w0 : (dd == 1 ? w1 : w2);
                        const uint32_t hi = dd == 0 ? w1 : w2;
                        uint32_t a;  // pair index at bits 12..7
                        if (ob > 26) a = __builtin_amdgcn_alignbit(hi, lo, ob - 7);
                        else if (ob >= 7) a = lo >> (ob - 7);
                        else a = lo << (7 - ob);
                        wp[tt] = lds_u32((a & 0x1F80u) | lut_lane);
                    }
#pragma unroll
                    for (int g = 0; g < MG; ++g) {
                        u32x2 xa[4];  // four steps of four columns of the group's activation row of this lane
#pragma unroll
                        for (int s = 0; s < 4; ++s)
                            xa[s] = *reinterpret_cast<const __attribute__((address_space(3))) u32x2 *>(
                                (uintptr_t)(S.x_strip[g] + (uint32_t)k * 64u + (uint32_t)(4 * h + s) * 8u));
#pragma unroll
                        for (int s = 0; s < 4; ++s) {
                            const u32x2 b2 = u32x2{wp[2 * s], wp[2 * s + 1]};
                            acc[r][g] = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(
                                __builtin_bit_cast(s16x4, xa[s]), __builtin_bit_cast(s16x4, b2), acc[r][g], 0, 0, 0);
                        }
                    }
                }
            }
        }
        // The strips of a unit are four lanes apart: lanes q == 3 end up with the unit's sums and add them to the wave's
        // row sums.  Where the wave's four tasks are four different row quads: one addition; otherwise two of them may
        // hold the same matrix row (for different column blocks) and the DPP rows take turns, which keeps the order of
        // the additions fixed.
#pragma unroll
        for (int r = 0; r < R; ++r) {
            float sums[MT];
#pragma unroll
            for (int i = 0; i < MT; ++i) {
                sums[i] = 0.0f;
                if (i < m) {
                    float v = acc[r][i >> 2][i & 3];
                    v += __uint_as_float(dpp_shr(__float_as_uint(v), 4));
                    v += __uint_as_float(dpp_shr(__float_as_uint(v), 8));
                    sums[i] = v;
                }
            }
            const uint32_t at = rowacc_addr + S.lrow[r] * (uint32_t)m * 4u;
            if (quads_fastest) {
                if (q == 3 && S.live[r]) {
#pragma unroll
                    for (int i = 0; i < MT; ++i)
                        if (i < m) lds_add_f32_raw(at + (uint32_t)i * 4u, sums[i]);
                }
            } else {
#pragma unroll
                for (uint32_t dd = 0; dd < 4; ++dd) {
                    if (q == 3 && S.live[r] && drow == dd) {
#pragma unroll
                        for (int i = 0; i < MT; ++i)
                            if (i < m) lds_add_f32_raw(at + (uint32_t)i * 4u, sums[i]);
                    }
                }
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    };

    // Three steps per task, each one task ahead of the next: table entry + bitmap words (request), ranks and code
    // requests (launch_codes), decode (compute).  Two stages take turns, so nothing is copied between iterations.
    if (wave_iters > 0) {
        Stage A, B;
        launch_codes(T, A);
        if (wave_iters > 1) request(1, T);
        for (uint32_t it = 0; it < wave_iters; it += 2) {
            if (it + 1 < wave_iters) {
                launch_codes(T, B);
                if (it + 2 < wave_iters) request(it + 2, T);
            }
            compute(A);
            if (it + 1 < wave_iters) {
                if (it + 2 < wave_iters) {
                    launch_codes(T, A);
                    if (it + 3 < wave_iters) request(it + 3, T);
                }
                compute(B);
            }
        }
    }

    if (!ANY && sv.staged) {
        uint32_t *side = reinterpret_cast<uint32_t *>(smem + L.side);
#pragma unroll
        for (uint32_t n = 0; n < kSideRegs; ++n)
            if (tid + n * blockDim.x < kRSideBytes / 4) side[tid + n * blockDim.x] = side_reg[n];
    }
    // ---- the elements above level 1: all waves' records resolved together, 64 elements a round, when they fit the
    // shared task list; otherwise (dense mixes) every wave resolves its own queue ----
    {
        uint32_t *const counts = reinterpret_cast<uint32_t *>(smem + L.counts);
        uint32_t mine = 0;
        for (uint32_t idx = lane; idx < qcount; idx += kWave) mine += (uint32_t)__popc(queue[idx].x);
        const uint32_t my_total = (uint32_t)__builtin_amdgcn_readlane((int)wave_scan(mine), 63);
        if (lane == 0) counts[wave] = my_total;
        __syncthreads();
        const uint32_t cv = lane < n_waves ? counts[lane] : 0u;
        const uint32_t cincl = wave_scan(cv);
        const uint32_t total = (uint32_t)__builtin_amdgcn_readlane((int)cincl, 63);
        if (total <= kSPool) {
            uint32_t at = (uint32_t)__builtin_amdgcn_readlane((int)(cincl - cv), (int)wave);  // this wave's first task
            uint32_t *const pool = reinterpret_cast<uint32_t *>(smem + L.pool);
            for (uint32_t base = 0; base < qcount; base += kWave) {
                const uint32_t idx = base + lane;
                uint32_t zeros = idx < qcount ? queue[idx].x : 0u;
                const uint32_t cnt = (uint32_t)__popc(zeros);
                const uint32_t incl = wave_scan(cnt);
                uint32_t t = at + incl - cnt, nth = 0;
                while (zeros != 0) {
                    pool[t++] = (wave << 18) | (idx << 10) | (nth++ << 5) | (uint32_t)__builtin_ctz(zeros);
                    zeros &= zeros - 1;
                }
                at += (uint32_t)__builtin_amdgcn_readlane((int)incl, 63);
            }
            __syncthreads();
            const TaskPool tp{L.pool, total, wave, n_waves, L.waves, L.wave_bytes};
            if (ANY)
                resolve_rows<MT, false, true, 2, true>(P, sv, tq1_addr, tq2_addr, unit0, queue, 0, rowacc_addr, tasks,
                                                          xs_addr, L.xs_row, 0, m, scale, lane, prefix, entries, tp);
            else if (sv.staged)
                resolve_rows<MT, true, false, 2, true>(P, sv, tq1_addr, tq2_addr, unit0, queue, 0, rowacc_addr, tasks,
                                                          xs_addr, L.xs_row, 0, m, scale, lane, nullptr, 0, tp);
            else
                resolve_rows<MT, false, false, 2, true>(P, sv, tq1_addr, tq2_addr, unit0, queue, 0, rowacc_addr, tasks,
                                                           xs_addr, L.xs_row, 0, m, scale, lane, nullptr, 0, tp);
        } else {
            resolve();
        }
    }
    __syncthreads();

    // ---- add the workers' row sums in wave and DPP-row order, write bf16 (or add into the caller's fp32 vector) ----
    for (uint32_t t = tid; t < rows_here * (uint32_t)m; t += blockDim.x) {
        const uint32_t slot = t / (uint32_t)m, i = t - slot * (uint32_t)m;
        float sum = 0.0f;
        for (uint32_t w = 0; w < n_waves; ++w)
                sum += *reinterpret_cast<const float *>(smem + L.waves + w * L.wave_bytes + L.rowacc_off +
                                                        (slot * (uint32_t)m + i) * 4u);
        if (y32) atomicAdd(&y32[(size_t)i * P.out_f + row0 + slot], sum);
        else y[(int64_t)i * ldy + row0 + slot] = (uint16_t)f32_to_bf16_bits(sum);
    }
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------

struct StripsPlan {
    uint32_t quads, waves, qcap;
};

// Rows per workgroup (whole rounds of one workgroup per CU) and waves per workgroup: as many as the registers and LDS
// allow, then as few as run the workgroup's tasks (column blocks x row quads, one per DPP row) in the same rounds.
static StripsPlan plan_strips(uint32_t n_quads, uint32_t n_chunks, uint32_t n_cu, int m, int mg) {
    const uint32_t max_quads = kSMaxRows / 4;
    const uint32_t rounds = (n_quads + n_cu * max_quads - 1) / (n_cu * max_quads);
    const uint32_t quads = max(1u, min(max_quads, (n_quads + rounds * n_cu - 1) / (rounds * n_cu)));
    const uint32_t tasks = n_chunks * quads;
    uint32_t waves = min((uint32_t)strips_max_waves(mg), (tasks + 3) / 4);
    uint32_t qcap = kSQueue;
    if (strips_layout(quads * 4, n_chunks, waves, m, qcap).total > kSLdsLimit) qcap = kSQueue / 2;
    while (waves > 1 && strips_layout(quads * 4, n_chunks, waves, m, qcap).total > kSLdsLimit) --waves;
    const uint32_t task_rounds = (tasks + 4 * waves - 1) / (4 * waves);
    waves = (tasks + 4 * task_rounds - 1) / (4 * task_rounds);
    return StripsPlan{quads, waves, qcap};
}

template <int MG, bool ANY>
static int launch_strips(const Dev &P, const int32_t *prefix, uint32_t n_chunks, const StripsPlan &plan, const uint16_t *x,
                         int m, int64_t ldx, uint16_t *y, int64_t ldy, float *y32, hipStream_t s) {
    static const bool raised =  // per instantiation
        hipFuncSetAttribute(reinterpret_cast<const void *>(k_gemv358_strips<MG, ANY>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)kSLdsLimit) == hipSuccess;
    if (!raised) return IXH_EUNSUPPORTED;
    const uint32_t n_quads = P.out_f / 4;
    const uint32_t groups = (n_quads + plan.quads - 1) / plan.quads;
    const size_t lds = strips_layout(plan.quads * 4, n_chunks, plan.waves, m, plan.qcap).total;
    if (lds > kSLdsLimit) return IXH_EUNSUPPORTED;
    uint32_t flags = 0;
    if (((uintptr_t)P.last & 3u) == 0) flags |= kFlagStageSide;
    hipLaunchKernelGGL((k_gemv358_strips<MG, ANY>), dim3(groups), dim3(plan.waves * kWave), lds, s, P, prefix, n_chunks,
                       plan.quads, plan.qcap, flags, x, m, ldx, y, ldy, y32);
    return hipGetLastError() == hipSuccess ? IXH_OK : IXH_ELAUNCH;
}

// The strip kernel: up to four activation rows, whole row quads, rows of whole 512-column blocks that fit LDS beside
// the tables; IXH_EUNSUPPORTED sends the caller on to the other row-block kernels.
int launch_gemv_358_strips(const Dev &P, const int32_t *prefix, const uint16_t *x, int m, int64_t ldx, uint16_t *y,
                           int64_t ldy, float *y32, hipStream_t s) {
    if (m < 1 || m > kSMaxM || P.out_f % 4u != 0 || P.in_f % kFastChunk != 0 || P.in_f > 65536u) return IXH_EUNSUPPORTED;
    if (((uintptr_t)x & 15u) != 0 || (m > 1 && (ldx & 7) != 0)) return IXH_EUNSUPPORTED;
    const bool any = !(P.n_levels == 3 && P.bits[1] == 5);  // not (3,5,8): the resolver that walks the nested bitmaps
    static const int n_cu = [] {
        int dev = 0, v = 256;
        if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev);
        return v;
    }();
    const uint32_t n_chunks = P.in_f / kFastChunk;
    const int opt = g_opt_gemv_strips.load(std::memory_order_relaxed);  // ixh_set_option("gemv_strips")
    if (opt < 0) return IXH_EUNSUPPORTED;
    // one or two activation rows: the kernels that multiply lane by lane are as fast or faster (measured on 5120 x 17408
    // and 17408 x 5120); the matrix pipe pays from three rows on
    if (opt == 0 && m <= 2) return IXH_EUNSUPPORTED;
    const int mg = m <= 4 ? 1 : (m <= 8 ? 2 : 4);
    const StripsPlan plan = plan_strips(P.out_f / 4, n_chunks, (uint32_t)n_cu, m, mg);
#define IXH_STRIPS(MGV)                                                                                      \
    if (mg == MGV)                                                                                           \
        return any ? launch_strips<MGV, true>(P, prefix, n_chunks, plan, x, m, ldx, y, ldy, y32, s)          \
                   : launch_strips<MGV, false>(P, prefix, n_chunks, plan, x, m, ldx, y, ldy, y32, s);
    IXH_STRIPS(1) IXH_STRIPS(2) IXH_STRIPS(4)
#undef IXH_STRIPS
    return IXH_EUNSUPPORTED;
}

}  // namespace ixh
