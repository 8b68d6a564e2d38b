// (3,5,8) fused decode + GEMV for gfx950, row-block variant: one workgroup owns
// whole rows, so the result leaves as bf16 from a single launch with no
// workspace, no atomics in global memory and a fixed summation order.
//
// Work split.  The matrix is cut into 512-wide column blocks ("units" of one
// row) and into row quads.  Wave w of a workgroup owns C neighbouring column
// blocks and keeps its x slices in registers; the workgroup walks down its row
// quads, each 16-lane DPP row of a wave taking one matrix row and each lane 32
// consecutive elements (one word of bitmap 0).
//
// Memory pipeline.  Nothing the kernel streams depends on what it decodes: the
// 3-bit stream range of a unit follows from the rank table alone.  The
// workgroup first copies its slice of the table into LDS; after that
// every wave keeps kRStages unit-quads in flight with LDS-DMA buffer loads (one
// dword per lane of bitmap 0, and 13 x 16 bytes per row of the 3-bit stream),
// which need no registers and are bounds-checked by the buffer descriptor.
//
// Decode.  Per unit a lane reads its bitmap word, ranks it with a 4-step DPP
// scan over its row, reads its own 96-bit code window from the staged stream
// and aligns it with three v_alignbit.  Elements that are not level 1 are
// spliced out of the window (their field becomes the code of 0) and handed, one
// record per lane, to a per-wave LDS queue that is resolved 64 records at a
// time.  When the workgroup's share of bitmap 1 and of the 5-bit and 8-bit
// streams is small (the usual case: few elements are above level 1) it is
// staged in LDS up front and the resolution touches no global memory.  Two
// neighbouring codes index a bank-conflict-free table of dequantised weight
// pairs in LDS (64 entries x 32 lane copies); the packed bf16 pair meets the x
// pair in v_dot2_f32_bf16.  The window of unit i+1 is opened while the pairs of
// unit i are processed.
//
// Reduction.  Lanes sum over the wave's C blocks, rows over their 16 lanes
// (DPP), waves through LDS after one barrier, in wave order.
//
// Two kernels share this decode: k_gemv358_rows (a wave owns column blocks, x in
// registers) and k_gemv358_rowsx further down (x in LDS once per workgroup, the
// unit-quads dealt to 16 waves), which serves the shapes whose row count is a
// multiple of four.
#include <math.h>
#include <stdlib.h>

#include <mutex>

#include "ixh_rows_common.h"

namespace ixh {

typedef float f32x2 __attribute__((ext_vector_type(2)));


// a wave's region: ring, record queue, row sums, task list, and a copy of the activations of its own column
// blocks (c blocks x mt rows x 512 bf16) for the elements above level 1
__host__ __device__ constexpr uint32_t wave_lds_bytes(int mt, int c) {
    return kRStages * kRStageBytes + kRQueue * 16 + kRSlots * mt * 4 + kRTasks2 * 2 + (uint32_t)(c * mt) * kFastChunk * 2;
}

// byte offsets of the regions of a workgroup's LDS; the pair table is at 0, the splice masks follow
struct RowsLds {
    uint32_t tq1, tq2, side, waves, total;
};

__host__ __device__ inline RowsLds rows_layout(uint32_t rows_cap, uint32_t n_chunks, uint32_t n_waves, int mt,
                                               int c) {
    RowsLds L;
    const uint32_t tbl = ((rows_cap * n_chunks + 1u + 3u) & ~3u) * 4u;  // one entry past the slice: its end ranks
    L.tq1 = kRLutBytes + kRSpliceBytes;
    L.tq2 = L.tq1 + tbl;
    L.side = L.tq2 + tbl;
    L.waves = L.side + kRSideBytes;
    L.total = L.waves + n_waves * wave_lds_bytes(mt, c);
    return L;
}


template <int MT, int C, bool ANY = false>
__global__ void __launch_bounds__(kRMaxWaves * kWave)
k_gemv358_rows(Dev P, const int32_t *__restrict__ prefix, uint32_t n_chunks, uint32_t quads_per_wg, uint32_t flags,
               const uint16_t *__restrict__ x, int m, int64_t ldx, uint16_t *__restrict__ y, int64_t ldy,
               float *__restrict__ y32) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const uint32_t n_waves = blockDim.x >> 6;
    const uint32_t quarter = lane >> 4, li = lane & 15;

    const uint32_t n_quads = (P.out_f + 3) >> 2;
    const uint32_t quad0 = blockIdx.x * quads_per_wg;
    const uint32_t n_steps = min(quads_per_wg, n_quads - quad0);
    const uint32_t row0 = quad0 * 4;
    const uint32_t rows_here = min(n_steps * 4, P.out_f - row0);
    const RowsLds L = rows_layout(min(quads_per_wg * 4, P.out_f), n_chunks, n_waves, MT, C);

    // The pair table is addressed with (index bits | lane bits), which needs it at
    // LDS address 0; that holds because the kernel has no other LDS.  Should it
    // ever not hold, say so in the output instead of computing garbage.
    if ((uint32_t)(uintptr_t)(lds_ptr_t)smem != 0) {
        for (uint32_t t = tid; t < rows_here * MT; t += blockDim.x)
            if ((int)(t % MT) < m) {
                if (y32) y32[(size_t)(t % MT) * P.out_f + row0 + t / MT] = __uint_as_float(0x7FC00000u);  // NaN
                else y[(int64_t)(t % MT) * ldy + row0 + t / MT] = 0x7FC0;
            }
        return;
    }
    uint32_t *const lut = reinterpret_cast<uint32_t *>(smem);            // [64][32]
    uint4 *const splice = reinterpret_cast<uint4 *>(smem + kRLutBytes);  // [33][2]
    uint32_t *const tq1 = reinterpret_cast<uint32_t *>(smem + L.tq1);
    uint32_t *const tq2 = reinterpret_cast<uint32_t *>(smem + L.tq2);
    uint8_t *const wave_base = smem + L.waves + wave * wave_lds_bytes(MT, C);
    uint8_t *const ring = wave_base;
    uint4 *const queue = reinterpret_cast<uint4 *>(wave_base + kRStages * kRStageBytes);
    float *const rowacc = reinterpret_cast<float *>(wave_base + kRStages * kRStageBytes + kRQueue * 16);
    uint16_t *const tasks = reinterpret_cast<uint16_t *>(rowacc + kRSlots * MT);
    uint32_t *const xs = reinterpret_cast<uint32_t *>(tasks + kRTasks2);  // [MT][C * 512] bf16

    // ---- workgroup set-up: table slices and x first (they wait on memory), then the tables built here ----
    const uint16_t scale_bits = *P.scale;  // asked for with the table slices, not in a trip to memory of its own after them
    const uint32_t unit0 = row0 * n_chunks;
    const uint32_t entries = P.out_f * n_chunks + 1;
    for (uint32_t i = tid; i <= rows_here * n_chunks; i += blockDim.x) {
            tq1[i] = (uint32_t)prefix[unit0 + i];
            if (!ANY) tq2[i] = (uint32_t)prefix[entries + unit0 + i];
        }
    const float scale = bf16_bits_to_f32(scale_bits);
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
        for (int d = 0; d < 3; ++d) {
            const uint32_t base = 32u * d;
            lm[d] = pos <= base ? 0u : (pos >= base + 32 ? ~0u : (1u << (pos - base)) - 1u);
            f[d] = (pos + 3 <= base || pos >= base + 32) ? 0u : (pos >= base ? 7u << (pos - base) : 7u >> (base - pos));
        }
        splice[2 * tid] = make_uint4(lm[0], lm[1], lm[2], 0u);
        splice[2 * tid + 1] = make_uint4(f[0], f[1], f[2], 0u);
    }
    for (uint32_t j = lane; j < kRSlots * MT; j += kWave) rowacc[j] = 0.0f;
    __syncthreads();

    const uint32_t col0 = wave * C;

    // The wave's activations (C blocks x MT rows x 512 bf16) go to its LDS area by LDS-DMA, 1 KB per instruction, and
    // from there into registers once the first copies have landed: one request per byte of x and wave (the four
    // 16-lane rows need the same bytes), and nothing waits for x before the ring's first copies are on their way.
    {
        const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc(
            (void *)x, 0, (int)((((int64_t)(m - 1) * ldx + P.in_f) * 2)), 0x00020000);
#pragma unroll
        for (int cc = 0; cc < C; ++cc) {
            const uint32_t col = min(col0 + cc, n_chunks - 1);
#pragma unroll
            for (int j = 0; j < MT; ++j)
                if (j < m)
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(
                        x_rsrc, (lds_ptr_t)(xs + (j * C + cc) * (kFastChunk / 2)), 16,
                        (int)(((int64_t)j * ldx + col * kFastChunk) * 2 + lane * 16), 0, 0, 0);
        }
    }

    const __amdgpu_buffer_rsrc_t b1_rsrc =
        __builtin_amdgcn_make_buffer_rsrc((void *)P.bm[0], 0, (int)(P.bm_words[0] * 4u), 0x00020000);
    const __amdgpu_buffer_rsrc_t l1_rsrc =
        __builtin_amdgcn_make_buffer_rsrc((void *)P.st[0], 0, (int)(P.st_words[0] * 4u), 0x00020000);

    // ---- this workgroup's share of bitmap 1 and of the 5-bit / 8-bit streams ----
    // Its extent follows from the ranks at the first and one past the last row.  If it fits, every wave
    // DMAs all of it (same bytes to the same place, so no barrier is needed: a wave's own loads
    // complete in order, before the first unit it waits for).
    SideView sv;
    sv.staged = false;
    if (!ANY) {
        const uint32_t n_local = rows_here * n_chunks;
        const uint32_t q1b = tq1[0], q2b = tq2[0], q1e = tq1[n_local], q2e = tq2[n_local];
        const uint32_t nl1b = row0 * P.in_f - q1b, nl1e = (row0 + rows_here) * P.in_f - q1e;
        sv.base = L.side;
        sv.b2w0 = nl1b >> 5;
        sv.l2w0 = (uint32_t)(((uint64_t)q2b * 5u) >> 5);
        sv.l3w0 = (nl1b - q2b) >> 2;
        const uint32_t n_b2 = ((nl1e + 31) >> 5) - sv.b2w0;
        const uint32_t n_l2 = (uint32_t)((((uint64_t)q2e * 5u) + 31) >> 5) - sv.l2w0;
        const uint32_t n_l3 = ((nl1e - q2e + 3) >> 2) - sv.l3w0;
        // one word of slack each: the resolver reads the word after a code's first word unconditionally
        sv.staged = (flags & kFlagStageSide) && n_b2 < 256 && n_l2 < 511 && n_l3 <= 256;
        if (sv.staged) {
            const __amdgpu_buffer_rsrc_t b2_rsrc =
                __builtin_amdgcn_make_buffer_rsrc((void *)P.bm[1], 0, (int)(P.bm_words[1] * 4u), 0x00020000);
            const __amdgpu_buffer_rsrc_t l2_rsrc =
                __builtin_amdgcn_make_buffer_rsrc((void *)P.st[1], 0, (int)(P.st_words[1] * 4u), 0x00020000);
            const __amdgpu_buffer_rsrc_t l3_rsrc =
                // whole dwords: the range check is per dword, and the stream's last 1..3 bytes are wanted too
                // (device allocations are 256-byte granular, so the dword is there to read)
                __builtin_amdgcn_make_buffer_rsrc((void *)P.last, 0, (int)((P.last_bytes + 3u) & ~3u), 0x00020000);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(b2_rsrc, (lds_ptr_t)(smem + L.side + kRSideB2), 16,
                                                     (int)(sv.b2w0 * 4 + lane * 16), 0, 0, 0);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(l2_rsrc, (lds_ptr_t)(smem + L.side + kRSideL2), 16,
                                                     (int)(sv.l2w0 * 4 + lane * 16), 0, 0, 0);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(l2_rsrc, (lds_ptr_t)(smem + L.side + kRSideL2 + 1024), 16,
                                                     (int)(sv.l2w0 * 4 + 1024 + lane * 16), 0, 0, 0);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(l3_rsrc, (lds_ptr_t)(smem + L.side + kRSideL3), 16,
                                                     (int)(sv.l3w0 * 4 + lane * 16), 0, 0, 0);
        }
    }

    const uint32_t lut_lane = (lane & 31u) << 2;
    const uint32_t splice_addr = kRLutBytes;
    const uint32_t tq1_addr = L.tq1, tq2_addr = L.tq2;
    const uint32_t ring_addr = (uint32_t)(uintptr_t)(lds_ptr_t)ring;

    // Unit-quads of this wave in walk order: index i -> (step i / C, block i % C).
    const uint32_t n_units = n_steps * C;

    // ---- producer: LDS-DMA of unit-quad i into ring stage i % kRStages ----
    uint32_t i_step = 0, i_cc = 0;                            // (step, block) of the next unit to issue
    uint32_t i_lrn = __umul24(min(quarter, rows_here - 1), n_chunks);  // its local row * n_chunks, per lane
    auto issue = [&](uint32_t i) {
        const uint32_t col = min(col0 + i_cc, n_chunks - 1);
        const uint32_t q1u = lds_u32(tq1_addr + (i_lrn + col) * 4);
        const uint32_t unit = unit0 + i_lrn + col;
        uint8_t *stage = ring + (i % kRStages) * kRStageBytes;
        asm volatile("" ::: "memory");
        if (li < 13)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(l1_rsrc, (lds_ptr_t)stage, 16,
                                                     (int)(((q1u * 3u) >> 5) * 4u + li * 16u), 0, 0, 0);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(b1_rsrc, (lds_ptr_t)(stage + 1024), 4,
                                                 (int)((unit * 16u + li) * 4u), 0, 0, 0);
        if (++i_cc == C) {
            i_cc = 0;
            ++i_step;
            i_lrn = __umul24(min(4 * i_step + quarter, rows_here - 1), n_chunks);
        }
    };

    uint32_t qcount = 0;  // wave-uniform

    // one splice of the 96-bit window at the lowest zero bit left in zrem (identity when none is left)
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

    // ---- consumer, first half: code window of unit-quad i (its data is in the ring), spliced once ----
    auto open_window = [&](uint32_t i, uint32_t slot, uint32_t lrn, bool valid, uint32_t cc, uint32_t &w0,
                           uint32_t &w1, uint32_t &w2, uint32_t &zrem) {
        valid = valid && (col0 + cc < n_chunks);
        const uint32_t col = min(col0 + cc, n_chunks - 1);
        const uint32_t stage = ring_addr + (i % kRStages) * kRStageBytes;
        const uint32_t word = lds_u32(stage + 1024 + lane * 4);
        const uint32_t q1u = lds_u32(tq1_addr + (lrn + col) * 4);
        const uint32_t c = __popc(word);
        const uint32_t excl = row_scan(c) - c;
        const uint32_t off = __umul24(excl, 3u) + ((q1u * 3u) & 31u);  // bit offset inside the staged stream piece
        const uint32_t wa = stage + quarter * 256 + (off >> 5) * 4;
        const uint32_t d0 = lds_u32(wa), d1 = lds_u32(wa + 4), d2 = lds_u32(wa + 8), d3 = lds_u32(wa + 12);
        w0 = __builtin_amdgcn_alignbit(d1, d0, off);
        w1 = __builtin_amdgcn_alignbit(d2, d1, off);
        w2 = __builtin_amdgcn_alignbit(d3, d2, off);
        uint32_t zeros = ~word;
        if (!valid) {
            zeros = 0u;
            w0 = kZeroCodes0; w1 = kZeroCodes1; w2 = kZeroCodes2;
        }
        // lanes with elements above level 1 leave a record (the loop head keeps 64 slots free)
        const uint64_t any = __ballot(zeros != 0);
        if (zeros != 0) {
            const uint32_t unit = unit0 + lrn + col;
            const uint32_t r0_lane = unit * kFastChunk + li * 32u - (q1u + excl);
            push_record(queue, qcount + lanes_below(any),
                        make_uint4(zeros, r0_lane, unit, (slot << 16) | (col * kFastChunk + li * 32u)));
        }
        qcount += (uint32_t)__popcll(any);
        zrem = zeros;
        splice_once(w0, w1, w2, zrem);
    };

    const uint32_t xs_addr = (uint32_t)(uintptr_t)(lds_ptr_t)xs;
    const uint32_t rowacc_addr = (uint32_t)(uintptr_t)(lds_ptr_t)rowacc;
    auto resolve = [&]() {
        if (ANY)
            resolve_rows<MT, false, true>(P, sv, tq1_addr, tq2_addr, unit0, queue, qcount, rowacc_addr, tasks, xs_addr,
                                          C * kFastChunk, col0 * kFastChunk, m, scale, lane, prefix, entries);
        else if (sv.staged)
            resolve_rows<MT, true>(P, sv, tq1_addr, tq2_addr, unit0, queue, qcount, rowacc_addr, tasks, xs_addr,
                                   C * kFastChunk, col0 * kFastChunk, m, scale, lane);
        else
            resolve_rows<MT, false>(P, sv, tq1_addr, tq2_addr, unit0, queue, qcount, rowacc_addr, tasks, xs_addr,
                                    C * kFastChunk, col0 * kFastChunk, m, scale, lane);
        qcount = 0;
    };

    // ---- start-up: fill the ring, open the first window ----
    const uint32_t n_pre = min((uint32_t)kRStages, n_units);
    for (uint32_t i = 0; i < n_pre; ++i) issue(i);
    if (n_units >= (uint32_t)kRStages) wait_vmem<2 * (kRStages - 1)>();
    else wait_vmem<0>();

    // this lane's activations: C blocks x MT rows x 16 packed bf16 pairs
    uint32_t xr[C][MT][16];
#pragma unroll
    for (int cc = 0; cc < C; ++cc)
#pragma unroll
        for (int j = 0; j < MT; ++j) {
            if (j < m) {
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const u32x4 v = lds_u128((uint32_t)(uintptr_t)(lds_ptr_t)xs +
                                             (((uint32_t)(j * C + cc) * (kFastChunk / 2) + li * 16 + 4 * t) * 4u));
                    xr[cc][j][4 * t] = v.x; xr[cc][j][4 * t + 1] = v.y;
                    xr[cc][j][4 * t + 2] = v.z; xr[cc][j][4 * t + 3] = v.w;
                }
            } else {
#pragma unroll
                for (int t = 0; t < 16; ++t) xr[cc][j][t] = 0u;
            }
        }

    uint32_t lrn_step = __umul24(min(quarter, rows_here - 1), n_chunks);  // local row * n_chunks of the current step
    bool valid_step = quarter < rows_here;
    uint32_t cw0, cw1, cw2, czrem;
    open_window(0, quarter, lrn_step, valid_step, 0, cw0, cw1, cw2, czrem);
    while (__ballot(czrem != 0) != 0) splice_once(cw0, cw1, cw2, czrem);

    constexpr int NA = MT == 1 ? 4 : (MT == 2 ? 2 : 1);  // independent accumulators per x row

    for (uint32_t step = 0; step < n_steps; ++step) {
        // The waves that share a SIMD take turns at the issue priority, one row quad each: without this the
        // oldest wave is served first throughout, finishes early and leaves the others to end the kernel with
        // nothing to hide their waits behind.
        set_wave_priority(((wave >> 2) + step) % 3u);
        float acc[MT][NA];
#pragma unroll
        for (int j = 0; j < MT; ++j)
#pragma unroll
            for (int a = 0; a < NA; ++a) acc[j][a] = 0.0f;
        const uint32_t lrn_next = __umul24(min(4 * (step + 1) + quarter, rows_here - 1), n_chunks);
        const bool valid_next = 4 * (step + 1) + quarter < rows_here;

#pragma unroll
        for (int cc = 0; cc < C; ++cc) {
            const uint32_t i = step * C + cc;
            if (qcount > kRQueue - kWave) resolve();  // keep room for a full wave of records
            // refill the stage whose window was read last time; make unit i+1 readable
            if (i + kRStages < n_units) {
                issue(i + kRStages);
                wait_vmem<2 * (kRStages - 1)>();
            } else {
                wait_vmem<0>();
            }

            // The 16 code pairs of unit i go through the pair table and meet the x pairs.  Written first: the pair
            // table reads and the first reads of the next window then sit in one basic block (the record store
            // below ends it), so they are issued together and the dot products fill the wait for the window.
#pragma unroll
            for (int t = 0; t < 16; ++t) {
                const int bit = 6 * t, ob = bit & 31, d = bit >> 5;
                const uint32_t lo = d == 0 ? cw0 : (d == 1 ? cw1 : cw2);
                const uint32_t hi = d == 0 ? cw1 : cw2;
                uint32_t a;  // pair index at bits 12..7
                if (ob > 26) a = __builtin_amdgcn_alignbit(hi, lo, ob - 7);
                else if (ob >= 7) a = lo >> (ob - 7);
                else a = lo << (7 - ob);
                const uint32_t wp = lds_u32((a & 0x1F80u) | lut_lane);
#pragma unroll
                for (int j = 0; j < MT; ++j)
                    acc[j][t % NA] = __builtin_amdgcn_fdot2_f32_bf16(
                        __builtin_bit_cast(bf16x2, wp), __builtin_bit_cast(bf16x2, xr[cc][j][t]), acc[j][t % NA], false);
            }

            // window of unit i+1 (or, past the end, a void one)
            uint32_t nw0, nw1, nw2, nzrem;
            {
                const bool last_cc = cc == C - 1;
                const uint32_t n_i = min(i + 1, n_units - 1);
                open_window(n_i, 4 * (last_cc ? step + 1 : step) + quarter, last_cc ? lrn_next : lrn_step,
                            (last_cc ? valid_next : valid_step) && (i + 1 < n_units), last_cc ? 0 : cc + 1, nw0, nw1,
                            nw2, nzrem);
            }

            // lanes with more than one element above level 1 (rare): splice on
            while (__ballot(nzrem != 0) != 0) splice_once(nw0, nw1, nw2, nzrem);
            cw0 = nw0; cw1 = nw1; cw2 = nw2;
        }
#pragma unroll
        for (int j = 0; j < MT; ++j) {
            float sum = acc[j][0];
#pragma unroll
            for (int a = 1; a < NA; ++a) sum += acc[j][a];
            const float total = row_sum(sum);
            if (li == 15) rowacc[(4 * step + quarter) * MT + j] += total;
        }
        lrn_step = lrn_next;
        valid_step = valid_next;
    }

    resolve();
    __syncthreads();

    // ---- add the waves' row sums in wave order, write bf16 ----
    const uint32_t first_acc = L.waves + kRStages * kRStageBytes + kRQueue * 16;
    for (uint32_t t = tid; t < rows_here * MT; t += blockDim.x) {
        const uint32_t slot = t / MT, j = t - slot * MT;
        if ((int)j >= m) continue;
        float sum = 0.0f;
        for (uint32_t w = 0; w < n_waves; ++w)
            sum += *reinterpret_cast<const float *>(smem + first_acc + w * wave_lds_bytes(MT, C) + t * 4);
        // a workgroup owns whole rows: the one addition per output a split-K caller's fp32 vector takes, or bf16
        if (y32) atomicAdd(&y32[(size_t)j * P.out_f + row0 + slot], sum);
        else y[(int64_t)j * ldy + row0 + slot] = (uint16_t)f32_to_bf16_bits(sum);
    }
}

// ---------------------------------------------------------------------------
// Up to four activation rows, x shared by the workgroup
// ---------------------------------------------------------------------------
// Same decode as k_gemv358_rows, different work split.  There a wave owns column blocks and keeps their activations
// in registers, which ties the number of waves to the number of column blocks (12 waves, three per SIMD, for 34
// blocks; 10 waves for 10 blocks) and makes every wave walk all row quads of its blocks one after the other.  Here
// the activation rows sit in LDS once per workgroup (swizzled, so that the 16 lanes of a row read consecutive
// 16-byte pieces), the workgroup's unit-quads are dealt round-robin to as many waves as LDS allows (16: four per
// SIMD), and a wave reads the 64 activation bytes of a lane afresh for every unit-quad (four ds_read_b128 per
// activation row).  Neighbouring waves work on neighbouring column blocks of the same row quad, so what a
// workgroup has in flight is contiguous in every row.  Every row quad is whole (out_f % 4 == 0; other shapes stay
// with k_gemv358_rows), which leaves the lanes one addition per table or bitmap address: a lane constant plus the
// scalar index of the unit-quad.
constexpr int kXMaxWaves = 16;
constexpr uint32_t kXSlots = 128;  // rows per workgroup at most
// Unit-quads in flight per wave, the one being read included.  Two: measured against three and four (with 16 waves
// per CU), every stage more costs 2-3 %; fewer copies in flight leave more of a CU's cache lines to be found again
// by the wave that works on the neighbouring column block.
constexpr int kXStages = 2;

// a wave's region: ring, record queue (qcap records), row sums (one per row of the workgroup and activation row), task list
__host__ __device__ constexpr uint32_t wave_lds_bytes_x(int mt, uint32_t rows_cap, uint32_t qcap) {
    return kXStages * kRStageBytes + qcap * 16 + ((rows_cap * (uint32_t)mt * 4 + 15u) & ~15u) + kRTasks2 * 2;
}

struct RowsXLds {
    uint32_t tq1, tq2, side, xs, waves, total;
};

__host__ __device__ inline RowsXLds rowsx_layout(uint32_t rows_cap, uint32_t n_chunks, uint32_t n_waves, int mt,
                                                 uint32_t qcap) {
    RowsXLds L;
    const uint32_t tbl = ((rows_cap * n_chunks + 1u + 3u) & ~3u) * 4u;
    L.tq1 = kRLutBytes + kRSpliceBytes;
    L.tq2 = L.tq1 + tbl;
    L.side = L.tq2 + tbl;
    L.xs = L.side + kRSideBytes;
    L.waves = L.xs + (uint32_t)mt * n_chunks * kFastChunk * 2;
    L.total = L.waves + n_waves * wave_lds_bytes_x(mt, rows_cap, qcap);
    return L;
}

// Five to eight activation rows (MT = 8) run with eight waves of up to 256 registers: the activations of a
// unit-quad are 128 registers per lane.
template <int MT, bool ANY>
__global__ void __launch_bounds__((MT > 4 ? kXMaxWaves / 2 : kXMaxWaves) * kWave)
k_gemv358_rowsx(const int32_t *__restrict__ prefix, const uint16_t *__restrict__ x, const uint16_t *__restrict__ scale_ptr,
                int64_t ldx, const uint32_t *__restrict__ bm0, const uint32_t *__restrict__ st0, uint32_t out_f, uint32_t geometry,
                Dev P, uint16_t *__restrict__ y, int64_t ldy, float *__restrict__ y32) {
    // The arguments before P are what the first requests to memory need.  They fill the 14 argument registers that
    // the hardware loads before a wave starts (the file is compiled with that many preloaded), so those requests do
    // not wait for a read of the argument block: scale_ptr, bm0, st0 and out_f repeat fields of P for that reason,
    // and the launch geometry (the workgroup size included, which the compiler would read from the block) is
    // packed into one word (column blocks, row quads per workgroup, waves, activation rows, flags).
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const uint32_t n_chunks = geometry & 0xFFFu, quads_per_wg = (geometry >> 12) & 0xFFu, n_waves = (geometry >> 20) & 0x1Fu;
    const int m = (int)((geometry >> 25) & 0xFu);
    const uint32_t flags = geometry >> 29;
    const uint32_t in_f = n_chunks * kFastChunk, n_threads = n_waves * kWave;

    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const uint32_t quarter = lane >> 4, li = lane & 15;

    const uint32_t n_quads = (out_f + 3) >> 2;
    const uint32_t quad0 = blockIdx.x * quads_per_wg;
    const uint32_t n_steps = min(quads_per_wg, n_quads - quad0);
    const uint32_t row0 = quad0 * 4;
    const uint32_t rows_here = min(n_steps * 4, out_f - row0);
    constexpr uint32_t qcap = kRQueue;  // records the wave's queue holds
    const uint32_t rows_cap = min(quads_per_wg * 4, out_f);
    const RowsXLds L = rowsx_layout(rows_cap, n_chunks, n_waves, MT, qcap);

    // the pair table is addressed with (index bits | lane bits): it must sit at LDS address 0
    if ((uint32_t)(uintptr_t)(lds_ptr_t)smem != 0) {
        for (uint32_t t = tid; t < rows_here * MT; t += n_threads)
            if ((int)(t % MT) < m) {
                if (y32) y32[(size_t)(t % MT) * out_f + row0 + t / MT] = __uint_as_float(0x7FC00000u);  // NaN
                else y[(int64_t)(t % MT) * ldy + row0 + t / MT] = 0x7FC0;
            }
        return;
    }
    uint32_t *const lut = reinterpret_cast<uint32_t *>(smem);            // [64][32]
    uint4 *const splice = reinterpret_cast<uint4 *>(smem + kRLutBytes);  // [33][2]
    uint32_t *const tq1 = reinterpret_cast<uint32_t *>(smem + L.tq1);
    uint32_t *const tq2 = reinterpret_cast<uint32_t *>(smem + L.tq2);
    uint8_t *const wave_base = smem + L.waves + wave * wave_lds_bytes_x(MT, rows_cap, qcap);
    uint8_t *const ring = wave_base;
    uint4 *const queue = reinterpret_cast<uint4 *>(wave_base + kXStages * kRStageBytes);
    float *const rowacc = reinterpret_cast<float *>(wave_base + kXStages * kRStageBytes + qcap * 16);
    uint16_t *const tasks = reinterpret_cast<uint16_t *>(wave_base + wave_lds_bytes_x(MT, rows_cap, qcap) - kRTasks2 * 2);

    // the scale is asked for here, with the first requests: read where the pair table is built, it was a trip to memory
    // of its own between the table slices' and the barrier
    const uint16_t scale_bits = *scale_ptr;
    // ---- the activation row: needs nothing but the arguments, so it is requested first.  Lane (t, l) of the copy
    // fetches piece l * 4 + t of the block and the hardware puts it at piece t * 16 + l.
    {
        const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc(
            (void *)x, 0, (int)((((int64_t)(m - 1) * ldx + in_f) * 2)), 0x00020000);
        for (uint32_t t = wave; t < (uint32_t)m * n_chunks; t += n_waves) {
            const uint32_t j = t / n_chunks, col = t - j * n_chunks;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(
                x_rsrc, (lds_ptr_t)(smem + L.xs + (j * n_chunks + col) * (kFastChunk * 2)), 16,
                (int)(((int64_t)j * ldx + col * kFastChunk) * 2 + (li * 4u + quarter) * 16u), 0, 0, 0);
        }
    }

    // ---- workgroup set-up: table slices, pair table, splice masks ----
    const uint32_t unit0 = row0 * n_chunks;
    const uint32_t entries = out_f * n_chunks + 1;
    for (uint32_t i = tid; i <= rows_here * n_chunks; i += n_threads) {
        tq1[i] = (uint32_t)prefix[unit0 + i];
        if (!ANY) tq2[i] = (uint32_t)prefix[entries + unit0 + i];
    }
    const float scale = bf16_bits_to_f32(scale_bits);
    for (uint32_t i = tid; i < 64 * 32; i += n_threads) {
        const int c0 = (i >> 5) & 7, c1 = i >> 8;
        const f32x2 w = {c0 < 7 ? (float)(c0 - 3) * scale : 0.0f, c1 < 7 ? (float)(c1 - 3) * scale : 0.0f};
        lut[i] = __builtin_bit_cast(uint32_t, __builtin_convertvector(w, bf16x2));  // round to nearest even
    }
    if (tid <= 32) {
        const uint32_t pos = 3 * tid;
        uint32_t lm[3], f[3];
#pragma unroll
        for (int d = 0; d < 3; ++d) {
            const uint32_t base = 32u * d;
            lm[d] = pos <= base ? 0u : (pos >= base + 32 ? ~0u : (1u << (pos - base)) - 1u);
            f[d] = (pos + 3 <= base || pos >= base + 32) ? 0u : (pos >= base ? 7u << (pos - base) : 7u >> (base - pos));
        }
        splice[2 * tid] = make_uint4(lm[0], lm[1], lm[2], 0u);
        splice[2 * tid + 1] = make_uint4(f[0], f[1], f[2], 0u);
    }
    for (uint32_t j = lane; j < rows_cap * MT; j += kWave) rowacc[j] = 0.0f;
    wait_vmem<0>();  // this wave's pieces of x are in LDS
    __syncthreads();

    const __amdgpu_buffer_rsrc_t b1_rsrc =
        __builtin_amdgcn_make_buffer_rsrc((void *)bm0, 0, (int)(out_f * (in_f >> 5) * 4u), 0x00020000);  // whole words here
    const __amdgpu_buffer_rsrc_t l1_rsrc =
        __builtin_amdgcn_make_buffer_rsrc((void *)st0, 0, (int)(P.st_words[0] * 4u), 0x00020000);

    // ---- this workgroup's share of bitmap 1 and of the 5-bit / 8-bit streams (as in k_gemv358_rows) ----
    SideView sv;
    sv.staged = false;
    if (!ANY) {
        const uint32_t n_local = rows_here * n_chunks;
        const uint32_t q1b = tq1[0], q2b = tq2[0], q1e = tq1[n_local], q2e = tq2[n_local];
        const uint32_t nl1b = row0 * in_f - q1b, nl1e = (row0 + rows_here) * in_f - q1e;
        sv.base = L.side;
        sv.b2w0 = nl1b >> 5;
        sv.l2w0 = (uint32_t)(((uint64_t)q2b * 5u) >> 5);
        sv.l3w0 = (nl1b - q2b) >> 2;
        const uint32_t n_b2 = ((nl1e + 31) >> 5) - sv.b2w0;
        const uint32_t n_l2 = (uint32_t)((((uint64_t)q2e * 5u) + 31) >> 5) - sv.l2w0;
        const uint32_t n_l3 = ((nl1e - q2e + 3) >> 2) - sv.l3w0;
        sv.staged = (flags & kFlagStageSide) && n_b2 < 256 && n_l2 < 511 && n_l3 <= 256;
        if (sv.staged) {
            const __amdgpu_buffer_rsrc_t b2_rsrc =
                __builtin_amdgcn_make_buffer_rsrc((void *)P.bm[1], 0, (int)(P.bm_words[1] * 4u), 0x00020000);
            const __amdgpu_buffer_rsrc_t l2_rsrc =
                __builtin_amdgcn_make_buffer_rsrc((void *)P.st[1], 0, (int)(P.st_words[1] * 4u), 0x00020000);
            const __amdgpu_buffer_rsrc_t l3_rsrc =
                __builtin_amdgcn_make_buffer_rsrc((void *)P.last, 0, (int)((P.last_bytes + 3u) & ~3u), 0x00020000);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(b2_rsrc, (lds_ptr_t)(smem + L.side + kRSideB2), 16,
                                                     (int)(sv.b2w0 * 4 + lane * 16), 0, 0, 0);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(l2_rsrc, (lds_ptr_t)(smem + L.side + kRSideL2), 16,
                                                     (int)(sv.l2w0 * 4 + lane * 16), 0, 0, 0);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(l2_rsrc, (lds_ptr_t)(smem + L.side + kRSideL2 + 1024), 16,
                                                     (int)(sv.l2w0 * 4 + 1024 + lane * 16), 0, 0, 0);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(l3_rsrc, (lds_ptr_t)(smem + L.side + kRSideL3), 16,
                                                     (int)(sv.l3w0 * 4 + lane * 16), 0, 0, 0);
        }
    }

    const uint32_t lut_lane = (lane & 31u) << 2;
    const uint32_t splice_addr = kRLutBytes;
    const uint32_t tq1_addr = L.tq1, tq2_addr = L.tq2;
    const uint32_t ring_addr = (uint32_t)(uintptr_t)(lds_ptr_t)ring;
    const uint32_t xs_addr = L.xs, xs_row = n_chunks * (kFastChunk * 2);  // bytes between activation rows
    const uint32_t rowacc_addr = (uint32_t)(uintptr_t)(lds_ptr_t)rowacc;

    // The workgroup's unit-quads in walk order are u = step * n_chunks + col; this wave takes u = wave, wave +
    // n_waves, ...  A cursor is the (step, col) of one of them and moves on by n_waves.  su = 4 * step * n_chunks +
    // col: the index of the lane's unit in the workgroup's table slice is su + quarter * n_chunks (out_f is a
    // multiple of four here, so every row quad is whole), which leaves one addition per address to the lanes.
    const uint32_t n_total = n_steps * n_chunks;
    const uint32_t n_mine = wave < n_total ? (n_total - wave + n_waves - 1) / n_waves : 0u;
    const uint32_t dq = n_waves / n_chunks, dr = n_waves - dq * n_chunks;
    struct Cur {
        uint32_t step, col, su;
    };
    auto advance = [&](Cur &c) {
        c.step += dq;
        c.col += dr;
        if (c.col >= n_chunks) {
            c.col -= n_chunks;
            ++c.step;
        }
        c.su = 4 * c.step * n_chunks + c.col;
    };
    Cur c_issue = {wave / n_chunks, wave % n_chunks, 0};
    c_issue.su = 4 * c_issue.step * n_chunks + c_issue.col;
    Cur c_now = c_issue, c_next = c_issue;
    advance(c_next);
    const uint32_t tq1_lane = tq1_addr + quarter * n_chunks * 4;    // LDS address of the lane's row's entries
    const uint32_t b1_lane = (quarter * n_chunks * 16u + li) * 4u;  // bitmap 0: byte offset of the lane's word
    const uint32_t l1_lane = li * 16u;
    const uint32_t xs_lane = xs_addr + li * 16u;

    uint32_t st_issue = 0;  // ring stage the next copy goes to
    auto issue = [&]() {
        const uint32_t q1u = lds_u32(tq1_lane + c_issue.su * 4);
        uint8_t *stage = ring + st_issue * kRStageBytes;
        asm volatile("" ::: "memory");
        if (li < 13)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(l1_rsrc, (lds_ptr_t)stage, 16,
                                                     (int)(((q1u * 3u) >> 5) * 4u + l1_lane), 0, 0, 0);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(b1_rsrc, (lds_ptr_t)(stage + 1024), 4, (int)b1_lane,
                                                 (int)((unit0 + c_issue.su) * 64u), 0, 0);
        st_issue = st_issue + 1 == (uint32_t)kXStages ? 0u : st_issue + 1;
        advance(c_issue);
    };

    uint32_t qcount = 0;  // wave-uniform

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

    // Code window of the unit-quad at cursor c, whose data is in ring stage `st`, spliced once.
    // A lane with elements above level 1 leaves a record: {their bitmap bits, the lane's rank offset inside the
    // unit, the LDS address of the unit's table entry, row slot << 16 | column block << 4 | lane of the row}.
    const uint32_t rec_lane = (quarter << 16) | li;
    auto open_window = [&](uint32_t st, const Cur &c, uint32_t &w0, uint32_t &w1, uint32_t &w2, uint32_t &zrem) {
        const uint32_t ta = tq1_lane + c.su * 4;
        const uint32_t stage = ring_addr + st * kRStageBytes;
        const uint32_t word = lds_u32(stage + 1024 + lane * 4);
        const uint32_t q1u = lds_u32(ta);
        const uint32_t cnt = __popc(word);
        const uint32_t excl = row_scan(cnt) - cnt;
        const uint32_t off = __umul24(excl, 3u) + ((q1u * 3u) & 31u);
        const uint32_t wa = stage + quarter * 256 + (off >> 5) * 4;
        const uint32_t d0 = lds_u32(wa), d1 = lds_u32(wa + 4), d2 = lds_u32(wa + 8), d3 = lds_u32(wa + 12);
        w0 = __builtin_amdgcn_alignbit(d1, d0, off);
        w1 = __builtin_amdgcn_alignbit(d2, d1, off);
        w2 = __builtin_amdgcn_alignbit(d3, d2, off);
        const uint32_t zeros = ~word;
        const uint64_t any = __ballot(zeros != 0);
        if (zeros != 0)
            push_record(queue, qcount + lanes_below(any),
                        make_uint4(zeros, excl, ta, rec_lane + ((c.step << 18) | (c.col << 4))));
        qcount += (uint32_t)__popcll(any);
        zrem = zeros;
        splice_once(w0, w1, w2, zrem);
    };

    auto resolve = [&]() {
        if (ANY)
            resolve_rows<MT, false, true, 1>(P, sv, tq1_addr, tq2_addr, unit0, queue, qcount, rowacc_addr, tasks,
                                               xs_addr, xs_row, 0, m, scale, lane, prefix, entries);
        else if (sv.staged)
            resolve_rows<MT, true, false, 1>(P, sv, tq1_addr, tq2_addr, unit0, queue, qcount, rowacc_addr, tasks,
                                               xs_addr, xs_row, 0, m, scale, lane);
        else
            resolve_rows<MT, false, false, 1>(P, sv, tq1_addr, tq2_addr, unit0, queue, qcount, rowacc_addr, tasks,
                                                xs_addr, xs_row, 0, m, scale, lane);
        qcount = 0;
    };

    if (n_mine > 0) {
        const uint32_t n_pre = min((uint32_t)kXStages, n_mine);
        for (uint32_t i = 0; i < n_pre; ++i) issue();
        if (n_mine >= (uint32_t)kXStages) wait_vmem<2 * (kXStages - 1)>();
        else wait_vmem<0>();

        uint32_t cw0, cw1, cw2, czrem;
        open_window(0, c_now, cw0, cw1, cw2, czrem);
        while (__ballot(czrem != 0) != 0) splice_once(cw0, cw1, cw2, czrem);
        uint32_t st_now = 0;  // ring stage of the unit-quad whose window is open
        const bool long_run = n_total > 4 * n_waves;
        constexpr int NA = MT == 1 ? 4 : (MT == 2 ? 2 : 1);  // independent accumulators per activation row
        float acc[MT][NA];
#pragma unroll
        for (int j = 0; j < MT; ++j)
#pragma unroll
            for (int a = 0; a < NA; ++a) acc[j][a] = 0.0f;

        for (uint32_t i = 0; i < n_mine; ++i) {
            // The waves that share a SIMD take turns at the issue priority (see k_gemv358_rows).  Measured: with more
            // than four unit-quads per wave (and four waves per SIMD) a turn of two unit-quads beats a turn of one by
            // 1-2 %, and turns of three or four; with fewer unit-quads, turns of one handed round in the other
            // direction are 1-2 % better for (3,5,8) and as much worse for the resolver that walks nested bitmaps.
            __builtin_amdgcn_s_setprio(0);
            const uint32_t turn = (MT > 4 ? (wave >> 2) + i
                                   : long_run ? (wave >> 2) + (i >> 1)
                                              : (ANY ? (wave >> 2) + i : (wave >> 2) - i)) & 3u;
            if (turn == 1) __builtin_amdgcn_s_setprio(1);
            else if (turn == 2) __builtin_amdgcn_s_setprio(2);
            else if (turn == 3) __builtin_amdgcn_s_setprio(3);

            // Keep room for a full wave of records.  (A queue of 256 records emptied once, at the end, was 2 % faster
            // where a wave collects 90 records and 20 % slower where it collects 140: what is resolved inside the loop
            // hides behind the other waves' decoding.)
            if (qcount > qcap - kWave) resolve();
            // refill the stage whose window was read last time (it is st_issue); make unit i+1 readable
            if (i + kXStages < n_mine) {
                issue();
                wait_vmem<2 * (kXStages - 1)>();
            } else {
                wait_vmem<0>();
            }

            // this lane's 16 activation pairs of the column block, per activation row
            uint32_t xr[MT][16];
#pragma unroll
            for (int j = 0; j < MT; ++j) {
                const uint32_t xa = xs_lane + (uint32_t)j * xs_row + c_now.col * (kFastChunk * 2);
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const u32x4 v = lds_u128(xa + (uint32_t)t * 256u);
                    xr[j][4 * t] = v.x; xr[j][4 * t + 1] = v.y; xr[j][4 * t + 2] = v.z; xr[j][4 * t + 3] = v.w;
                }
            }

#pragma unroll
            for (int t = 0; t < 16; ++t) {
                const int bit = 6 * t, ob = bit & 31, d = bit >> 5;
                const uint32_t lo = d == 0 ? cw0 : (d == 1 ? cw1 : cw2);
                const uint32_t hi = d == 0 ? cw1 : cw2;
                uint32_t a;  // pair index at bits 12..7
                if (ob > 26) a = __builtin_amdgcn_alignbit(hi, lo, ob - 7);
                else if (ob >= 7) a = lo >> (ob - 7);
                else a = lo << (7 - ob);
                const uint32_t wp = lds_u32((a & 0x1F80u) | lut_lane);
#pragma unroll
                for (int j = 0; j < MT; ++j)
                    acc[j][t % NA] = __builtin_amdgcn_fdot2_f32_bf16(
                        __builtin_bit_cast(bf16x2, wp), __builtin_bit_cast(bf16x2, xr[j][t]), acc[j][t % NA], false);
            }

            // window of this wave's next unit-quad
            const uint32_t st_next = st_now + 1 == (uint32_t)kXStages ? 0u : st_now + 1;
            const bool more = i + 1 < n_mine;
            if (more) {
                uint32_t nzrem;
                open_window(st_next, c_next, cw0, cw1, cw2, nzrem);
                while (__ballot(nzrem != 0) != 0) splice_once(cw0, cw1, cw2, nzrem);
            }

            // the lane's sum stays in its register while the wave's next unit-quad is in the same row quad
            if (!more || c_next.step != c_now.step) {
#pragma unroll
                for (int j = 0; j < MT; ++j) {
                    float sum = acc[j][0];
#pragma unroll
                    for (int a = 1; a < NA; ++a) sum += acc[j][a];
                    const float total = row_sum(sum);
                    if (li == 15) rowacc[(4 * c_now.step + quarter) * MT + j] += total;
#pragma unroll
                    for (int a = 0; a < NA; ++a) acc[j][a] = 0.0f;
                }
            }

            st_now = st_next;
            c_now = c_next;
            advance(c_next);
        }
        __builtin_amdgcn_s_setprio(0);
        resolve();
    }
    __syncthreads();

    // ---- add the waves' row sums in wave order, write bf16 ----
    const uint32_t first_acc = L.waves + kXStages * kRStageBytes + qcap * 16;
    for (uint32_t t = tid; t < rows_here * MT; t += n_threads) {
        const uint32_t slot = t / MT, j = t - slot * MT;
        if ((int)j >= m) continue;
        float sum = 0.0f;
        for (uint32_t w = 0; w < n_waves; ++w)
            sum += *reinterpret_cast<const float *>(smem + first_acc + w * wave_lds_bytes_x(MT, rows_cap, qcap) + t * 4);
        // a workgroup owns whole rows: the one addition per output a split-K caller's fp32 vector takes, or bf16
        if (y32) atomicAdd(&y32[(size_t)j * out_f + row0 + slot], sum);
        else y[(int64_t)j * ldy + row0 + slot] = (uint16_t)f32_to_bf16_bits(sum);
    }
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------

constexpr size_t kLdsLimit = 160 * 1024;

template <int MT, int C, bool ANY>
static int launch_rows(const Dev &P, const int32_t *prefix, uint32_t n_chunks, const uint16_t *x, int m,
                       int64_t ldx, uint16_t *y, int64_t ldy, float *y32, hipStream_t s) {
    const uint32_t waves = (n_chunks + C - 1) / C;
    const uint32_t n_quads = (P.out_f + 3) / 4;
    // how many workgroups a CU holds, by registers and LDS (asked once per workgroup size)
    static int per_cu_cache[17] = {0};
    int per_cu = per_cu_cache[waves];
    if (per_cu == 0) {
        const size_t probe = rows_layout(min(16u, P.out_f), n_chunks, waves, MT, C).total;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, k_gemv358_rows<MT, C, ANY>, (int)(waves * kWave), probe) !=
                hipSuccess || per_cu < 1)
            per_cu = -1;
        per_cu_cache[waves] = per_cu;
    }
    if (per_cu < 1) return IXH_EUNSUPPORTED;
    static const int n_cu = [] {
        int dev = 0, v = 256;
        if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev);
        return v;
    }();
    // whole rounds of resident workgroups, each workgroup with a contiguous run of at most 16 row quads:
    // a last round with a few workgroups in it would cost as much as a full one
    const uint32_t resident = (uint32_t)n_cu * (uint32_t)per_cu;
    const uint32_t rounds = (n_quads + resident * (kRSlots / 4) - 1) / (resident * (kRSlots / 4));
    uint32_t quads = (n_quads + rounds * resident - 1) / (rounds * resident);
    quads = max(1u, min(quads, kRSlots / 4));
    const uint32_t groups = (n_quads + quads - 1) / quads;
    const uint32_t rows_cap = min(quads * 4, P.out_f);
    uint32_t flags = 0;
    if (((uintptr_t)P.last & 3u) == 0) flags |= kFlagStageSide;
    const size_t lds = rows_layout(rows_cap, n_chunks, waves, MT, C).total;
    if (lds > kLdsLimit) return IXH_EUNSUPPORTED;
    if (lds > 64 * 1024) {
        static bool raised = false;  // per instantiation
        if (!raised) {
            if (hipFuncSetAttribute(reinterpret_cast<const void *>(k_gemv358_rows<MT, C, ANY>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsLimit) != hipSuccess)
                return IXH_EUNSUPPORTED;
            raised = true;
        }
    }
    hipLaunchKernelGGL((k_gemv358_rows<MT, C, ANY>), dim3(groups), dim3(waves * kWave), lds, s, P, prefix, n_chunks, quads,
                       flags, x, m, ldx, y, ldy, y32);
    return hipGetLastError() == hipSuccess ? IXH_OK : IXH_ELAUNCH;
}

// The shared-x kernel: as many waves as LDS allows (16, 12 or 8); IXH_EUNSUPPORTED when the activation rows do not
// fit beside them.
template <int MT, bool ANY>
static int launch_rowsx(const Dev &P, const int32_t *prefix, uint32_t n_chunks, const uint16_t *x, int m, int64_t ldx,
                        uint16_t *y, int64_t ldy, float *y32, hipStream_t s) {
    const uint32_t n_quads = (P.out_f + 3) / 4;
    static const int n_cu = [] {
        int dev = 0, v = 256;
        if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev);
        return v;
    }();
    static const bool raised =  // per instantiation
        hipFuncSetAttribute(reinterpret_cast<const void *>(k_gemv358_rowsx<MT, ANY>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsLimit) == hipSuccess;
    if (!raised) return IXH_EUNSUPPORTED;
    // the answers for the last few shapes are kept (a model asks for the same handful over and over), under a
    // lock: a torn entry would launch one shape with another one's LDS layout
    struct Plan {
        uint32_t chunks, out_f, waves, quads;
    };
    static Plan plans[8] = {};
    static uint32_t next_plan = 0;
    static std::mutex plans_lock;
    uint32_t k_waves = 0, k_quads = 0;
    {
        std::lock_guard<std::mutex> guard(plans_lock);
        const Plan *hit = nullptr;
        for (const Plan &pl : plans)
            if (pl.chunks == n_chunks && pl.out_f == P.out_f) hit = &pl;
        if (!hit) {
            uint32_t waves = 0, quads = 0;
            for (uint32_t w : {16u, 12u, 8u}) {
                if (MT > 4 && w > (uint32_t)kXMaxWaves / 2) continue;
                const size_t probe = rowsx_layout(min(16u, P.out_f), n_chunks, w, MT, kRQueue).total;
                int per_cu = 0;
                if (probe > kLdsLimit ||
                    hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, k_gemv358_rowsx<MT, ANY>, (int)(w * kWave),
                                                                 probe) != hipSuccess || per_cu < 1)
                    continue;
                // Whole rounds of resident workgroups, as few as LDS admits (every round pays the set-up, the last
                // resolve and the final sums again: 17408 x 5120 in two rounds of 9 row quads took 22.4 us, in one of
                // 17 it takes 19), each workgroup with a contiguous run of at most kXSlots / 4 row quads.
                uint32_t q = 0;
                for (uint32_t rounds = 1; rounds <= 64 && q == 0; ++rounds) {
                    uint32_t groups_at_once = (uint32_t)n_cu * (uint32_t)per_cu;
                    uint32_t cand = max(1u, (n_quads + rounds * groups_at_once - 1) / (rounds * groups_at_once));
                    size_t total = rowsx_layout(min(cand * 4, P.out_f), n_chunks, w, MT, kRQueue).total;
                    if (per_cu > 1 && total * (size_t)per_cu > kLdsLimit) {  // fewer of these fit a CU than of the probe
                        groups_at_once = (uint32_t)n_cu * (uint32_t)max((size_t)1, kLdsLimit / max(total, (size_t)1));
                        cand = max(1u, (n_quads + rounds * groups_at_once - 1) / (rounds * groups_at_once));
                        total = rowsx_layout(min(cand * 4, P.out_f), n_chunks, w, MT, kRQueue).total;
                    }
                    if (cand <= kXSlots / 4 && total <= kLdsLimit) q = cand;
                }
                if (q == 0) continue;
                waves = w;
                quads = q;
                break;
            }
            Plan &slot = plans[next_plan++ % 8u];
            slot = Plan{n_chunks, P.out_f, waves, quads};
            hit = &slot;
        }
        k_waves = hit->waves;
        k_quads = hit->quads;
    }
    if (k_waves == 0) return IXH_EUNSUPPORTED;
    const uint32_t waves = k_waves, quads = k_quads;
    const uint32_t groups = (n_quads + quads - 1) / quads;
    uint32_t flags = 0;
    if (((uintptr_t)P.last & 3u) == 0) flags |= kFlagStageSide;
    const size_t lds = rowsx_layout(min(quads * 4, P.out_f), n_chunks, waves, MT, kRQueue).total;
    // the launch geometry in one word: column blocks (12 bits), row quads per workgroup (8), waves (5), activation rows
    // (4), flags (3)
    if (n_chunks > 0xFFFu || quads > 0xFFu || waves > 0x1Fu || m > 0xF || flags > 7u) return IXH_EUNSUPPORTED;
    const uint32_t geometry = n_chunks | (quads << 12) | (waves << 20) | ((uint32_t)m << 25) | (flags << 29);
    hipLaunchKernelGGL((k_gemv358_rowsx<MT, ANY>), dim3(groups), dim3(waves * kWave), lds, s, prefix, x, P.scale, ldx,
                       P.bm[0], P.st[0], P.out_f, geometry, P, y, ldy, y32);
    return hipGetLastError() == hipSuccess ? IXH_OK : IXH_ELAUNCH;
}

// Row-block kernel for the shapes whose x slices fit the register budget of a
// full workgroup; IXH_EUNSUPPORTED sends the caller to the column kernel.
int launch_gemv_358_rows(const Dev &P, const int32_t *prefix, const uint16_t *x, int m, int64_t ldx, uint16_t *y,
                         int64_t ldy, float *y32, hipStream_t s) {
    const bool any = !(P.n_levels == 3 && P.bits[1] == 5);  // not (3,5,8): the resolver that walks the nested bitmaps
    if (((uintptr_t)x & 15u) != 0 || (m > 1 && (ldx & 7) != 0)) return IXH_EUNSUPPORTED;
    const uint32_t n_chunks = P.in_f / kFastChunk;
    if (m <= 4) {  // products on the matrix pipe (ixh_slots358.hip)
        const int rc = launch_gemv_358_slots(P, prefix, x, m, ldx, y, ldy, y32, s);
        if (rc != IXH_EUNSUPPORTED) return rc;
    }
    // option "gemv_shared_x" (ixh_set_option): 0 = never the shared-x kernel, 1 = for one activation row only, 2 = up
    // to two rows, 4 = up to four, 8 = up to eight (default)
    const int shared_x = g_opt_gemv_shared_x.load(std::memory_order_relaxed);
    if (shared_x && P.in_f <= 65536u && P.out_f % 4u == 0 && (m == 1 || (m == 2 && shared_x >= 2) || (m <= 4 && shared_x >= 4) || (m <= 8 && shared_x >= 8))) {
        int rc;
        if (m == 1) rc = any ? launch_rowsx<1, true>(P, prefix, n_chunks, x, m, ldx, y, ldy, y32, s) : launch_rowsx<1, false>(P, prefix, n_chunks, x, m, ldx, y, ldy, y32, s);
        else if (m == 2) rc = any ? launch_rowsx<2, true>(P, prefix, n_chunks, x, m, ldx, y, ldy, y32, s) : launch_rowsx<2, false>(P, prefix, n_chunks, x, m, ldx, y, ldy, y32, s);
        else if (m <= 4) rc = any ? launch_rowsx<4, true>(P, prefix, n_chunks, x, m, ldx, y, ldy, y32, s) : launch_rowsx<4, false>(P, prefix, n_chunks, x, m, ldx, y, ldy, y32, s);
        else rc = any ? launch_rowsx<8, true>(P, prefix, n_chunks, x, m, ldx, y, ldy, y32, s) : launch_rowsx<8, false>(P, prefix, n_chunks, x, m, ldx, y, ldy, y32, s);
        if (rc != IXH_EUNSUPPORTED) return rc;
    }
    const uint32_t c = (n_chunks + kRMaxWaves - 1) / kRMaxWaves;  // blocks per wave: a workgroup has at most kRMaxWaves waves
    if (m > 4) return IXH_EUNSUPPORTED;  // five to eight rows: the shared-x kernel above or nothing
    const int mt = m == 1 ? 1 : (m == 2 ? 2 : 4);
#define IXH_ROWS(MTV, CV) \
    if (mt == MTV && c == CV)                                                                  \
        return any ? launch_rows<MTV, CV, true>(P, prefix, n_chunks, x, m, ldx, y, ldy, y32, s)     \
                   : launch_rows<MTV, CV, false>(P, prefix, n_chunks, x, m, ldx, y, ldy, y32, s);
    IXH_ROWS(1, 1) IXH_ROWS(1, 2) IXH_ROWS(1, 3) IXH_ROWS(1, 4)
    IXH_ROWS(2, 1) IXH_ROWS(2, 2)
    IXH_ROWS(4, 1)
#undef IXH_ROWS
    return IXH_EUNSUPPORTED;
}

}  // namespace ixh
