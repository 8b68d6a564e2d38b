// (3,5,8) fused decode + GEMV for gfx950, slot variant: the row-block kernel's decode (ixh_rows358.hip) with the
// products on the matrix pipe, for one to four activation rows and tensors that are almost all level 1.
//
// Work split.  As in k_gemv358_rowsx a workgroup owns whole row quads, holds the activation rows in LDS (swizzled
// copy) and deals its unit-quads (4 rows x one 512-wide column block, u = row quad * n_chunks + column block) to its
// waves, here four at a time: a group is unit-quads 4g .. 4g + 3, i.e. 16 (row, column block) pairs, the slots.
// Slot n = r + 4 s is row r of unit-quad 4g + s.  Lane (n, kg), n = lane % 16, kg = lane / 16, decodes the words
// 2 kg, 2 kg + 1 (first half of the unit) and 8 + 2 kg, 9 + 2 kg (second half) of slot n: a lane walks 64 consecutive
// columns per half, so the rank of a word is the rank of its predecessor plus a popcount, and what crosses lanes is one
// exclusive sum over the four k groups per unit (two v_permlane swaps), against a four-step scan per word.
//
// Products.  v_mfma_f32_16x16x32_bf16: the eight weights a lane gets from four pair-table reads are column n, k group
// kg of the one operand; the other operand's row a = 4 j + s is activation row j at the columns of the group's
// unit-quad s (read by lanes n < 4 m only, 16 bytes each), so D[4 j + s][n] is the sum of slot n where s is n's own
// unit-quad.  A word costs four matrix instructions and no vector multiply; the sums never leave the accumulators
// until the group ends.
//
// Memory pipeline.  The codes of a half (256 columns of 16 slots, at most 104 bytes each) are staged by two LDS-DMA
// instructions (seven 16-byte pieces a slot, 56 lanes) into a stage of 1792 bytes; two stages, one per half, so the
// copy of the next half is in flight while this one is decoded.  Slots are 112 bytes apart: the 16 lanes of a k
// group read the same dword index of their slots, and 28 dwords between them spread those reads over the LDS banks.
// The first half's stream position follows from the rank table alone; the second half's is the first's plus the
// level-1 count of the first half, known from the bitmap words, which are loaded into registers one group ahead.
// The copy lanes get their slot's position through ds_bpermute.  A group's ranks, records and second-half request are
// worked out at the end of the group before it (the first group's before the workgroup's barrier, which orders LDS
// only, so the copies asked for ahead of it stay in flight).
//
// Two properties of the hardware that the waits are built around: copies into LDS complete in the order of their
// issue, but not in order with loads into registers, so a counted wait (vmcnt(n), n > 0) is only ever used with
// nothing but copies in flight; and a vector-memory instruction must not read a scalar register within five states
// of a vector instruction writing it, which the compiler guarantees for its own instructions only (the bitmap words
// are loaded by raw instructions, so that the compiler does not wait for them, and for every copy in flight, at
// their first use).
//
// Everything else (pair table, splice, resolver of the elements above level 1, final sums) is the row-block
// kernel's; the records are 8 bytes (ixh_rows_common.h, XL == 3).
#include <math.h>
#include <stdlib.h>

#include <mutex>

#include "ixh_rows_common.h"

namespace ixh {

// ixh_set_option("gemv_slots"): -1 = never this kernel, 0 = where it is the fastest (default), 1 = wherever it fits
std::atomic<int> g_opt_gemv_slots{0};
// ixh_set_option("gemv_slot_waves"): waves per workgroup, 0 = the planner's choice
std::atomic<int> g_opt_gemv_slot_waves{0};

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2s __attribute__((ext_vector_type(2)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int kSMaxWaves = 16;
constexpr uint32_t kSRows = 128;          // rows per workgroup at most
constexpr uint32_t kSSlotBytes = 112;     // staged bytes of a slot's half: seven 16-byte pieces
constexpr uint32_t kSStageBytes = 16 * kSSlotBytes;
constexpr size_t kSLdsLimit = 160 * 1024;

// a wave's region: two stages, record queue (qcap records), row sums, task list
__host__ __device__ constexpr uint32_t wave_lds_bytes_s(int mt, uint32_t rows_cap, uint32_t qcap) {
    return 2 * kSStageBytes + qcap * 8 + ((rows_cap * (uint32_t)mt * 4 + 15u) & ~15u) + kRTasks2 * 2;
}

struct SlotsLds {
    uint32_t tq1, tq2, side, xs, waves, total;
};

__host__ __device__ inline SlotsLds slots_layout(uint32_t rows_cap, uint32_t n_chunks, uint32_t n_waves, int mt,
                                                 uint32_t qcap) {
    SlotsLds L;
    const uint32_t tbl = ((rows_cap * n_chunks + 1u + 3u) & ~3u) * 4u;
    L.tq1 = kRLutBytes + kRSpliceBytes;
    L.tq2 = L.tq1 + tbl;
    L.side = L.tq2 + tbl;
    L.xs = L.side + kRSideBytes;
    L.waves = L.xs + (uint32_t)mt * n_chunks * kSkewedBlock;
    L.total = L.waves + n_waves * wave_lds_bytes_s(mt, rows_cap, qcap);
    return L;
}

template <int MT, bool ANY>
__global__ void __launch_bounds__(kSMaxWaves * kWave)
k_gemv358_slots(Dev P, const int32_t *__restrict__ prefix, uint32_t n_chunks, uint32_t quads_per_wg, uint32_t flags,
                uint32_t qcap, uint32_t inv_chunks, const uint16_t *__restrict__ x, int m, int64_t ldx,
                uint16_t *__restrict__ y, int64_t ldy, float *__restrict__ y32) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const uint32_t n_waves = blockDim.x >> 6;
    const uint32_t quarter = lane >> 4, li = lane & 15;  // the set-up's copy lanes (as in k_gemv358_rowsx)
    const uint32_t n = lane & 15u, kg = lane >> 4, r = n & 3u, s = n >> 2;

    const uint32_t n_quads = (P.out_f + 3) >> 2;
    const uint32_t quad0 = blockIdx.x * quads_per_wg;
    const uint32_t n_steps = min(quads_per_wg, n_quads - quad0);
    const uint32_t row0 = quad0 * 4;
    const uint32_t rows_here = min(n_steps * 4, P.out_f - row0);
    const uint32_t rows_cap = min(quads_per_wg * 4, P.out_f);
    const SlotsLds L = slots_layout(rows_cap, n_chunks, n_waves, MT, qcap);

    // the pair table is addressed with (index bits | lane bits): it must sit at LDS address 0
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
    const uint32_t wave_bytes = wave_lds_bytes_s(MT, rows_cap, qcap);
    uint8_t *const wave_base = smem + L.waves + wave * wave_bytes;
    uint8_t *const stages = wave_base;
    uint4 *const queue = reinterpret_cast<uint4 *>(wave_base + 2 * kSStageBytes);
    float *const rowacc = reinterpret_cast<float *>(wave_base + 2 * kSStageBytes + qcap * 8);
    uint16_t *const tasks = reinterpret_cast<uint16_t *>(wave_base + wave_bytes - kRTasks2 * 2);
    const uint16_t scale_bits = *P.scale;
    const uint32_t unit0 = row0 * n_chunks;
    const uint32_t entries = P.out_f * n_chunks + 1;
    const uint32_t tq1_addr = L.tq1, tq2_addr = L.tq2;
    const uint32_t stages_addr = (uint32_t)(uintptr_t)(lds_ptr_t)stages;
    const uint32_t xs_addr = L.xs, xs_row = n_chunks * kSkewedBlock;  // bytes between activation rows
    const uint32_t rowacc_addr = (uint32_t)(uintptr_t)(lds_ptr_t)rowacc;
    const __amdgpu_buffer_rsrc_t l1_rsrc =
        __builtin_amdgcn_make_buffer_rsrc((void *)P.st[0], 0, (int)(P.st_words[0] * 4u), 0x00020000);

    // ---- the walk: this wave takes the groups wave, wave + n_waves, ...  (inv_chunks = ceil(2^32 / n_chunks), so
    // that the few divisions by n_chunks are one multiplication each; the operands stay far below 2^16) ----
    auto div_chunks = [&](uint32_t v) { return n_chunks == 1u ? v : __umulhi(v, inv_chunks); };
    const uint32_t n_total = n_steps * n_chunks;  // unit-quads of the workgroup
    const uint32_t n_groups = (n_total + 3u) >> 2;
    uint32_t n_mine = 0;
    for (uint32_t g = wave; g < n_groups; g += n_waves) ++n_mine;  // scalar, a few rounds
    const uint32_t du = 4u * n_waves, dq = div_chunks(du), dr = du - dq * n_chunks;
    // a lane's cursor: the unit-quad of its slot, as (row quad, column block); one past the end stays there and is
    // clamped to the workgroup's last unit-quad wherever it is turned into an address
    struct Cur {
        uint32_t u, step, col;
    };
    auto advance = [&](Cur &c) {
        c.u += du;
        c.step += dq;
        c.col += dr;
        if (c.col >= n_chunks) {
            c.col -= n_chunks;
            ++c.step;
        }
    };
    Cur cur;
    cur.u = 4u * wave + s;
    cur.step = div_chunks(cur.u);
    cur.col = cur.u - cur.step * n_chunks;
    // the column block whose activations this lane feeds to the matrix instruction: that of unit-quad 4g + (n % 4)
    uint32_t colx = 4u * wave + r;
    colx -= div_chunks(colx) * n_chunks;
    const bool x_lane = n < 4u * (uint32_t)m;
    const uint32_t x_base = xs_addr + (n >> 2) * xs_row + kg * 32u;  // + column block * kSkewedBlock + word offset
    const uint32_t idx_last = (4u * (n_steps - 1u) + r) * n_chunks + n_chunks - 1u;
    auto index_of = [&](const Cur &c) {  // index of the lane's (row, column block) in the table slice
        return c.u < n_total ? (4u * c.step + r) * n_chunks + c.col : idx_last;
    };
    // bitmap words of the lane's strip: .x .y first half, .z .w second half
    // (Raw instructions: the compiler does not know of these loads and puts no wait of its own in front of their
    // first use, which would also wait for every copy then in flight; the waits are the hand-counted ones below,
    // each followed by arrived(), through which the registers reach their users.)
    const u32x4 b1_desc = {(uint32_t)(uintptr_t)P.bm[0], (uint32_t)((uintptr_t)P.bm[0] >> 32) & 0xFFFFu,
                           P.bm_words[0] * 4u, 0x00020000u};  // base, stride 0, bytes, raw dword access
    auto load_words = [&](uint32_t index, u32x2 &lo, u32x2 &hi) {
        const uint32_t at = (unit0 + index) * 64u + kg * 8u;
        // (s_nop 4: the descriptor may have been moved into its scalar registers by the vector unit just before, and a
        // vector-memory instruction must not read such a register within five states; the compiler keeps that
        // distance for its own instructions, not for these)
        asm volatile("s_nop 4\n\tbuffer_load_dwordx2 %0, %2, %3, 0 offen\n\tbuffer_load_dwordx2 %1, %2, %3, 0 offen offset:32"
                     : "+v"(lo), "+v"(hi)  // in-out: the registers of the caller's variables, no copy behind the loads
                     : "v"(at), "s"(b1_desc)
                     : "memory");
    };
    auto arrived = [&](u32x2 &lo, u32x2 &hi) { asm volatile("" : "+v"(lo), "+v"(hi)); };

    // copy lanes: lane l < 56 fetches piece l % 7 of slot l / 7 (first instruction) or 8 + l / 7 (second)
    const uint32_t dma_slot = (lane * 37u) >> 8;
    const uint32_t dma_src0 = dma_slot * 4u, dma_src1 = dma_src0 + 32u;
    const uint32_t dma_piece = (lane - dma_slot * 7u) * 16u;
    const bool dma_lane = lane < 56u;
    // where a lane finds its slot in a stage
    const uint32_t slot_addr = stages_addr + n * kSSlotBytes;
    // Issue the copy of a half: `rank` is the number of level-1 elements before the half's first (the same in every
    // lane of a slot).  Returns the LDS address of the dword that holds the half's first code bit.
    auto issue_codes = [&](uint32_t rank, uint32_t stage) -> uint32_t {
        const uint32_t first = ((rank * 3u) >> 5) * 4u;  // byte offset of the slot's staged region in the stream
        const uint32_t a0 = (uint32_t)__builtin_amdgcn_ds_bpermute((int)dma_src0, (int)first);
        const uint32_t a1 = (uint32_t)__builtin_amdgcn_ds_bpermute((int)dma_src1, (int)first);
        uint8_t *const st = stages + stage * kSStageBytes;
        asm volatile("" ::: "memory");
        if (dma_lane) {
            __builtin_amdgcn_raw_ptr_buffer_load_lds(l1_rsrc, (lds_ptr_t)st, 16, (int)(a0 + dma_piece), 0, 0, 0);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(l1_rsrc, (lds_ptr_t)(st + 8 * kSSlotBytes), 16, (int)(a1 + dma_piece), 0, 0, 0);
        }
        return slot_addr + stage * kSStageBytes;
    };

    // ---- requests that need nothing but the arguments: the activation rows (a copy into LDS: lane (t, l) fetches
    // piece l * 4 + t of a column block and the hardware puts it at piece t * 16 + l), and into registers the first
    // group's bitmap words and table entry and this thread's entries of the table slices.  Copies into LDS and loads
    // into registers do not complete in order with each other: they are waited for together, with vmcnt(0) ----
    {
        const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc(
            (void *)x, 0, (int)((((int64_t)(m - 1) * ldx + P.in_f) * 2)), 0x00020000);
        for (uint32_t t = wave; t < (uint32_t)m * n_chunks; t += n_waves) {
            const uint32_t j = div_chunks(t), col = t - j * n_chunks;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(
                x_rsrc, (lds_ptr_t)(smem + L.xs + (j * n_chunks + col) * kSkewedBlock), 16,
                (int)(((int64_t)j * ldx + col * kFastChunk) * 2 + (li * 4u + quarter) * 16u), 0, 0, 0);
        }
    }
    uint32_t idx = index_of(cur);
    u32x2 bw_lo = {0u, 0u}, bw_hi = {0u, 0u};
    load_words(idx, bw_lo, bw_hi);
    uint32_t q1u = (uint32_t)prefix[unit0 + idx];
    const uint32_t n_local = rows_here * n_chunks;
    const uint32_t n_tbl = n_local + 1u;
    const uint32_t tbl_i = min(tid, n_local);
    const uint32_t tbl_1 = (uint32_t)prefix[unit0 + tbl_i];
    const uint32_t tbl_2 = ANY ? 0u : (uint32_t)prefix[entries + unit0 + tbl_i];
    // the ranks at the ends of the workgroup's rows: what its share of the side streams is worked out from
    uint32_t q1b = 0, q2b = 0, q1e = 0, q2e = 0;
    if (!ANY) {
        q1b = (uint32_t)prefix[unit0], q2b = (uint32_t)prefix[entries + unit0];
        q1e = (uint32_t)prefix[unit0 + n_local], q2e = (uint32_t)prefix[entries + unit0 + n_local];
    }

    // ---- what needs no memory: pair table, splice masks, row sums ----
    const float scale = bf16_bits_to_f32(scale_bits);
    for (uint32_t i = tid; i < 64 * 32; i += blockDim.x) {
        const int c0 = (i >> 5) & 7, c1 = i >> 8;
        const f32x2s w = {c0 < 7 ? (float)(c0 - 3) * scale : 0.0f, c1 < 7 ? (float)(c1 - 3) * scale : 0.0f};
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
    wait_vmem<0>();  // this wave's pieces of the activation rows are in LDS, the rest in registers
    // (a use the compiler can see: it puts its own wait for these registers here, where it costs nothing, and not in
    // front of their first real use, behind copies that are then in flight)
    arrived(bw_lo, bw_hi);
    uint32_t tbl_1v = tbl_1, tbl_2v = tbl_2, scale_v = scale_bits;
    asm volatile("" : "+v"(q1u), "+v"(tbl_1v), "+v"(tbl_2v), "+v"(scale_v));
    // ---- the table slices ----
    if (tid < n_tbl) {
        tq1[tid] = tbl_1v;
        if (!ANY) tq2[tid] = tbl_2v;
    }
    for (uint32_t i = tid + blockDim.x; i < n_tbl; i += blockDim.x) {
        tq1[i] = (uint32_t)prefix[unit0 + i];
        if (!ANY) tq2[i] = (uint32_t)prefix[entries + unit0 + i];
    }
    wait_vmem<0>();

    // ---- the other copies into LDS, asked for now that nothing else is in flight (copies complete in the order of
    // their issue, which is what the counted waits below rely on): the workgroup's share of the side streams, the
    // first group's halves ----
    // this workgroup's share of bitmap 1 and of the 5-bit / 8-bit streams (as in k_gemv358_rows); every wave copies
    // it, so that it needs no barrier of its own
    SideView sv;
    sv.staged = false;
    if (!ANY) {
        const uint32_t nl1b = row0 * P.in_f - q1b, nl1e = (row0 + rows_here) * P.in_f - q1e;
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
    uint32_t region0 = 0;
    if (n_mine > 0) region0 = issue_codes(q1u, 0);

    const uint32_t lut_lane = (lane & 31u) << 2;
    const uint32_t splice_addr = kRLutBytes;

    uint32_t qcount = 0;  // wave-uniform

    auto splice_once = [&](uint32_t &w0, uint32_t &w1, uint32_t &w2, uint32_t &zrem) __attribute__((always_inline)) {
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

    auto resolve = [&]() __attribute__((always_inline)) {
        if (qcount == 0) return;
        const TaskPool none{0, 0, 0, 1, 0, 0};
        // The resolvers that read global memory wait for their loads with counts the compiler works out, and copies
        // into LDS do not complete in order with loads into registers: nothing may be in flight when they start.
        if (ANY || !sv.staged) wait_vmem<0>();
        if (ANY)
            resolve_rows<MT, false, true, 3>(P, sv, tq1_addr, tq2_addr, unit0, queue, qcount, rowacc_addr, tasks,
                                               xs_addr, xs_row, 0, m, scale, lane, prefix, entries, none, n_chunks);
        else if (sv.staged)
            resolve_rows<MT, true, false, 3>(P, sv, tq1_addr, tq2_addr, unit0, queue, qcount, rowacc_addr, tasks,
                                               xs_addr, xs_row, 0, m, scale, lane, nullptr, 0, none, n_chunks);
        else
            resolve_rows<MT, false, false, 3>(P, sv, tq1_addr, tq2_addr, unit0, queue, qcount, rowacc_addr, tasks,
                                                xs_addr, xs_row, 0, m, scale, lane, nullptr, 0, none, n_chunks);
        qcount = 0;
    };

    f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};  // D[4 kg + t][n]: activation row kg at the columns of unit-quad t x slot n

    // the sixteen pairs of a spliced window through the pair table, and the word's four matrix instructions
    auto multiply = [&](uint32_t w0, uint32_t w1, uint32_t w2, const u32x4 (&xa)[4]) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint32_t wp[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int bit = 6 * (4 * i + q), ob = bit & 31, d = bit >> 5;
                const uint32_t lo = d == 0 ? w0 : (d == 1 ? w1 : w2);
                const uint32_t hi = d == 0 ? w1 : w2;
                uint32_t a;  // pair index at bits 12..7
                if (ob > 26) a = __builtin_amdgcn_alignbit(hi, lo, ob - 7);
                else if (ob >= 7) a = lo >> (ob - 7);
                else a = lo << (7 - ob);
                wp[q] = lds_u32((a & 0x1F80u) | lut_lane);
            }
            const u32x4 b4 = u32x4{wp[0], wp[1], wp[2], wp[3]};
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, xa[i]),
                                                         __builtin_bit_cast(bf16x8, b4), acc, 0, 0, 0);
        }
    };

    // One half of a group, two words per lane: bitmap words wa / wb, code bits offa / offb from the first staged dword
    // at `region`, the lane's activations of the first word at xw (the second word's are 16 bytes on).  Both windows
    // are opened and spliced before the first pair is looked up, so that a lane's trips to LDS overlap.
    u32x4 xa[4], xb[4];  // lanes that feed no activations keep zeros
#pragma unroll
    for (int i = 0; i < 4; ++i) xa[i] = xb[i] = u32x4{0u, 0u, 0u, 0u};
    auto do_half = [&](uint32_t wa, uint32_t wb, uint32_t region, uint32_t offa, uint32_t offb, uint32_t xw)
                       __attribute__((always_inline)) {
        const uint32_t aa = region + ((offa >> 3) & ~3u), ab = region + ((offb >> 3) & ~3u);
        const uint32_t a0 = lds_u32(aa), a1 = lds_u32(aa + 4), a2 = lds_u32(aa + 8), a3 = lds_u32(aa + 12);
        const uint32_t b0 = lds_u32(ab), b1 = lds_u32(ab + 4), b2 = lds_u32(ab + 8), b3 = lds_u32(ab + 12);
        if (x_lane) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                xa[i] = lds_u128(xw + (uint32_t)i * 256u);
                xb[i] = lds_u128(xw + 16u + (uint32_t)i * 256u);
            }
        }
        uint32_t u0 = __builtin_amdgcn_alignbit(a1, a0, offa);
        uint32_t u1 = __builtin_amdgcn_alignbit(a2, a1, offa);
        uint32_t u2 = __builtin_amdgcn_alignbit(a3, a2, offa);
        uint32_t v0 = __builtin_amdgcn_alignbit(b1, b0, offb);
        uint32_t v1 = __builtin_amdgcn_alignbit(b2, b1, offb);
        uint32_t v2 = __builtin_amdgcn_alignbit(b3, b2, offb);
        uint32_t za = ~wa, zb = ~wb;
        splice_once(u0, u1, u2, za);
        splice_once(v0, v1, v2, zb);
        while (__ballot((za | zb) != 0) != 0) {  // lanes with more than one element above level 1 in a word (rare)
            splice_once(u0, u1, u2, za);
            splice_once(v0, v1, v2, zb);
        }
        multiply(u0, u1, u2, xa);
        multiply(v0, v1, v2, xb);
    };

    // What a group needs of its unit's bitmap words, worked out one group ahead (prepare): ranks, records, the request
    // for its second half and for the next group's bitmap words.
    struct Group {
        u32x4 words;
        uint32_t p0, p2;      // level-1 elements of the first word of each half
        uint32_t off0, off1;  // code bit of each half's first word, from the first staged dword
        uint32_t region1;     // where the second half is staged
        uint32_t row_addr;    // LDS address of the lane's row sum (activation row kg)
        uint32_t xw;          // LDS address of the lane's activations of the first word
        bool live;
    };
    Cur nxt = cur;     // the group after the one prepared last
    uint32_t idx_n = 0;
    auto prepare = [&](const Cur c, uint32_t q1u_c, u32x4 words) __attribute__((always_inline)) -> Group {
        Group g;
        g.live = c.u < n_total;
        // a slot past the end: no records; its sums are dropped
        if (!g.live) words = u32x4{~0u, ~0u, ~0u, ~0u};
        g.words = words;
        // ---- the unit's ranks: level-1 counts of the lane's two strips, exclusive sums over the k groups ----
        const uint32_t p0 = (uint32_t)__popc(words.x), p01 = p0 + (uint32_t)__popc(words.y);
        const uint32_t p2 = (uint32_t)__popc(words.z), p23 = p2 + (uint32_t)__popc(words.w);
        const uint32_t both = p01 | (p23 << 16);
        const auto sw16 = __builtin_amdgcn_permlane16_swap(both, both, false, false);
        const uint32_t pairs = sw16[0] + sw16[1];
        const auto sw32 = __builtin_amdgcn_permlane32_swap(pairs, pairs, false, false);
        const uint32_t excl = ((kg & 1u) ? sw16[0] : 0u) + ((kg & 2u) ? sw32[0] : 0u);
        const uint32_t total = sw32[0] + sw32[1];
        const uint32_t half0 = total & 0xFFFFu;  // level-1 elements of the unit's first half
        const uint32_t ones0 = excl & 0xFFFFu, ones2 = half0 + (excl >> 16);
        const uint32_t rank1 = q1u_c + half0;
        g.p0 = p0;
        g.p2 = p2;
        g.off0 = ((q1u_c * 3u) & 31u) + ones0 * 3u;
        g.off1 = ((rank1 * 3u) & 31u) + (excl >> 16) * 3u;
        g.row_addr = rowacc_addr + ((4u * c.step + r) * MT + kg) * 4u;
        g.xw = x_base + __umul24(colx, kSkewedBlock);
        // ---- the group's records: a lane's word with elements above level 1 leaves {its zero bits, level-1
        // elements of the unit before it | word << 9 | column block << 13 | row << 20} ----
        {
            const uint32_t z0 = ~words.x, z1 = ~words.y, z2 = ~words.z, z3 = ~words.w;
            const uint64_t m0 = __ballot(z0 != 0), m1 = __ballot(z1 != 0), m2 = __ballot(z2 != 0), m3 = __ballot(z3 != 0);
            const uint32_t c0 = (uint32_t)__popcll(m0), c1 = (uint32_t)__popcll(m1), c2 = (uint32_t)__popcll(m2),
                           c3 = (uint32_t)__popcll(m3);
            if (c0 + c1 + c2 + c3 != 0) {
                if (qcount + c0 + c1 + c2 + c3 > qcap) resolve();
                const uint32_t meta = ((4u * c.step + r) << 20) | (c.col << 13) | (kg << 10);
                if (z0 != 0) push_record8(queue, qcount + lanes_below(m0), z0, meta | ones0);
                qcount += c0;
                if (z1 != 0) push_record8(queue, qcount + lanes_below(m1), z1, meta | (1u << 9) | (ones0 + p0));
                qcount += c1;
                if (z2 != 0) push_record8(queue, qcount + lanes_below(m2), z2, meta | (8u << 9) | ones2);
                qcount += c2;
                if (z3 != 0) push_record8(queue, qcount + lanes_below(m3), z3, meta | (9u << 9) | (ones2 + p2));
                qcount += c3;
            }
        }
        // ---- request: this group's second half ----
        g.region1 = issue_codes(rank1, 1);
        nxt = c;
        advance(nxt);
        colx += dr;
        if (colx >= n_chunks) colx -= n_chunks;
        return g;
    };

    if (n_mine > 0) {
        Group g = prepare(cur, q1u, u32x4{bw_lo.x, bw_lo.y, bw_hi.x, bw_hi.y});
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");  // LDS only: the copies stay in flight
        for (uint32_t i = 0; i < n_mine; ++i) {
            __builtin_amdgcn_s_setprio(0);
            const uint32_t turn = ((wave >> 2) + i) & 3u;
            if (turn == 1) __builtin_amdgcn_s_setprio(1);
            else if (turn == 2) __builtin_amdgcn_s_setprio(2);
            else if (turn == 3) __builtin_amdgcn_s_setprio(3);
            const bool more = i + 1 < n_mine;

            // ---- first half (behind it in flight: the second half).  Counted waits only ever have copies into LDS
            // behind them: those complete in the order of their issue, but not in order with loads into registers,
            // so the next group's bitmap words are asked for here and waited for with everything else below ----
            wait_vmem<2>();
            if (more) {
                idx_n = index_of(nxt);
                load_words(idx_n, bw_lo, bw_hi);
            }
            do_half(g.words.x, g.words.y, region0, g.off0, g.off0 + g.p0 * 3u, g.xw);

            // ---- request: the next group's first half ----
            // (behind the second half in flight: the next group's bitmap words; waiting for them here, where the
            // second half is needed anyway, keeps the compiler's wait for them from landing behind the next request)
            uint32_t q1u_n = 0;
            wait_vmem<0>();
            if (more) {
                arrived(bw_lo, bw_hi);
                q1u_n = lds_u32(tq1_addr + idx_n * 4u);
                region0 = issue_codes(q1u_n, 0);
            }

            // ---- second half ----
            do_half(g.words.z, g.words.w, g.region1, g.off1, g.off1 + g.p2 * 3u, g.xw + 128u);

            // ---- the group's sums leave the accumulators: activation row kg of slot n is D[4 kg + s][n] ----
            {
                const float v = s == 0 ? acc[0] : (s == 1 ? acc[1] : (s == 2 ? acc[2] : acc[3]));
                if (g.live && kg < (uint32_t)m) lds_add_f32_raw(g.row_addr, v);
                acc = f32x4{0.f, 0.f, 0.f, 0.f};
            }
            // ---- the next group's ranks and records, its second half's request ----
            if (more) g = prepare(nxt, q1u_n, u32x4{bw_lo.x, bw_lo.y, bw_hi.x, bw_hi.y});
        }
        __builtin_amdgcn_s_setprio(0);
        resolve();
    } else {
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __syncthreads();

    // ---- add the waves' row sums in wave order, write bf16 ----
    const uint32_t first_acc = L.waves + 2 * kSStageBytes + qcap * 8;
    for (uint32_t t = tid; t < rows_here * MT; t += blockDim.x) {
        const uint32_t slot = t / MT, j = t - slot * MT;
        if ((int)j >= m) continue;
        float sum = 0.0f;
        for (uint32_t w = 0; w < n_waves; ++w)
            sum += *reinterpret_cast<const float *>(smem + first_acc + w * wave_bytes + t * 4);
        if (y32) atomicAdd(&y32[(size_t)j * P.out_f + row0 + slot], sum);
        else y[(int64_t)j * ldy + row0 + slot] = (uint16_t)f32_to_bf16_bits(sum);
    }
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------

template <int MT, bool ANY>
static int launch_slots(const Dev &P, const int32_t *prefix, uint32_t n_chunks, const uint16_t *x, int m, int64_t ldx,
                        uint16_t *y, int64_t ldy, float *y32, hipStream_t s) {
    const uint32_t n_quads = P.out_f / 4;
    static const int n_cu = [] {
        int dev = 0, v = 256;
        if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev);
        return v;
    }();
    static const bool raised =  // per instantiation
        hipFuncSetAttribute(reinterpret_cast<const void *>(k_gemv358_slots<MT, ANY>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)kSLdsLimit) == hipSuccess;
    if (!raised) return IXH_EUNSUPPORTED;
    struct Plan {
        uint32_t chunks, out_f, forced, waves, quads, qcap;
    };
    static Plan plans[8] = {};
    static uint32_t next_plan = 0;
    static std::mutex plans_lock;
    const uint32_t forced = (uint32_t)g_opt_gemv_slot_waves.load(std::memory_order_relaxed);
    Plan plan{};
    {
        std::lock_guard<std::mutex> guard(plans_lock);
        const Plan *hit = nullptr;
        for (const Plan &pl : plans)
            if (pl.chunks == n_chunks && pl.out_f == P.out_f && pl.forced == forced) hit = &pl;
        if (!hit) {
            // One workgroup per CU; whole rounds of them, as few as LDS admits (every round pays the set-up and the
            // final sums again).  Waves: the count in 8..16 that leaves the fewest word steps to the busiest wave
            // (groups are dealt whole), the larger count on a tie.
            uint32_t best_w = 0, best_q = 0, best_cap = 0, best_cost = ~0u;
            for (uint32_t w = kSMaxWaves; w >= 8; --w) {
                if (forced && w != forced) continue;
                uint32_t q = 0, cap = 0;
                for (uint32_t rounds = 1; rounds <= 64 && q == 0; ++rounds) {
                    const uint32_t cand = max(1u, (n_quads + rounds * (uint32_t)n_cu - 1) / (rounds * (uint32_t)n_cu));
                    if (cand * 4 > kSRows) continue;
                    // a group leaves at most 256 records (four words of 64 lanes)
                    if (slots_layout(min(cand * 4, P.out_f), n_chunks, w, MT, 256).total <= kSLdsLimit) {
                        q = cand;
                        cap = 256;
                    }
                }
                if (q == 0) continue;
                const uint32_t groups = (q * n_chunks + 3) / 4;
                const uint32_t rounds = (n_quads + q * (uint32_t)n_cu - 1) / (q * (uint32_t)n_cu);
                const uint32_t cost = rounds * ((groups + w - 1) / w) * 16 + rounds * 12;  // word steps + set-up
                if (cost < best_cost) {
                    best_cost = cost;
                    best_w = w;
                    best_q = q;
                    best_cap = cap;
                }
            }
            Plan &slot = plans[next_plan++ % 8u];
            slot = Plan{n_chunks, P.out_f, forced, best_w, best_q, best_cap};
            hit = &slot;
        }
        plan = *hit;
    }
    if (plan.waves == 0) return IXH_EUNSUPPORTED;
    const uint32_t groups = (n_quads + plan.quads - 1) / plan.quads;
    uint32_t flags = 0;
    if (((uintptr_t)P.last & 3u) == 0) flags |= kFlagStageSide;
    const size_t lds = slots_layout(min(plan.quads * 4, P.out_f), n_chunks, plan.waves, MT, plan.qcap).total;
    hipLaunchKernelGGL((k_gemv358_slots<MT, ANY>), dim3(groups), dim3(plan.waves * kWave), lds, s, P, prefix, n_chunks,
                       plan.quads, flags, plan.qcap, (uint32_t)((0x100000000ull + n_chunks - 1) / n_chunks), x, m, ldx, y, ldy,
                       y32);
    return hipGetLastError() == hipSuccess ? IXH_OK : IXH_ELAUNCH;
}

// One to four activation rows, rows a multiple of four, whole 512-column blocks; IXH_EUNSUPPORTED otherwise.
int launch_gemv_358_slots(const Dev &P, const int32_t *prefix, const uint16_t *x, int m, int64_t ldx, uint16_t *y,
                          int64_t ldy, float *y32, hipStream_t s) {
    const int want = g_opt_gemv_slots.load(std::memory_order_relaxed);
    if (want < 0) return IXH_EUNSUPPORTED;
    if (m < 1 || m > 4 || P.out_f == 0 || P.out_f % 4u != 0 || P.in_f % kFastChunk != 0 || P.in_f > 65536u)
        return IXH_EUNSUPPORTED;
    if (want == 0) {
        // Measured against the shared-x row-block kernel: 4-5 % faster at two activation rows where a workgroup has
        // at least two groups a wave (17408 x 5120: 19.1 against 19.9 us, 5120 x 17408: 20.7 against 21.7); slower at
        // one row (18.0 against 17.2) and on layers with a group a wave or less (5120 x 5120: 13.6 against 11.4),
        // where its coarser unit of work (16 (row, column block) pairs) leaves waves idle; at three and four rows
        // the tile kernel is ahead.
        static const int n_cu = [] {
            int dev = 0, v = 256;
            if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev);
            return v;
        }();
        const uint64_t unit_quads_per_wg = (uint64_t)((P.out_f / 4u + (uint32_t)n_cu - 1) / (uint32_t)n_cu) * (P.in_f / kFastChunk);
        if (m != 2 || unit_quads_per_wg < 128) return IXH_EUNSUPPORTED;
    }
    if (((uintptr_t)x & 15u) != 0 || (m > 1 && (ldx & 7) != 0)) return IXH_EUNSUPPORTED;
    const bool any = !(P.n_levels == 3 && P.bits[1] == 5);
    const uint32_t n_chunks = P.in_f / kFastChunk;
    if (m == 1) return any ? launch_slots<1, true>(P, prefix, n_chunks, x, m, ldx, y, ldy, y32, s)
                           : launch_slots<1, false>(P, prefix, n_chunks, x, m, ldx, y, ldy, y32, s);
    if (m == 2) return any ? launch_slots<2, true>(P, prefix, n_chunks, x, m, ldx, y, ldy, y32, s)
                           : launch_slots<2, false>(P, prefix, n_chunks, x, m, ldx, y, ldy, y32, s);
    return any ? launch_slots<4, true>(P, prefix, n_chunks, x, m, ldx, y, ldy, y32, s)
               : launch_slots<4, false>(P, prefix, n_chunks, x, m, ldx, y, ldy, y32, s);
}

}  // namespace ixh

