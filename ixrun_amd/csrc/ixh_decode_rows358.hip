// Full decode to bf16 for tensors that are almost all level 1, for (3,5,8) and any other scheme whose first level has
// 3 bits: built like the row-block product kernel (ixh_rows358.hip) with the dot products taken out and the weights
// written instead.
//
// Work split.  The tensor is a flat run of 512-element units; four consecutive units are a unit-quad.  A workgroup
// owns a contiguous run of unit-quads, its waves take them in turn; each 16-lane DPP row of a wave takes one unit of
// the quad and each lane 32 consecutive elements (one word of bitmap 0), that is 64 bytes of output.
//
// Memory pipeline.  As in the product kernel: the workgroup copies its slice of the rank table to LDS, then every
// wave keeps kDrStages unit-quads in flight with LDS-DMA buffer loads (bitmap words and the 3-bit stream range that
// follows from the table alone).
//
// Decode.  A lane ranks its bitmap word (popcount + DPP scan over its row), reads its own 96-bit code window from
// the staged stream, and splices out the elements that are not level 1 (their field becomes the code of 0); two
// neighbouring codes index the table of dequantised pairs in LDS.  The lane's 16 pairs go through a per-wave LDS
// tile (rows 80 bytes apart) so that a store instruction writes 256 consecutive bytes per unit instead of 16 bytes
// per lane, 64 bytes apart (which costs more than twice the time on this memory system).
//
// Elements above level 1.  They leave one record per bitmap word in a per-wave LDS queue and are written as zero
// by the main path.  Records are resolved 64 at a time (elements spread over the lanes) and the weight is stored
// over the zero, two bytes.  A record is resolved only after its unit's rows have been stored, and the resolver
// first waits until every earlier store of the wave has been acknowledged, so the two stores to one address land in
// order.
#include <stdlib.h>

#include "ixh_fast358.h"

namespace ixh {

typedef uint32_t dr_u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void *dr_lds_ptr_t;

constexpr int kDrStages = 2;  // unit-quads in flight per wave, the one being read included (three: 1 % slower)
constexpr uint32_t kDrStageBytes = 1280;  // 1024 stream + 256 bitmap
constexpr uint32_t kDrQueue = 128;        // records per wave
constexpr uint32_t kDrTasks = 192;        // elements of 64 records that are spread over the lanes
constexpr uint32_t kDrTileBytes = 64 * 80;
constexpr int kDrWaves = 12;              // waves per workgroup (one workgroup per CU)
constexpr uint32_t kDrLutBytes = 64 * 32 * 4;
constexpr uint32_t kDrSpliceBytes = 33 * 32;
constexpr uint32_t kDrSideB2 = 0, kDrSideL2 = 1024, kDrSideL3 = 3072, kDrSideBytes = 4096;
constexpr uint32_t kDrMaxQuads = 256;     // unit-quads per workgroup at most (its table slice is kept in LDS)
constexpr uint32_t kDrWaveBytes = kDrStages * kDrStageBytes + kDrQueue * 16 + kDrTasks * 2 + kDrTileBytes;
constexpr uint32_t kDrZero0 = 0xDB6DB6DBu, kDrZero1 = 0xB6DB6DB6u, kDrZero2 = 0x6DB6DB6Du;  // 32 codes of value 0

struct DrLds {
    uint32_t tq1, tq2, side, waves, total;
};

__host__ __device__ inline DrLds dr_layout(uint32_t quads_cap) {
    DrLds L;
    const uint32_t tbl = ((quads_cap * 4u + 1u + 3u) & ~3u) * 4u;  // one entry past the slice: its end ranks
    L.tq1 = kDrLutBytes + kDrSpliceBytes;
    L.tq2 = L.tq1 + tbl;
    L.side = L.tq2 + tbl;
    L.waves = L.side + kDrSideBytes;
    L.total = L.waves + kDrWaves * kDrWaveBytes;
    return L;
}

__device__ __forceinline__ uint32_t dr_shr(uint32_t v, int n) {
    switch (n) {
        case 1: return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x111, 0xf, 0xf, true);
        case 2: return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x112, 0xf, 0xf, true);
        case 4: return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x114, 0xf, 0xf, true);
        default: return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x118, 0xf, 0xf, true);
    }
}

__device__ __forceinline__ uint32_t dr_row_scan(uint32_t v) {
    v += dr_shr(v, 1);
    v += dr_shr(v, 2);
    v += dr_shr(v, 4);
    v += dr_shr(v, 8);
    return v;
}

template <int N>
__device__ __forceinline__ void dr_wait_vmem() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

__device__ __forceinline__ uint32_t dr_lds_u32(uint32_t addr) {
    return *reinterpret_cast<const __attribute__((address_space(3))) uint32_t *>((uintptr_t)addr);
}
__device__ __forceinline__ uint32_t dr_lds_u8(uint32_t addr) {
    return *reinterpret_cast<const __attribute__((address_space(3))) uint8_t *>((uintptr_t)addr);
}
__device__ __forceinline__ dr_u32x4 dr_lds_u128(uint32_t addr) {
    return *reinterpret_cast<const __attribute__((address_space(3))) dr_u32x4 *>((uintptr_t)addr);
}

struct DrSide {
    bool staged;                // true: in LDS at `base`; false: read from global memory
    uint32_t base;              // LDS address of the staged region
    uint32_t b2w0, l2w0, l3w0;  // first staged word of bitmap 1 / 5-bit stream / 8-bit stream
};

// a store through a restrict-qualified parameter: with the alias scope it gets when inlined, the compiler does not
// put "wait for every LDS-DMA copy in flight" in front of it
__device__ __forceinline__ void dr_push(uint4 *__restrict__ q, uint32_t idx, uint4 v) { q[idx] = v; }

// issued outside the compiler's memory model, for code that runs while the wave has LDS-DMA copies in flight
__device__ __forceinline__ uint64_t dr_read2_raw(uint32_t addr) {  // words at addr and addr + 4
    uint64_t v;
    asm volatile("ds_read2_b32 %0, %1 offset1:1\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(addr) : "memory");
    return v;
}

// The lane's 64 bytes into its row of the tile, and the four 16-byte pieces back that this lane stores: piece j is
// bytes [256 j + 16 li, + 16) of its unit's 1 KB, which lane 4 j + li / 4 of the same DPP row produced as its piece
// li % 4.  LDS executes a wave's instructions in order, every lane of one before the next, so no barrier is needed.
__device__ __forceinline__ void dr_exchange(uint32_t wr_addr, uint32_t rd_addr, const uint32_t (&w)[16], dr_u32x4 (&r)[4]) {
    const dr_u32x4 a = {w[0], w[1], w[2], w[3]}, b = {w[4], w[5], w[6], w[7]}, c = {w[8], w[9], w[10], w[11]},
                   d = {w[12], w[13], w[14], w[15]};
    asm volatile(
        "ds_write_b128 %4, %5\n\t"
        "ds_write_b128 %4, %6 offset:16\n\t"
        "ds_write_b128 %4, %7 offset:32\n\t"
        "ds_write_b128 %4, %8 offset:48\n\t"
        "ds_read_b128 %0, %9\n\t"
        "ds_read_b128 %1, %9 offset:320\n\t"
        "ds_read_b128 %2, %9 offset:640\n\t"
        "ds_read_b128 %3, %9 offset:960\n\t"
        "s_waitcnt lgkmcnt(0)"
        : "=&v"(r[0]), "=&v"(r[1]), "=&v"(r[2]), "=&v"(r[3])
        : "v"(wr_addr), "v"(a), "v"(b), "v"(c), "v"(d), "v"(rd_addr)
        : "memory");
}

// Resolve `count` queued records (see ixh_rows358.hip for the scheme) and store each element's weight over the zero
// that the main path wrote.  Every store the wave issued before has been acknowledged when the first one here leaves.
template <bool STAGED>
__device__ __forceinline__ void dr_resolve(const Dev &P, const DrSide &sv, uint32_t tq1_addr, uint32_t tq2_addr,
                                           uint32_t unit0, const uint4 *__restrict__ queue, uint32_t count,
                                           uint16_t *__restrict__ tasks, uint16_t *__restrict__ out, float scale,
                                           uint32_t lane) {
    const uint32_t *__restrict__ b2 = P.bm[1];
    const uint32_t b2_words = P.bm_words[1];
    auto one = [&](const uint4 rec, uint32_t nth, uint32_t e) {
        const uint32_t r0_lane = rec.y, unit = rec.z;
        const uint32_t r0u = unit * kFastChunk - dr_lds_u32(tq1_addr + (unit - unit0) * 4);
        const uint32_t q2u = dr_lds_u32(tq2_addr + (unit - unit0) * 4);
        const uint32_t wf = r0u >> 5;
        const uint32_t first_mask = ~0u << (r0u & 31);
        const uint32_t r = r0_lane + nth;
        // level-2 elements among bitmap-1 bits [r0u, r) (a unit spans at most 17 words), and the bit at r
        const uint32_t wl = min(r >> 5, wf + 17u);
        uint32_t cnt = 0;
        for (uint32_t w = wf; w < wl; ++w) {
            uint32_t bits = STAGED ? dr_lds_u32(sv.base + kDrSideB2 + (w - sv.b2w0) * 4) : (w < b2_words ? b2[w] : 0u);
            if (w == wf) bits &= first_mask;
            cnt += __popc(bits);
        }
        const uint32_t bits = STAGED ? dr_lds_u32(sv.base + kDrSideB2 + (wl - sv.b2w0) * 4)
                                     : (wl < b2_words ? b2[wl] : 0u);
        uint32_t low = (1u << (r & 31)) - 1u;
        if (wl == wf) low &= first_mask;
        cnt += __popc(bits & low);
        int v = 0;
        if ((bits >> (r & 31)) & 1u) {
            const uint64_t bitpos = (uint64_t)(q2u + cnt) * 5u;
            const uint32_t wi = (uint32_t)(bitpos >> 5), sh = (uint32_t)bitpos & 31u;
            uint32_t lo, hi;
            if (STAGED) {
                const uint64_t pair = dr_read2_raw(sv.base + kDrSideL2 + (wi - sv.l2w0) * 4);
                lo = (uint32_t)pair;
                hi = (uint32_t)(pair >> 32);
            } else {
                lo = wi < P.st_words[1] ? P.st[1][wi] : 0u;
                hi = (sh > 27 && wi + 1 < P.st_words[1]) ? P.st[1][wi + 1] : 0u;
            }
            v = (int)((uint32_t)((((uint64_t)hi << 32) | lo) >> sh) & 31u) - 15;
        } else {
            const uint32_t i3 = r - (q2u + cnt);
            if (STAGED) v = i3 < P.last_bytes ? (int)dr_lds_u8(sv.base + kDrSideL3 + (i3 - sv.l3w0 * 4)) - 127 : 0;
            else v = i3 < P.last_bytes ? (int)P.last[i3] - 127 : 0;
        }
        out[(size_t)unit * kFastChunk + rec.w + e] = (uint16_t)f32_to_bf16_bits((float)v * scale);
    };
    dr_wait_vmem<0>();
    for (uint32_t base = 0; base < count; base += kWave) {
        const uint32_t idx = base + lane;
        const bool has = idx < count;
        uint4 rec = make_uint4(0, 0, 0, 0);
        if (has) rec = queue[idx];
        uint32_t zeros = rec.x;
        const uint32_t mine = (uint32_t)__popc(zeros);
        const uint32_t incl = wave_scan_inclusive(mine);
        const uint32_t n_tasks = (uint32_t)__builtin_amdgcn_readlane((int)incl, 63);
        if (n_tasks <= kDrTasks) {
            uint32_t t = incl - mine, nth = 0;
            while (zeros != 0) {
                tasks[t++] = (uint16_t)((lane << 10) | (nth++ << 5) | (uint32_t)__builtin_ctz(zeros));
                zeros &= zeros - 1;
            }
            for (uint32_t tb = 0; tb < n_tasks; tb += kWave) {
                if (tb + lane < n_tasks) {
                    const uint32_t task = tasks[tb + lane];
                    one(queue[base + (task >> 10)], (task >> 5) & 31u, task & 31u);
                }
            }
        } else {
            uint32_t nth = 0;
            while (zeros != 0) {
                const uint32_t e = (uint32_t)__builtin_ctz(zeros);
                zeros &= zeros - 1;
                one(rec, nth++, e);
            }
        }
    }
}

// The same for any scheme whose first level has 3 bits: an element above level 1 is followed down the nested
// bitmaps (level i: rank among the elements that are in no level below i), every rank counted from the unit's start,
// where the table holds it; all reads from global memory (these elements are rare in the tensors this kernel gets).
__device__ __forceinline__ void dr_resolve_any(const Dev &P, const int32_t *__restrict__ prefix, uint32_t entries,
                                               uint32_t tq1_addr, uint32_t unit0, const uint4 *__restrict__ queue,
                                               uint32_t count, uint16_t *__restrict__ out, float scale, uint32_t lane) {
    auto one = [&](const uint4 rec, uint32_t nth, uint32_t e) {
        const uint32_t unit = rec.z;
        uint32_t r = rec.y + nth;                                                           // rank at level i
        uint32_t ru = unit * kFastChunk - dr_lds_u32(tq1_addr + (unit - unit0) * 4);        // the unit's first rank there
        int v = 0;
        bool found = false;
        for (int i = 1; i + 1 < P.n_levels; ++i) {
            const uint32_t *__restrict__ bm = P.bm[i];
            const uint32_t words = P.bm_words[i];
            const uint32_t qu = (uint32_t)prefix[(size_t)i * entries + unit];  // level-i elements before the unit
            const uint32_t wf = ru >> 5, wl = min(r >> 5, wf + 17u);
            const uint32_t first_mask = ~0u << (ru & 31);
            uint32_t cnt = 0;
            for (uint32_t w = wf; w < wl; ++w) {
                uint32_t bits = w < words ? bm[w] : 0u;
                if (w == wf) bits &= first_mask;
                cnt += __popc(bits);
            }
            const uint32_t bits = wl < words ? bm[wl] : 0u;
            uint32_t low = (1u << (r & 31)) - 1u;
            if (wl == wf) low &= first_mask;
            cnt += __popc(bits & low);
            if ((bits >> (r & 31)) & 1u) {
                const uint32_t nb = (uint32_t)P.bits[i];
                const uint64_t bitpos = (uint64_t)(qu + cnt) * nb;
                const uint32_t wi = (uint32_t)(bitpos >> 5), sh = (uint32_t)bitpos & 31u;
                const uint32_t lo = wi < P.st_words[i] ? P.st[i][wi] : 0u;
                const uint32_t hi = (sh + nb > 32 && wi + 1 < P.st_words[i]) ? P.st[i][wi + 1] : 0u;
                v = (int)((uint32_t)((((uint64_t)hi << 32) | lo) >> sh) & ((1u << nb) - 1u)) - threshold_of((int)nb);
                found = true;
                break;
            }
            r -= qu + cnt;
            ru -= qu;
        }
        if (!found) v = r < P.last_bytes ? (int)P.last[r] - 127 : 0;
        out[(size_t)unit * kFastChunk + rec.w + e] = (uint16_t)f32_to_bf16_bits((float)v * scale);
    };
    dr_wait_vmem<0>();
    for (uint32_t base = 0; base < count; base += kWave) {
        const uint32_t idx = base + lane;
        uint4 rec = make_uint4(0, 0, 0, 0);
        if (idx < count) rec = queue[idx];
        uint32_t zeros = rec.x, nth = 0;
        while (zeros != 0) {
            const uint32_t e = (uint32_t)__builtin_ctz(zeros);
            zeros &= zeros - 1;
            one(rec, nth++, e);
        }
    }
}

// ANY: any scheme whose first level has 3 bits (else: (3,5,8), with the small-share staging of the other streams)
template <bool ANY>
__global__ void __launch_bounds__(kDrWaves *kWave)
k_decode358_rows(Dev P, const int32_t *__restrict__ prefix, uint32_t n_quads, uint32_t quads_per_wg, uint32_t flags,
                 uint16_t *__restrict__ out) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const uint32_t quarter = lane >> 4, li = lane & 15;

    const uint32_t quad0 = blockIdx.x * quads_per_wg;
    const uint32_t quads_here = min(quads_per_wg, n_quads - quad0);
    const uint32_t unit0 = quad0 * 4, units_here = quads_here * 4;
    const DrLds L = dr_layout(quads_per_wg);

    // The pair table is addressed with (index bits | lane bits), which needs it at LDS address 0 (the kernel has no
    // other LDS).  Should that ever not hold, say so in the output instead of computing garbage.
    if ((uint32_t)(uintptr_t)(dr_lds_ptr_t)smem != 0) {
        for (uint32_t t = tid; t < units_here * kFastChunk; t += blockDim.x) out[(size_t)unit0 * kFastChunk + t] = 0x7FC0;
        return;
    }
    uint32_t *const lut = reinterpret_cast<uint32_t *>(smem);             // [64][32]
    uint4 *const splice = reinterpret_cast<uint4 *>(smem + kDrLutBytes);  // [33][2]
    uint32_t *const tq1 = reinterpret_cast<uint32_t *>(smem + L.tq1);
    uint32_t *const tq2 = reinterpret_cast<uint32_t *>(smem + L.tq2);
    uint8_t *const wave_base = smem + L.waves + wave * kDrWaveBytes;
    uint8_t *const ring = wave_base;
    uint4 *const queue = reinterpret_cast<uint4 *>(wave_base + kDrStages * kDrStageBytes);
    uint16_t *const tasks = reinterpret_cast<uint16_t *>(wave_base + kDrStages * kDrStageBytes + kDrQueue * 16);
    const uint32_t tile_addr =
        (uint32_t)(uintptr_t)(dr_lds_ptr_t)(wave_base + kDrStages * kDrStageBytes + kDrQueue * 16 + kDrTasks * 2);

    // ---- workgroup set-up: table slice first (it waits on memory), then the tables built here ----
    const uint16_t scale_bits = *P.scale;  // asked for with the table slice, not in a trip to memory of its own after it
    const uint32_t entries = n_quads * 4 + 1;
    for (uint32_t i = tid; i <= units_here; i += blockDim.x) {
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
    __syncthreads();

    const __amdgpu_buffer_rsrc_t b1_rsrc =
        __builtin_amdgcn_make_buffer_rsrc((void *)P.bm[0], 0, (int)(P.bm_words[0] * 4u), 0x00020000);
    const __amdgpu_buffer_rsrc_t l1_rsrc =
        __builtin_amdgcn_make_buffer_rsrc((void *)P.st[0], 0, (int)(P.st_words[0] * 4u), 0x00020000);

    // ---- this workgroup's share of bitmap 1 and of the 5-bit / 8-bit streams: staged in LDS if it is small ----
    // (every wave copies all of it: same bytes to the same place, and a wave's own loads complete in order, before
    // the first unit it waits for, so no barrier is needed)
    DrSide sv;
    sv.staged = false;
    if (!ANY) {
        const uint32_t q1b = tq1[0], q2b = tq2[0], q1e = tq1[units_here], q2e = tq2[units_here];
        const uint32_t nl1b = unit0 * kFastChunk - q1b, nl1e = (unit0 + units_here) * kFastChunk - q1e;
        sv.base = L.side;
        sv.b2w0 = nl1b >> 5;
        sv.l2w0 = (uint32_t)(((uint64_t)q2b * 5u) >> 5);
        sv.l3w0 = (nl1b - q2b) >> 2;
        const uint32_t n_b2 = ((nl1e + 31) >> 5) - sv.b2w0;
        const uint32_t n_l2 = (uint32_t)((((uint64_t)q2e * 5u) + 31) >> 5) - sv.l2w0;
        const uint32_t n_l3 = ((nl1e - q2e + 3) >> 2) - sv.l3w0;
        // one word of slack each: the resolver reads the word after a code's first word unconditionally
        sv.staged = (flags & 1u) && n_b2 < 256 && n_l2 < 511 && n_l3 <= 256;
        if (sv.staged) {
            const __amdgpu_buffer_rsrc_t b2_rsrc =
                __builtin_amdgcn_make_buffer_rsrc((void *)P.bm[1], 0, (int)(P.bm_words[1] * 4u), 0x00020000);
            const __amdgpu_buffer_rsrc_t l2_rsrc =
                __builtin_amdgcn_make_buffer_rsrc((void *)P.st[1], 0, (int)(P.st_words[1] * 4u), 0x00020000);
            const __amdgpu_buffer_rsrc_t l3_rsrc =
                __builtin_amdgcn_make_buffer_rsrc((void *)P.last, 0, (int)((P.last_bytes + 3u) & ~3u), 0x00020000);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(b2_rsrc, (dr_lds_ptr_t)(smem + L.side + kDrSideB2), 16,
                                                     (int)(sv.b2w0 * 4 + lane * 16), 0, 0, 0);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(l2_rsrc, (dr_lds_ptr_t)(smem + L.side + kDrSideL2), 16,
                                                     (int)(sv.l2w0 * 4 + lane * 16), 0, 0, 0);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(l2_rsrc, (dr_lds_ptr_t)(smem + L.side + kDrSideL2 + 1024), 16,
                                                     (int)(sv.l2w0 * 4 + 1024 + lane * 16), 0, 0, 0);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(l3_rsrc, (dr_lds_ptr_t)(smem + L.side + kDrSideL3), 16,
                                                     (int)(sv.l3w0 * 4 + lane * 16), 0, 0, 0);
        }
    }

    const uint32_t lut_lane = (lane & 31u) << 2;
    const uint32_t splice_addr = kDrLutBytes;
    const uint32_t tq1_addr = L.tq1, tq2_addr = L.tq2;
    const uint32_t ring_addr = (uint32_t)(uintptr_t)(dr_lds_ptr_t)ring;

    // this wave's unit-quads: local quads wave, wave + kDrWaves, ...; walk index i -> local quad wave + i * kDrWaves
    const uint32_t n_mine = wave < quads_here ? (quads_here - wave + kDrWaves - 1) / kDrWaves : 0u;
    if (n_mine == 0) return;
    auto local_unit = [&](uint32_t i) { return (wave + i * kDrWaves) * 4 + quarter; };  // this DPP row's unit of quad i

    // ---- producer: LDS-DMA of unit-quad i into ring stage i % kDrStages ----
    auto issue = [&](uint32_t i) {
        const uint32_t lu = local_unit(i);
        const uint32_t q1u = dr_lds_u32(tq1_addr + lu * 4);
        uint8_t *stage = ring + (i % kDrStages) * kDrStageBytes;
        asm volatile("" ::: "memory");
        if (li < 13)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(l1_rsrc, (dr_lds_ptr_t)stage, 16,
                                                     (int)(((q1u * 3u) >> 5) * 4u + li * 16u), 0, 0, 0);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(b1_rsrc, (dr_lds_ptr_t)(stage + 1024), 4,
                                                 (int)(((unit0 + lu) * 16u + li) * 4u), 0, 0, 0);
    };

    uint32_t qcount = 0;  // records in the queue (wave-uniform)
    uint32_t qmark = 0;   // of which: records of units whose rows have been stored

    auto splice_once = [&](uint32_t &w0, uint32_t &w1, uint32_t &w2, uint32_t &zrem) {
        const uint32_t e = zrem != 0 ? (uint32_t)__builtin_ctz(zrem) : 32u;
        zrem &= zrem - 1;
        const dr_u32x4 lm = dr_lds_u128(splice_addr + e * 32), fm = dr_lds_u128(splice_addr + e * 32 + 16);
        const uint32_t s0 = w0 << 3;
        const uint32_t s1 = __builtin_amdgcn_alignbit(w1, w0, 29);
        const uint32_t s2 = __builtin_amdgcn_alignbit(w2, w1, 29);
        w0 = (w0 & lm.x) | (s0 & ~lm.x);
        w1 = (w1 & lm.y) | (s1 & ~lm.y);
        w2 = (w2 & lm.z) | (s2 & ~lm.z);
        w0 = (w0 & ~fm.x) | (kDrZero0 & fm.x);
        w1 = (w1 & ~fm.y) | (kDrZero1 & fm.y);
        w2 = (w2 & ~fm.z) | (kDrZero2 & fm.z);
    };

    // code window of unit-quad i (its data is in the ring), spliced once; lanes with elements above level 1 leave a record
    auto open_window = [&](uint32_t i, uint32_t &w0, uint32_t &w1, uint32_t &w2, uint32_t &zrem) {
        const uint32_t lu = local_unit(i);
        const uint32_t stage = ring_addr + (i % kDrStages) * kDrStageBytes;
        const uint32_t word = dr_lds_u32(stage + 1024 + lane * 4);
        const uint32_t q1u = dr_lds_u32(tq1_addr + lu * 4);
        const uint32_t c = __popc(word);
        const uint32_t excl = dr_row_scan(c) - c;
        const uint32_t off = excl * 3u + ((q1u * 3u) & 31u);  // bit offset inside the staged stream piece
        const uint32_t wa = stage + quarter * 256 + (off >> 5) * 4;
        const uint32_t d0 = dr_lds_u32(wa), d1 = dr_lds_u32(wa + 4), d2 = dr_lds_u32(wa + 8), d3 = dr_lds_u32(wa + 12);
        w0 = __builtin_amdgcn_alignbit(d1, d0, off);
        w1 = __builtin_amdgcn_alignbit(d2, d1, off);
        w2 = __builtin_amdgcn_alignbit(d3, d2, off);
        const uint32_t zeros = ~word;
        const uint64_t any = __ballot(zeros != 0);
        if (zeros != 0) {
            const uint32_t unit = unit0 + lu;
            const uint32_t r0_lane = unit * kFastChunk + li * 32u - (q1u + excl);
            dr_push(queue, qcount + lanes_below(any), make_uint4(zeros, r0_lane, unit, li * 32u));
        }
        qcount += (uint32_t)__popcll(any);
        zrem = zeros;
        splice_once(w0, w1, w2, zrem);
    };

    auto resolve = [&](uint32_t count) {
        if (ANY) dr_resolve_any(P, prefix, entries, tq1_addr, unit0, queue, count, out, scale, lane);
        else if (sv.staged) dr_resolve<true>(P, sv, tq1_addr, tq2_addr, unit0, queue, count, tasks, out, scale, lane);
        else dr_resolve<false>(P, sv, tq1_addr, tq2_addr, unit0, queue, count, tasks, out, scale, lane);
    };

    // ---- start-up: fill the ring, open the first window ----
    const uint32_t n_pre = min((uint32_t)kDrStages, n_mine);
    for (uint32_t i = 0; i < n_pre; ++i) issue(i);
    if (n_mine >= (uint32_t)kDrStages) dr_wait_vmem<2 * (kDrStages - 1)>();
    else dr_wait_vmem<0>();

    uint32_t cw0, cw1, cw2, czrem;
    open_window(0, cw0, cw1, cw2, czrem);
    while (__ballot(czrem != 0) != 0) splice_once(cw0, cw1, cw2, czrem);

    const uint32_t wr_addr = tile_addr + lane * 80u;
    const uint32_t rd_addr = tile_addr + (quarter * 16u + (li >> 2)) * 80u + (li & 3u) * 16u;

    for (uint32_t i = 0; i < n_mine; ++i) {
        // the waves that share a SIMD (wave, wave + 4, wave + 8) take turns at the issue priority, one unit-quad each
        {
            const uint32_t pr = ((wave >> 2) + i) % 3u;  // s_setprio takes an immediate
            if (pr == 0) __builtin_amdgcn_s_setprio(0);
            else if (pr == 1) __builtin_amdgcn_s_setprio(1);
            else __builtin_amdgcn_s_setprio(2);
        }
        // Room for a full wave of records.  Only the records of units whose rows are stored may be resolved: the
        // current unit's (at most 64, at the queue's end) move to its front.
        if (qcount > kDrQueue - kWave) {
            resolve(qmark);
            const uint32_t rest = qcount - qmark;
            uint4 rec = make_uint4(0, 0, 0, 0);
            if (lane < rest) rec = queue[qmark + lane];
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
            __builtin_amdgcn_wave_barrier();
            if (lane < rest) dr_push(queue, lane, rec);
            qcount = rest;
            qmark = 0;
        }
        // Refill the stage whose window was read last time; make unit-quad i+1 readable.  Behind its two copies the
        // wave has issued, with a ring of two: four stores (quad i-1), two copies; with a ring of three: four
        // stores (quad i-2), two copies, four stores (quad i-1), two copies; the first quads have fewer stores
        // behind them.  (The count is exact because every quad is whole: all four stores of an iteration are always
        // issued.)
        if (i + kDrStages < n_mine) {
            issue(i + kDrStages);
            if (kDrStages == 2) {  // behind the copies of quad i+1: four stores (quad i-1), two copies
                if (i == 0) dr_wait_vmem<2>();
                else dr_wait_vmem<6>();
            } else if (i == 0) dr_wait_vmem<4>();
            else if (i == 1) dr_wait_vmem<8>();
            else dr_wait_vmem<12>();
        } else {
            dr_wait_vmem<0>();
        }

        uint32_t wp[16];
#pragma unroll
        for (int t = 0; t < 16; ++t) {
            const int bit = 6 * t, ob = bit & 31, d = bit >> 5;
            const uint32_t lo = d == 0 ? cw0 : (d == 1 ? cw1 : cw2);
            const uint32_t hi = d == 0 ? cw1 : cw2;
            uint32_t a;  // pair index at bits 12..7
            if (ob > 26) a = __builtin_amdgcn_alignbit(hi, lo, ob - 7);
            else if (ob >= 7) a = lo >> (ob - 7);
            else a = lo << (7 - ob);
            wp[t] = dr_lds_u32((a & 0x1F80u) | lut_lane);
        }
        const uint32_t unit_now = unit0 + local_unit(i);

        // window of unit-quad i+1 (or, past the end, quad i once more without leaving records)
        qmark = qcount;
        uint32_t nw0 = cw0, nw1 = cw1, nw2 = cw2, nzrem = 0;
        if (i + 1 < n_mine) {
            open_window(i + 1, nw0, nw1, nw2, nzrem);
            while (__ballot(nzrem != 0) != 0) splice_once(nw0, nw1, nw2, nzrem);
        }
        cw0 = nw0; cw1 = nw1; cw2 = nw2;

        dr_u32x4 piece[4];
        dr_exchange(wr_addr, rd_addr, wp, piece);
        dr_u32x4 *const dst = reinterpret_cast<dr_u32x4 *>(out + (size_t)unit_now * kFastChunk) + li;
#pragma unroll
        for (int j = 0; j < 4; ++j) dst[16 * j] = piece[j];
    }
    resolve(qcount);
}

bool decode_rows358_supports(const Dev &P, uint32_t chunk, const int8_t *o8, const uint16_t *o16) {
    return P.n_levels >= 2 && P.bits[0] == 3 && chunk == kFastChunk && !o8 && o16 &&
           ((uintptr_t)o16 & 15u) == 0 && P.n != 0 && P.n % (4 * kFastChunk) == 0 && P.n < (1u << 30);
}

int launch_decode_rows358(const Dev &P, const int32_t *prefix, uint16_t *o16, hipStream_t s) {
    const uint32_t n_quads = P.n / (4 * kFastChunk);
    static const int n_cu = [] {
        int dev = 0, v = 256;
        if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev);
        return v;
    }();
    // whole rounds of one workgroup per CU, each with a contiguous run of at most kDrMaxQuads unit-quads
    const uint32_t rounds = (n_quads + (uint32_t)n_cu * kDrMaxQuads - 1) / ((uint32_t)n_cu * kDrMaxQuads);
    const uint32_t quads = max(1u, (n_quads + rounds * (uint32_t)n_cu - 1) / (rounds * (uint32_t)n_cu));
    const uint32_t groups = (n_quads + quads - 1) / quads;
    const size_t lds = dr_layout(quads).total;
    static bool raised = false;
    if (!raised) {
        if (hipFuncSetAttribute(reinterpret_cast<const void *>(k_decode358_rows<false>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess ||
            hipFuncSetAttribute(reinterpret_cast<const void *>(k_decode358_rows<true>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess)
            return IXH_EUNSUPPORTED;
        raised = true;
    }
    if (lds > 160 * 1024) return IXH_EUNSUPPORTED;
    const uint32_t flags = ((uintptr_t)P.last & 3u) == 0 ? 1u : 0u;
    if (P.n_levels == 3 && P.bits[1] == 5)
        hipLaunchKernelGGL(k_decode358_rows<false>, dim3(groups), dim3(kDrWaves * kWave), lds, s, P, prefix, n_quads, quads,
                           flags, o16);
    else
        hipLaunchKernelGGL(k_decode358_rows<true>, dim3(groups), dim3(kDrWaves * kWave), lds, s, P, prefix, n_quads, quads,
                           flags, o16);
    return hipGetLastError() == hipSuccess ? IXH_OK : IXH_ELAUNCH;
}

}  // namespace ixh
