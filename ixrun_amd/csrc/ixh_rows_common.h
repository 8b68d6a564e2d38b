// Device helpers shared by the (3,5,8) row-block kernels (ixh_rows358.hip, ixh_strips358.hip): LDS access, DPP
// scans, the splice constants and the resolver of the elements above level 1.  Internal to the library.
#pragma once
#include "ixh_fast358.h"

namespace ixh {

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void *lds_ptr_t;

constexpr int kRStages = 3;              // unit-quads in flight per wave
constexpr uint32_t kRStageBytes = 1280;  // 1024 stream + 256 bitmap
constexpr uint32_t kRQueue = 128;        // records per wave
constexpr uint32_t kRTasks = 192;        // elements above level 1 of 64 records that are spread over the lanes
constexpr uint32_t kRTasks2 = 320;       // the same for the kernels that resolve 128 records at a time
constexpr uint32_t kRSlots = 64;         // rows per workgroup at most
constexpr int kRMaxWaves = 12;           // waves per workgroup at most: 3 per SIMD, up to 168 VGPRs each
constexpr uint32_t kRLutBytes = 64 * 32 * 4;
constexpr uint32_t kRSpliceBytes = 33 * 32;
// staged share of the other streams: bitmap 1 (1 KB), 5-bit stream (2 KB), 8-bit stream (1 KB)
constexpr uint32_t kRSideB2 = 0, kRSideL2 = 1024, kRSideL3 = 3072, kRSideBytes = 4096;

constexpr uint32_t kFlagStageSide = 2u;  // the 8-bit stream is dword aligned, the side streams may be staged

constexpr uint32_t kZeroCodes0 = 0xDB6DB6DBu, kZeroCodes1 = 0xB6DB6DB6u, kZeroCodes2 = 0x6DB6DB6Du;

__device__ __forceinline__ uint32_t dpp_shr(uint32_t v, int n) {
    switch (n) {
        case 1: return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x111, 0xf, 0xf, true);
        case 2: return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x112, 0xf, 0xf, true);
        case 4: return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x114, 0xf, 0xf, true);
        default: return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x118, 0xf, 0xf, true);
    }
}

__device__ __forceinline__ uint32_t row_scan(uint32_t v) {
    v += dpp_shr(v, 1);
    v += dpp_shr(v, 2);
    v += dpp_shr(v, 4);
    v += dpp_shr(v, 8);
    return v;
}

__device__ __forceinline__ float row_sum(float v) {
    v += __uint_as_float(dpp_shr(__float_as_uint(v), 1));
    v += __uint_as_float(dpp_shr(__float_as_uint(v), 2));
    v += __uint_as_float(dpp_shr(__float_as_uint(v), 4));
    v += __uint_as_float(dpp_shr(__float_as_uint(v), 8));
    return v;
}

template <int N>
__device__ __forceinline__ void wait_vmem() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

__device__ __forceinline__ uint32_t lds_u32(uint32_t addr) {
    return *reinterpret_cast<const __attribute__((address_space(3))) uint32_t *>((uintptr_t)addr);
}
__device__ __forceinline__ uint32_t lds_u16(uint32_t addr) {
    return *reinterpret_cast<const __attribute__((address_space(3))) uint16_t *>((uintptr_t)addr);
}
__device__ __forceinline__ uint32_t lds_u8(uint32_t addr) {
    return *reinterpret_cast<const __attribute__((address_space(3))) uint8_t *>((uintptr_t)addr);
}
__device__ __forceinline__ u32x4 lds_u128(uint32_t addr) {
    return *reinterpret_cast<const __attribute__((address_space(3))) u32x4 *>((uintptr_t)addr);
}

// where the elements above level 1 of this workgroup's rows live
struct SideView {
    bool staged;             // true: in LDS at `base`; false: read from global memory
    uint32_t base;           // LDS address of the staged region
    uint32_t b2w0, l2w0, l3w0;  // first staged word of bitmap 1 / 5-bit stream / 8-bit stream
};

// A store through a restrict-qualified parameter: once inlined it carries alias-scope information, which is
// what keeps the compiler from putting "wait for every LDS-DMA copy in flight" (s_waitcnt vmcnt(0)) in front
// of an LDS access that has nothing to do with the ring the copies land in.
__device__ __forceinline__ void push_record(uint4 *__restrict__ q, uint32_t idx, uint4 v) { q[idx] = v; }
// the 8-byte records of a kernel with a sink (resolve_rows_to), in the same queue
__device__ __forceinline__ void push_record8(uint4 *__restrict__ q, uint32_t idx, uint32_t word, uint32_t packed) {
    reinterpret_cast<uint2 *>(q)[idx] = make_uint2(word, packed);
}
template <bool COMPACT>
__device__ __forceinline__ uint4 read_record(const uint4 *__restrict__ q, uint32_t idx) {
    if (!COMPACT) return q[idx];
    const uint2 v = reinterpret_cast<const uint2 *>(q)[idx];
    return make_uint4(v.x, v.y, 0u, 0u);
}

// Two LDS operations issued outside the compiler's memory model, for the code that runs while the wave has
// LDS-DMA copies in flight: in front of a merged two-word LDS read and of an LDS atomic the compiler puts
// "wait for every copy" (it cannot tell that they do not touch the ring), which would stall the ring.
__device__ __forceinline__ uint64_t lds_read2_raw(uint32_t addr) {  // words at addr and addr + 4
    uint64_t v;
    asm volatile("ds_read2_b32 %0, %1 offset1:1\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(addr) : "memory");
    return v;
}
__device__ __forceinline__ void lds_add_f32_raw(uint32_t addr, float v) {  // complete after s_waitcnt lgkmcnt(0)
    asm volatile("ds_add_f32 %0, %1" ::"v"(addr), "v"(v) : "memory");
}

// Sums over runs of equal keys among neighbouring lanes of a 16-lane row (a segmented scan in four DPP steps):
// v becomes the sum of the run's values up to and including this lane; returns true in the last lane of a run.
// Used in front of LDS atomics whose lanes mostly target a handful of addresses: the elements of one weight row come
// in runs, and lanes that add to one address are served one after the other.
template <int MT>
__device__ __forceinline__ bool run_sums(uint32_t key, float (&v)[MT], uint32_t lane) {
    const uint32_t k1 = key + 1u;  // never 0, which is what a row's first lane reads from "the lane below"
    const uint32_t head = dpp_shr(k1, 1) != k1 ? 1u : 0u;
    uint32_t f = head;
#pragma unroll
    for (int d = 1; d < 16; d <<= 1) {
        const uint32_t fs = dpp_shr(f, d);
#pragma unroll
        for (int j = 0; j < MT; ++j) {
            const float vs = __uint_as_float(dpp_shr(__float_as_uint(v[j]), d));
            v[j] += f ? 0.0f : vs;
        }
        f |= fs;
    }
    // the head flag of the lane above (row_shl:1; a row's last lane reads 0 and is a tail anyway)
    const uint32_t next_head = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)head, 0x101, 0xf, 0xf, true);
    return next_head != 0 || (lane & 15u) == 15u;
}

// inclusive sum over the lanes at or below this one
__device__ __forceinline__ uint32_t wave_scan(uint32_t v) {
    v = row_scan(v);
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x142, 0xa, 0xf, false);  // row_bcast:15 into rows 1, 3
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x143, 0xc, 0xf, false);  // row_bcast:31 into rows 2, 3
    return v;
}

// Resolve queued records: every record is one bitmap word with elements above level 1.  The elements of 64
// records are first spread over the lanes (one element per lane and round, through a task list in LDS), so
// that the dependent reads of an element (bitmap 1, its code, x) are paid once per round and not once per
// element of the fullest record; a batch with more than kRTasks elements is walked record by record instead.
// STAGED: the workgroup's share of bitmap 1 and of the 5-bit / 8-bit streams is in LDS; that version reads
// no global memory at all (the activations come from the wave's LDS copy), so nothing in it waits for the
// copies the wave has in flight: a load from global memory returns behind all of them.
// ANY: any scheme whose first level has 3 bits: the element is followed down the nested bitmaps (level i: rank among
// the elements in no level below i), every rank counted from the unit's start, where the table holds it (read
// from global memory; tq2 and the staged side streams are not used).
// XL, where the activations are: 0 = the wave's own copy of the rows of its column blocks (xs_row elements apart,
// first column k_first); 1 = the workgroup's shared, swizzled copy of the whole x rows (xs_row bytes apart): 16-byte
// piece p of the 64 bytes that lane l of a 16-lane row owns in a column block sits at piece p * 16 + l of the block;
// 2 = the workgroup's shared copy, from column k_first (a multiple of 128) on, in strips of 128 columns, STRIP bytes
// apart (xs_row bytes between rows); 3 = as 1, with the column blocks kSkewedBlock bytes apart instead of 1024 and
// records of 8 bytes: the bitmap word, and {level-1 elements of the unit before the word (9 bits), word of the unit
// << 9, column block << 13, row of the workgroup << 20}; n_blocks is then the number of column blocks of a row.
constexpr uint32_t kSkewedBlock = kFastChunk * 2 + 16;  // neighbouring column blocks start four LDS banks apart
constexpr uint32_t kStripBytes = 264;  // 128 bf16 + 8: neighbouring strips start two LDS banks apart

// POOL: the elements come from a task list that the waves of the workgroup filled together (entry = wave << 18 |
// record << 10 | nth element of the record << 5 | bit of the record's word; the waves' queues are queue_stride bytes
// apart from queues_addr); this wave takes the rounds of 64 tasks first_round, first_round + round_stride, ... and adds
// into its own row sums, so what every wave adds, and in which order, is fixed.
struct TaskPool {
    uint32_t addr, total, first_round, round_stride, queues_addr, queue_stride;
};

// SINK: where a resolved element goes when it is not added to the row sums here (XL == 2 only): put() takes the
// weight's bf16 bits, the record's row field and the LDS address of the element's column in the first activation
// row, idle() is called by the lanes that have no element in a round, and flush() by the whole wave after every
// round of at most 64 elements (its argument: the lanes below that number may have taken part).
// A sink also brings its own record format: 8 bytes, the bitmap word and a word that unpack() turns into the
// fields of the 16-byte record (rank of the word's first element in bitmap 1's domain, unit, column, row field).
struct Now { static constexpr bool value = false; };    // one(): add the element's products to the row sums
struct Later { static constexpr bool value = true; };  // one(): leave them to the caller
struct NoSink {
    static constexpr bool active = false;
    __device__ __forceinline__ void unpack(uint32_t, uint32_t, uint32_t, uint32_t &, uint32_t &, uint32_t &, uint32_t &) {}
    __device__ __forceinline__ void put(uint32_t, uint32_t, uint32_t) {}
    __device__ __forceinline__ void idle() {}
    __device__ __forceinline__ void flush(uint32_t) {}
};

template <int MT, bool STAGED, bool ANY, int XL, bool POOL, uint32_t STRIP, class SINK>
__device__ __forceinline__ void resolve_rows_to(SINK &sink, const Dev &P, const SideView &sv, uint32_t tq1_addr, uint32_t tq2_addr,
                                             uint32_t unit0, const uint4 *__restrict__ queue, uint32_t count,
                                             uint32_t rowacc_addr, uint16_t *__restrict__ tasks,
                                             uint32_t xs_addr, uint32_t xs_row, uint32_t k_first,
                                             int m, float scale, uint32_t lane,
                                             const int32_t *__restrict__ prefix, uint32_t entries, TaskPool pool,
                                             uint32_t n_blocks = 0) {
    constexpr bool kCompact = SINK::active || XL == 3;
    const uint32_t *__restrict__ b2 = P.bm[1];
    const uint32_t b2_words = P.bm_words[1];
    // value of the element at rank r of bitmap 1's domain, unit `unit`, any scheme
    auto value_any = [&](uint32_t unit, uint32_t r) {
        uint32_t ru = unit * kFastChunk - lds_u32(tq1_addr + (unit - unit0) * 4);  // the unit's first rank at level i
        for (int i = 1; i + 1 < P.n_levels; ++i) {
            const uint32_t *__restrict__ bm = P.bm[i];
            const uint32_t words = P.bm_words[i];
            const uint32_t qu = (uint32_t)prefix[(size_t)i * entries + unit];  // level-i elements before the unit
            const uint32_t wf = ru >> 5, wl = min(r >> 5, wf + 17u);
            const uint32_t first_mask = ~0u << (ru & 31);
            // the first two words are asked for together with the table entry: where few elements are above level 1
            // the element's bit is in one of them, and the chain is one trip to memory long instead of three
            const uint32_t word0 = wf < words ? bm[wf] : 0u, word1 = wf + 1 < words ? bm[wf + 1] : 0u;
            uint32_t cnt = wl > wf ? __popc(word0 & first_mask) : 0u;
            uint32_t bits = wl == wf ? word0 : word1;
            if (wl > wf + 1) {
                cnt += __popc(word1);
                for (uint32_t w = wf + 2; w < wl; ++w) cnt += __popc(w < words ? bm[w] : 0u);
                bits = wl < words ? bm[wl] : 0u;
            }
            uint32_t low = (1u << (r & 31)) - 1u;
            if (wl == wf) low &= first_mask;
            cnt += __popc(bits & low);
            if ((bits >> (r & 31)) & 1u) {
                const uint32_t nb = (uint32_t)P.bits[i];
                const uint64_t bitpos = (uint64_t)(qu + cnt) * nb;
                const uint32_t wi = (uint32_t)(bitpos >> 5), sh = (uint32_t)bitpos & 31u;
                const uint32_t lo = wi < P.st_words[i] ? P.st[i][wi] : 0u;
                const uint32_t hi = (sh + nb > 32 && wi + 1 < P.st_words[i]) ? P.st[i][wi + 1] : 0u;
                return (int)((uint32_t)((((uint64_t)hi << 32) | lo) >> sh) & ((1u << nb) - 1u)) - threshold_of((int)nb);
            }
            r -= qu + cnt;
            ru -= qu;
        }
        return r < P.last_bytes ? (int)P.last[r] - 127 : 0;
    };
    // element `e` (bit of the record's word), the nth element above level 1 of its record; with Later the products
    // are not added to the row sums here but left in d_p / d_slot for the caller (XL != 2 only)
    float d_p[XL == 2 ? 1 : MT];
    uint32_t d_slot = 0;
    auto one = [&](const uint4 rec, uint32_t nth, uint32_t e, auto when) {
        constexpr bool kDefer = decltype(when)::value && XL != 2;
        uint32_t r0_lane = rec.y, unit = rec.z, k0 = rec.w & 0xFFFFu;
        uint32_t slot = rec.w >> 16;
        if (SINK::active) sink.unpack(rec.y, unit0, tq1_addr, r0_lane, unit, k0, slot);
        if (XL == 3) {
            const uint32_t in_unit = ((rec.y >> 9) & 15u) * 32u, col = (rec.y >> 13) & 127u;
            slot = rec.y >> 20;
            const uint32_t tidx = slot * n_blocks + col;
            unit = unit0 + tidx;
            r0_lane = unit * kFastChunk + in_unit - (lds_u32(tq1_addr + tidx * 4u) + (rec.y & 511u));
            k0 = col * kFastChunk + in_unit;
        }
        if (XL == 1) {  // the shared-x kernel's records: rank offset in the unit, LDS address of the unit's table
                    // entry, column block << 4 | lane
            const uint32_t in_unit = (rec.w & 15u) * 32u;
            unit = unit0 + ((rec.z - tq1_addr) >> 2);
            r0_lane = unit * kFastChunk + in_unit - (lds_u32(rec.z) + rec.y);
            k0 = ((rec.w >> 4) & 0xFFFu) * kFastChunk + in_unit;
        }
        // XL == 2 (up to 16 activation rows): the activations are read in a loop at the end, one register at a time
        auto add_all = [&](float w) {
            const uint32_t xa = xs_addr + ((k0 - k_first) >> 7) * STRIP + ((k0 & 127u) + e) * 2u;
            if (SINK::active) {
                sink.put(__float_as_uint(w) >> 16, slot, xa);
                return;
            }
            const uint32_t ra = rowacc_addr + slot * (uint32_t)m * 4u;
#pragma unroll 1
            for (int j = 0; j < m; ++j)
                lds_add_f32_raw(ra + (uint32_t)j * 4u, bf16_bits_to_f32(lds_u16(xa + (uint32_t)j * xs_row)) * w);
        };
        uint32_t xe[XL == 2 ? 1 : MT];  // the activations this element meets
#pragma unroll
        for (int j = 0; j < (XL == 2 ? 0 : MT); ++j) {
            if (XL == 1 || XL == 3)
                xe[j] = lds_u16(xs_addr + (uint32_t)j * xs_row + (k0 >> 9) * (XL == 3 ? kSkewedBlock : kFastChunk * 2) +
                                (((e >> 3) * 16u + ((k0 >> 5) & 15u)) * 16u) + (e & 7u) * 2u);
            else
                xe[j] = lds_u16(xs_addr + ((uint32_t)j * xs_row + k0 - k_first + e) * 2u);
        }
        if (ANY) {
            const float w = dequant(value_any(unit, r0_lane + nth), scale);
            if (XL == 2) {
                add_all(w);
                return;
            }
            if (kDefer) {
                d_slot = slot;
#pragma unroll
                for (int j = 0; j < (XL == 2 ? 0 : MT); ++j) d_p[j] = j < m ? bf16_bits_to_f32(xe[j]) * w : 0.0f;
                return;
            }
#pragma unroll
            for (int j = 0; j < MT; ++j)
                if (j < m) lds_add_f32_raw(rowacc_addr + (slot * MT + j) * 4, bf16_bits_to_f32(xe[j]) * w);
            return;
        }
        const uint32_t r0u = unit * kFastChunk - lds_u32(tq1_addr + (unit - unit0) * 4);
        const uint32_t q2u = lds_u32(tq2_addr + (unit - unit0) * 4);
        const uint32_t wf = r0u >> 5;
        const uint32_t first_mask = ~0u << (r0u & 31);
        const uint32_t r = r0_lane + nth;
        // level-2 elements among bitmap-1 bits [r0u, r) (a unit spans at most 17 words), and the bit at r
        const uint32_t wl = min(r >> 5, wf + 17u);
        // the first two words together (see value_any); a staged word past the share's end is a word of the next region
        auto b2_word = [&](uint32_t w) {
            return STAGED ? lds_u32(sv.base + kRSideB2 + (w - sv.b2w0) * 4) : (w < b2_words ? b2[w] : 0u);
        };
        const uint32_t word0 = b2_word(wf), word1 = b2_word(wf + 1);
        uint32_t cnt = wl > wf ? __popc(word0 & first_mask) : 0u;
        uint32_t bits = wl == wf ? word0 : word1;
        if (wl > wf + 1) {
            cnt += __popc(word1);
            for (uint32_t w = wf + 2; w < wl; ++w) cnt += __popc(b2_word(w));
            bits = b2_word(wl);
        }
        uint32_t low = (1u << (r & 31)) - 1u;
        if (wl == wf) low &= first_mask;
        cnt += __popc(bits & low);
        int v = 0;
        if ((bits >> (r & 31)) & 1u) {
            const uint64_t bitpos = (uint64_t)(q2u + cnt) * 5u;
            const uint32_t wi = (uint32_t)(bitpos >> 5), sh = (uint32_t)bitpos & 31u;
            uint32_t lo, hi;
            if (STAGED) {
                const uint64_t pair = lds_read2_raw(sv.base + kRSideL2 + (wi - sv.l2w0) * 4);
                lo = (uint32_t)pair;
                hi = (uint32_t)(pair >> 32);
            } else {
                lo = wi < P.st_words[1] ? P.st[1][wi] : 0u;
                hi = (sh > 27 && wi + 1 < P.st_words[1]) ? P.st[1][wi + 1] : 0u;
            }
            v = (int)((uint32_t)((((uint64_t)hi << 32) | lo) >> sh) & 31u) - 15;
        } else {
            const uint32_t i3 = r - (q2u + cnt);
            if (STAGED) v = i3 < P.last_bytes ? (int)lds_u8(sv.base + kRSideL3 + (i3 - sv.l3w0 * 4)) - 127 : 0;
            else v = i3 < P.last_bytes ? (int)P.last[i3] - 127 : 0;
        }
        const float w = dequant(v, scale);
        if (XL == 2) {
            add_all(w);
            return;
        }
        if (kDefer) {
            d_slot = slot;
#pragma unroll
            for (int j = 0; j < (XL == 2 ? 0 : MT); ++j) d_p[j] = j < m ? bf16_bits_to_f32(xe[j]) * w : 0.0f;
            return;
        }
#pragma unroll
        for (int j = 0; j < MT; ++j)
            if (j < m) lds_add_f32_raw(rowacc_addr + (slot * MT + j) * 4, bf16_bits_to_f32(xe[j]) * w);
    };
    if (POOL) {
        for (uint32_t r = pool.first_round; r * kWave < pool.total; r += pool.round_stride) {
            const uint32_t t = r * kWave + lane;
            if (t < pool.total) {
                const uint32_t task = lds_u32(pool.addr + t * 4u);
                const u32x4 rv = lds_u128(pool.queues_addr + (task >> 18) * pool.queue_stride + ((task >> 10) & 255u) * 16u);
                one(make_uint4(rv.x, rv.y, rv.z, rv.w), (task >> 5) & 31u, task & 31u, Now{});
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        return;
    }
    // Batches of up to 128 records, two per lane (A: record base + lane, B: base + 64 + lane): one scan, one task list
    // (A's elements first, then B's, kRTasks2 at most) and full rounds for a wave that comes with 65..128 records.
    // With XL == 2 and no sink: 64 records, one per lane, kRTasks elements.
    constexpr bool kTwo = SINK::active || XL != 2;
    constexpr uint32_t kTaskCap = kTwo ? kRTasks2 : kRTasks;
    for (uint32_t base = 0; base < count; base += (kTwo ? 2 : 1) * kWave) {
        const uint32_t idx_a = base + lane, idx_b = idx_a + kWave;
        uint32_t zeros_a = 0, zeros_b = 0;
        if (idx_a < count) zeros_a = read_record<kCompact>(queue, idx_a).x;
        if (kTwo && idx_b < count) zeros_b = read_record<kCompact>(queue, idx_b).x;
        const uint32_t mine_a = (uint32_t)__popc(zeros_a), mine_b = (uint32_t)__popc(zeros_b);
        const uint32_t incl = wave_scan(mine_a | (mine_b << 16));  // at most 64 x 32 elements each: 12 bits
        const uint32_t totals = (uint32_t)__builtin_amdgcn_readlane((int)incl, 63);
        const uint32_t n_a = totals & 0xFFFFu, n_tasks = n_a + (totals >> 16);
        if (n_tasks <= kTaskCap) {
            // task = record of the batch << 5 | bit of its word
            for (uint32_t t = (incl & 0xFFFFu) - mine_a; zeros_a != 0; zeros_a &= zeros_a - 1)
                tasks[t++] = (uint16_t)((lane << 5) | (uint32_t)__builtin_ctz(zeros_a));
            if (kTwo)
                for (uint32_t t = n_a + (incl >> 16) - mine_b; zeros_b != 0; zeros_b &= zeros_b - 1)
                    tasks[t++] = (uint16_t)(((lane + kWave) << 5) | (uint32_t)__builtin_ctz(zeros_b));
            // Without a sink the products of a round are summed over runs of one weight row first (the tasks are in
            // record order, so a row's elements sit in neighbouring lanes), and only the last lane of a run adds.
            constexpr bool kRuns = !SINK::active && XL != 2;
            for (uint32_t tb = 0; tb < n_tasks; tb += kWave) {
                if (kRuns) {
                    d_slot = ~1u;  // lanes without an element: a key no row has
#pragma unroll
                    for (int j = 0; j < (XL == 2 ? 0 : MT); ++j) d_p[j] = 0.0f;
                }
                if (tb + lane < n_tasks) {
                    const uint32_t task = tasks[tb + lane];
                    const uint4 rec = read_record<kCompact>(queue, base + (task >> 5));
                    const uint32_t e = task & 31u;
                    one(rec, (uint32_t)__popc(rec.x & ((1u << e) - 1u)), e, Later{});
                } else if (SINK::active) {
                    sink.idle();
                }
                if (SINK::active) sink.flush(n_tasks - tb);
                if (kRuns) {
                    const bool tail = run_sums<(XL == 2 ? 1 : MT)>(d_slot, d_p, lane);
                    if (tail && d_slot != ~1u) {
#pragma unroll
                        for (int j = 0; j < (XL == 2 ? 0 : MT); ++j)
                            if (j < m) lds_add_f32_raw(rowacc_addr + (d_slot * MT + j) * 4, d_p[j]);
                    }
                }
            }
            continue;
        }
        // more elements than the task list holds: every lane walks its own records, A then B
        for (uint32_t half = 0; half < (kTwo ? 2u : 1u); ++half) {
            const uint32_t idx = half == 0 ? idx_a : idx_b;
            uint4 rec = make_uint4(0, 0, 0, 0);
            if (idx < count) rec = read_record<kCompact>(queue, idx);
            uint32_t zeros = rec.x, nth = 0;
            if (SINK::active) {
                for (uint64_t left = __ballot(zeros != 0); left != 0; left = __ballot(zeros != 0)) {
                    if (zeros != 0) {
                        const uint32_t e = (uint32_t)__builtin_ctz(zeros);
                        zeros &= zeros - 1;
                        one(rec, nth++, e, Now{});
                    } else {
                        sink.idle();
                    }
                    sink.flush(64u - (uint32_t)__builtin_clzll(left));
                }
            } else {
                while (zeros != 0) {
                    const uint32_t e = (uint32_t)__builtin_ctz(zeros);
                    zeros &= zeros - 1;
                    one(rec, nth++, e, Now{});
                }
            }
        }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the row sums have taken the additions
}

template <int MT, bool STAGED, bool ANY = false, int XL = 0, bool POOL = false, uint32_t STRIP = kStripBytes>
__device__ __forceinline__ void resolve_rows(const Dev &P, const SideView &sv, uint32_t tq1_addr, uint32_t tq2_addr,
                                             uint32_t unit0, const uint4 *__restrict__ queue, uint32_t count,
                                             uint32_t rowacc_addr, uint16_t *__restrict__ tasks,
                                             uint32_t xs_addr, uint32_t xs_row, uint32_t k_first,
                                             int m, float scale, uint32_t lane,
                                             const int32_t *__restrict__ prefix = nullptr, uint32_t entries = 0,
                                             TaskPool pool = TaskPool{0, 0, 0, 1, 0, 0}, uint32_t n_blocks = 0) {
    NoSink none;
    resolve_rows_to<MT, STAGED, ANY, XL, POOL, STRIP>(none, P, sv, tq1_addr, tq2_addr, unit0, queue, count, rowacc_addr, tasks,
                                                      xs_addr, xs_row, k_first, m, scale, lane, prefix, entries, pool, n_blocks);
}

// s_setprio takes an immediate
__device__ __forceinline__ void set_wave_priority(uint32_t p) {
    if (p == 0) __builtin_amdgcn_s_setprio(0);
    else if (p == 1) __builtin_amdgcn_s_setprio(1);
    else __builtin_amdgcn_s_setprio(2);
}

}  // namespace ixh
