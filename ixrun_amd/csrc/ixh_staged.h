// Level-scheme-agnostic decode from LDS: the streams of one table unit (a run of
// `chunk` <= 512 flat elements) are first copied into an LDS slot with LDS-DMA
// buffer loads, then ranked and decoded 64 elements at a time with wave ballots,
// reading only LDS.  Used where the gather latency of the global-memory decoder
// (decode64 in ixh_dev.h) cannot be hidden: the prefill GEMM and dense tensors.
#pragma once

#include "ixh_dev.h"

namespace ixh {

typedef __attribute__((address_space(3))) void *lds_ptr_t;

constexpr uint32_t kStagedChunk = 512;  // largest unit the slot is sized for

// LDS words a unit of 512 elements can need.  Every span is copied 16 bytes per lane and
// padded to a multiple of 16 bytes: a bitmap span is at most 17 words (20 padded), all code
// streams together at most 512*8/32 words plus, per stream, the partial first word, one
// word for a straddling read and the padding.
__host__ __device__ constexpr uint32_t staged_slot_words(int n_levels) {
    return (uint32_t)(n_levels - 1) * 20u + 128u + 8u * (uint32_t)n_levels;
}
// buffer loads into LDS that one call of stage_unit issues, always: the count a caller needs to wait for
// one unit's copies while later ones are still in flight (s_waitcnt vmcnt)
__host__ __device__ constexpr int staged_dma_count(int n_levels) { return 2 * n_levels - 1; }

__device__ __forceinline__ uint32_t slds_u32(uint32_t addr) {
    return *reinterpret_cast<const __attribute__((address_space(3))) uint32_t *>((uintptr_t)addr);
}
__device__ __forceinline__ uint32_t slds_u8(uint32_t addr) {
    return *reinterpret_cast<const __attribute__((address_space(3))) uint8_t *>((uintptr_t)addr);
}

// Where the staged spans of one unit sit, folded so that a lane only adds its own
// index: 5 * (L - 1) + 1 wave-uniform words per unit.
template <int L>
struct StagedUnit {
    uint32_t bm_addr[L - 1];  // LDS address of the bitmap word holding the unit's first bit
    uint32_t bm_off[L - 1];   // add to a level-i space index to get the bit index inside the staged span
    uint32_t st_addr[L - 1];  // LDS address of the stream word holding the unit's first code
    uint32_t st_off[L - 1];   // add to rank * bits to get the bit index inside the staged span
    uint32_t cnt0[L - 1];     // level counts before the unit (the table entry)
    uint32_t last_off;        // add to a last-level rank to get the LDS byte address
};

template <int L>
__host__ __device__ constexpr uint32_t staged_record_words() { return 5u * (uint32_t)(L - 1) + 1u; }

// A unit's record parked in LDS between the wave that staged it and the decode (which may
// be a row later): lane 0 writes, every lane reads the same words back into registers.
template <int L>
__device__ __forceinline__ void put_unit(uint32_t rec, uint32_t lane, const StagedUnit<L> &S) {
    if (lane == 0) {
        __attribute__((address_space(3))) uint32_t *r = (__attribute__((address_space(3))) uint32_t *)(uintptr_t)rec;
#pragma unroll
        for (int i = 0; i < L - 1; ++i) {
            r[5 * i + 0] = S.bm_addr[i];
            r[5 * i + 1] = S.bm_off[i];
            r[5 * i + 2] = S.st_addr[i];
            r[5 * i + 3] = S.st_off[i];
            r[5 * i + 4] = S.cnt0[i];
        }
        r[5 * (L - 1)] = S.last_off;
    }
}
template <int L>
__device__ __forceinline__ void get_unit(uint32_t rec, StagedUnit<L> &S) {
    const __attribute__((address_space(3))) uint32_t *r = (const __attribute__((address_space(3))) uint32_t *)(uintptr_t)rec;
#pragma unroll
    for (int i = 0; i < L - 1; ++i) {
        S.bm_addr[i] = r[5 * i + 0];
        S.bm_off[i] = r[5 * i + 1];
        S.st_addr[i] = r[5 * i + 2];
        S.st_off[i] = r[5 * i + 3];
        S.cnt0[i] = r[5 * i + 4];
    }
    S.last_off = r[5 * (L - 1)];
}

// Start the LDS-DMA of unit u's spans into the slot at LDS byte address `slot`
// (16-byte aligned, staged_slot_words(L) words).  Wave-uniform arguments.  Exactly
// staged_dma_count(L) buffer loads are issued, each with lane 0 active.  `q_lo`/`q_hi` are
// the table entries of unit u and u+1 (level counts before the unit and before the next).
// chunk <= 512; the last-level stream must be 4-byte aligned.
template <int L>
__device__ __forceinline__ void stage_unit(const Dev &P, uint32_t u, uint32_t chunk, const uint32_t (&q_lo)[L - 1],
                                           const uint32_t (&q_hi)[L - 1], uint32_t slot, uint32_t lane,
                                           StagedUnit<L> &S) {
    const uint64_t e0 = (uint64_t)u * chunk;
    uint32_t space0 = (uint32_t)e0, space1 = (uint32_t)min(e0 + chunk, (uint64_t)P.n);
    uint32_t off = 0;  // bytes used so far, a multiple of 16
    auto copy = [&](__amdgpu_buffer_rsrc_t rs, uint32_t first_word, uint32_t n_words) {
        const uint32_t n4 = max((n_words + 3u) >> 2, 1u);  // 16-byte pieces, one per lane (at most 33)
        if (lane < n4)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_ptr_t)(uintptr_t)(slot + off), 16,
                                                     (int)(first_word * 4u + lane * 16u), 0, 0, 0);
        off += n4 * 16u;
    };
#pragma unroll
    for (int i = 0; i < L - 1; ++i) {
        {   // bitmap i: bits [space0, space1)
            const uint32_t w0 = space0 >> 5, n = ((space1 + 31) >> 5) - w0;
            S.bm_addr[i] = slot + off;
            S.bm_off[i] = (space0 & 31) - space0;
            copy(__builtin_amdgcn_make_buffer_rsrc((void *)P.bm[i], 0, (int)(P.bm_words[i] * 4u), 0x00020000), w0, n);
        }
        {   // stream i: codes [q_lo, q_hi), b bits each; one extra word so that a straddling read stays inside
            const uint32_t b = (uint32_t)P.bits[i];
            const uint64_t bit0 = (uint64_t)q_lo[i] * b, bit1 = (uint64_t)q_hi[i] * b;
            const uint32_t w0 = (uint32_t)(bit0 >> 5), n = (uint32_t)((bit1 + 31) >> 5) - w0 + 1;
            S.st_addr[i] = slot + off;
            S.st_off[i] = ((uint32_t)bit0 & 31) - q_lo[i] * b;
            S.cnt0[i] = q_lo[i];
            copy(__builtin_amdgcn_make_buffer_rsrc((void *)P.st[i], 0, (int)(P.st_words[i] * 4u), 0x00020000), w0, n);
        }
        space0 -= q_lo[i];
        space1 -= q_hi[i];
    }
    {   // last level: bytes [space0, space1), staged as whole dwords.  The buffer check is per dword, so the
        // descriptor reaches the end of the last dword (device allocations are 256-byte granular).
        const uint32_t w0 = space0 >> 2, n = ((space1 + 3) >> 2) - w0;
        S.last_off = slot + off + (space0 & 3) - space0;
        copy(__builtin_amdgcn_make_buffer_rsrc((void *)P.last, 0, (int)((P.last_bytes + 3u) & ~3u), 0x00020000), w0, n);
    }
}

// Rank-table entries of consecutive units, fetched one unit ahead of their use with scalar loads: entry index
// k holds the level counts before unit k.  Scalar loads are waited for on their own counter (together with LDS
// operations), so a wave that uses them does not wait for the vector-memory copies it has in flight; a vector
// load would return behind all of those.
template <int L>
struct TableWalk {
    const int32_t *base;  // table, [L-1][entries]
    uint32_t entries, at;
    uint32_t e_cur[L - 1], e_nxt[L - 1];  // entries at `at` and at `at + 1`

    __device__ __forceinline__ void start(const int32_t *table, uint32_t n_entries, uint32_t first) {
        base = table, entries = n_entries, at = first;
#pragma unroll
        for (int i = 0; i < L - 1; ++i) {
            e_cur[i] = (uint32_t)base[(size_t)i * entries + min(first, entries - 1)];
            e_nxt[i] = (uint32_t)base[(size_t)i * entries + min(first + 1, entries - 1)];
        }
    }
    // entries of unit `at` and of the unit after it; moves on to unit at + 1 and requests the entry after that
    __device__ __forceinline__ void next(uint32_t (&q_lo)[L - 1], uint32_t (&q_hi)[L - 1]) {
        ++at;
#pragma unroll
        for (int i = 0; i < L - 1; ++i) {
            q_lo[i] = e_cur[i];
            q_hi[i] = e_nxt[i];
            e_cur[i] = e_nxt[i];
            e_nxt[i] = (uint32_t)base[(size_t)i * entries + min(at + 1, entries - 1)];
        }
    }
};

// Levels START .. L-1 of up to 64 elements of a staged unit, one per lane (lanes with
// alive == false take no part).  `space` is the index, in the space of level START, of the
// first alive lane's element; the alive lanes hold consecutive elements of that space.
// cnt[i] (i >= START) is the number of level-i elements before that element (global) and is
// advanced past the group.  Same ranking as decode64, every read from LDS.
template <int L, int START>
__device__ __forceinline__ int decode_from_lds(const Dev &P, const StagedUnit<L> &S, uint32_t space, bool alive,
                                               uint32_t (&cnt)[L - 1]) {
    int v = 0;
#pragma unroll
    for (int i = START; i < L - 1; ++i) {
        const uint64_t alive_mask = __ballot(alive);
        if (alive_mask == 0) return v;  // every element has found its level: the deeper counts do not move
        const uint32_t rel = space + S.bm_off[i] + lanes_below(alive_mask);  // bit inside the staged span
        uint32_t bit = 0;
        if (alive) bit = (slds_u32(S.bm_addr[i] + (rel >> 5) * 4) >> (rel & 31)) & 1u;
        const bool taken = alive && bit;
        const uint64_t taken_mask = __ballot(taken);
        if (taken) {
            const uint32_t b = (uint32_t)P.bits[i];
            const uint32_t bitrel = (cnt[i] + lanes_below(taken_mask)) * b + S.st_off[i];
            const uint32_t a = S.st_addr[i] + (bitrel >> 5) * 4;
            const uint32_t lo = slds_u32(a), hi = slds_u32(a + 4);
            v = (int)(__builtin_amdgcn_alignbit(hi, lo, bitrel) & ((1u << b) - 1u)) - threshold_of((int)b);
        }
        alive = alive && !bit;
        space -= cnt[i];
        cnt[i] += (uint32_t)__popcll(taken_mask);
    }
    const uint64_t alive_mask = __ballot(alive);
    if (alive) v = (int)slds_u8(S.last_off + space + lanes_below(alive_mask)) - 127;
    return v;
}

// The 64 consecutive flat elements p0 .. p0+63 of a staged unit, all levels.
template <int L>
__device__ __forceinline__ int decode64_lds(const Dev &P, const StagedUnit<L> &S, uint32_t p0, bool alive,
                                            uint32_t (&cnt)[L - 1]) {
    return decode_from_lds<L, 0>(P, S, p0, alive, cnt);
}

typedef float staged_f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 staged_bf16x2 __attribute__((ext_vector_type(2)));
typedef uint32_t staged_u32x4 __attribute__((ext_vector_type(4)));

// two fp32 -> packed bf16 (round to nearest even: v_cvt_pk_bf16_f32), first value in the low half
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    const staged_f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, staged_bf16x2));
}

// A whole staged unit of `n_el` <= 512 elements starting at flat element p_begin, dequantised to bf16 into
// dst[0 .. 512) (LDS, 16-byte aligned; entries past n_el are written as zero).  Level 1 is decoded eight
// consecutive elements per lane: the lane takes its byte of the bitmap, a wave prefix sum of the bytes'
// popcounts gives the rank of its first code, and its codes are peeled off a 64-bit window of the stream.
// When level 1 leaves at most 64 elements (the tensors this format is built for), those are queued (`queue`:
// LDS, kStagedQueue uint16) and taken through the deeper levels together by ballot ranking; when it leaves
// more (dense mixes), the lanes keep their eight elements and repeat the level-1 scheme level by level.
constexpr uint32_t kStagedQueue = kStagedChunk;

// `scale_at(e)` gives the dequantisation scale of element e of the unit; it is asked once for a lane's eight
// consecutive elements (e a multiple of 8), so scale groups must be multiples of eight elements.
template <int L, class ScaleAt>
__device__ __forceinline__ void decode_unit_lds(const Dev &P, const StagedUnit<L> &S, uint32_t p_begin, uint32_t n_el,
                                                ScaleAt scale_at, uint16_t *dst, uint16_t *queue, uint32_t lane) {
    uint32_t cnt[L - 1];
#pragma unroll
    for (int i = 0; i < L - 1; ++i) cnt[i] = S.cnt0[i];
    const uint32_t b = (uint32_t)P.bits[0];
    const int thr = threshold_of((int)b);
    const uint32_t e0 = 8 * lane;
    const uint32_t n_here = e0 < n_el ? min(8u, n_el - e0) : 0u;  // elements of this lane inside the unit
    const uint32_t here = (1u << n_here) - 1u;
    uint32_t m;  // bit t: element e0 + t is level 1
    {
        const uint32_t rel = p_begin + e0 + S.bm_off[0];
        const uint32_t a = S.bm_addr[0] + (rel >> 5) * 4;
        m = __builtin_amdgcn_alignbit(slds_u32(a + 4), slds_u32(a), rel) & here;
    }
    const uint32_t n_mine = (uint32_t)__popc(m);
    const uint32_t incl = wave_scan_inclusive(n_mine);
    const uint32_t n_taken = (uint32_t)__builtin_amdgcn_readlane((int)incl, 63);
    uint32_t clo, chi;  // 64 bits of the stream from this lane's first code on
    {
        const uint32_t bitpos = (cnt[0] + incl - n_mine) * b + S.st_off[0];
        const uint32_t a = S.st_addr[0] + (bitpos >> 5) * 4;
        const uint32_t w0 = slds_u32(a), w1 = slds_u32(a + 4), w2 = slds_u32(a + 8);
        clo = __builtin_amdgcn_alignbit(w1, w0, bitpos);
        chi = __builtin_amdgcn_alignbit(w2, w1, bitpos);
    }
    int v[8];  // values of the lane's eight elements (0 until a level claims the element)
    uint32_t off = 0;
    if (b <= 4) {  // eight codes fit 32 bits
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            const uint32_t bit = (m >> t) & 1u;
            v[t] = ((int)__builtin_amdgcn_ubfe(clo, off, b) - thr) * (int)bit;
            off += bit * b;
        }
    } else {
        const uint64_t window = ((uint64_t)chi << 32) | clo;
        const uint32_t code_mask = (1u << b) - 1u;
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            const uint32_t bit = (m >> t) & 1u;
            v[t] = ((int)((uint32_t)(window >> off) & code_mask) - thr) * (int)bit;
            off += bit * b;
        }
    }
    auto store = [&]() {  // dequantise, round to bf16, one 16-byte write
        float f[8];
        const float scale = scale_at(e0);
#pragma unroll
        for (int t = 0; t < 8; ++t) f[t] = (float)v[t] * scale;
        const staged_u32x4 packed = {pack_bf16x2(f[0], f[1]), pack_bf16x2(f[2], f[3]), pack_bf16x2(f[4], f[5]),
                                     pack_bf16x2(f[6], f[7])};
        *reinterpret_cast<staged_u32x4 *>(dst + e0) = packed;
    };
    const uint32_t n_queued = n_el - n_taken;
    if (n_queued > kWave) {
        // Many elements above level 1 (a dense mix): the lane keeps its eight elements through every level.
        // `alive`: its elements no level has claimed yet; `before`: such elements in the lanes below; the
        // lane's bits of the next bitmap are consecutive from there, its codes follow from one more prefix sum.
        uint32_t alive = ~m & here;
        uint32_t before = min(e0, n_el) - (incl - n_mine);
        uint32_t space = p_begin - S.cnt0[0];  // the unit's first element in the space of the level at hand
#pragma unroll
        for (int i = 1; i < L - 1; ++i) {
            const uint32_t bi = (uint32_t)P.bits[i], code_mask = (1u << bi) - 1u;
            const int thr_i = threshold_of((int)bi);
            const uint32_t rel = space + before + S.bm_off[i];
            const uint32_t ba = S.bm_addr[i] + (rel >> 5) * 4;
            const uint32_t bits = __builtin_amdgcn_alignbit(slds_u32(ba + 4), slds_u32(ba), rel) &
                                  ((1u << __popc(alive)) - 1u);
            const uint32_t n_t = (uint32_t)__popc(bits);
            const uint32_t inc = wave_scan_inclusive(n_t);
            const uint32_t bitpos = (S.cnt0[i] + inc - n_t) * bi + S.st_off[i];
            const uint32_t wa = S.st_addr[i] + (bitpos >> 5) * 4;
            const uint32_t w0 = slds_u32(wa), w1 = slds_u32(wa + 4), w2 = slds_u32(wa + 8);
            const uint64_t window =
                ((uint64_t)__builtin_amdgcn_alignbit(w2, w1, bitpos) << 32) | __builtin_amdgcn_alignbit(w1, w0, bitpos);
            uint32_t pos = 0, idx = 0, still = 0;
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                const uint32_t a_t = (alive >> t) & 1u;
                const uint32_t bit = (bits >> idx) & a_t;
                const int val = (int)((uint32_t)(window >> pos) & code_mask) - thr_i;
                v[t] = bit ? val : v[t];
                pos += bit * bi;
                idx += a_t;
                still |= (a_t ^ bit) << t;
            }
            alive = still;
            before -= inc - n_t;
            space -= S.cnt0[i];
        }
        {   // last level: one byte per element still alive
            const uint32_t addr = S.last_off + space + before;
            const uint32_t wa = addr & ~3u, sh = (addr & 3u) * 8u;
            const uint32_t w0 = slds_u32(wa), w1 = slds_u32(wa + 4), w2 = slds_u32(wa + 8);
            const uint64_t window =
                ((uint64_t)__builtin_amdgcn_alignbit(w2, w1, sh) << 32) | __builtin_amdgcn_alignbit(w1, w0, sh);
            uint32_t pos = 0;
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                const uint32_t a_t = (alive >> t) & 1u;
                const int val = (int)((uint32_t)(window >> pos) & 0xFFu) - 127;
                v[t] = a_t ? val : v[t];
                pos += a_t * 8u;
            }
        }
        store();
        return;
    }
    store();

    // positions of the elements above level 1, in order
    {
        uint32_t z = ~m & here;
        uint32_t q = min(e0, n_el) - (incl - n_mine);
        while (z) {
            queue[q++] = (uint16_t)(e0 + (uint32_t)__builtin_ctz(z));
            z &= z - 1;
        }
    }
    cnt[0] += n_taken;
    const uint32_t space1 = p_begin - S.cnt0[0];  // the unit's first element in the space of level 2
    for (uint32_t base = 0; base < n_queued; base += kWave) {
        const bool alive = base + lane < n_queued;
        const uint32_t p = alive ? queue[base + lane] : 0u;
        const int ve = decode_from_lds<L, 1>(P, S, space1 + base, alive, cnt);
        if (alive) dst[p] = (uint16_t)f32_to_bf16_bits((float)ve * scale_at(p));
    }
}

}  // namespace ixh
