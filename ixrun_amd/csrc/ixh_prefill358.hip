// Fused decode + GEMM for many activation rows, for tensors that are almost all level 1 and whose first level has
// 3 bits ((3,5,8), (3,4,5,6,8), ...): Y[m, n] = sum_k X[m, k] * W[n, k] with W decoded into LDS and multiplied on the
// matrix cores (v_mfma_f32_16x16x32_bf16, fp32 accumulate); the bf16 weight never reaches HBM.
//
// Work split.  A workgroup of 8 waves (two per SIMD, one workgroup per CU) owns 128 weight rows x up to 512 activation
// rows x one K slice (a run of at most 7 unit columns of 512 k).  Per unit column it alternates between two phases:
//   decode   every wave decodes 16 of the 128 row units (four at a time, one per 16-lane DPP row, a lane 32 elements)
//            into the 128 x 512 bf16 weight tile in LDS, the way the full decode of such tensors works
//            (ixh_decode_rows358.hip): rank the lane's bitmap word, read its 96-bit code window from the staged
//            stream, splice the elements above level 1 out, look the code pairs up in the table of dequantised pairs;
//   multiply every wave multiplies 64 activation rows x the 128 weight rows x 512 k: the weight operand from the LDS
//            tile (rows 1 KB apart, the 16-byte pieces of a row XOR-swizzled with the row so that the sixteen rows of
//            an operand hit all banks), the activation operand from global memory.
// The 128-row tile is what makes the activations affordable: a workgroup reads its K slice of X once per 128 weight
// rows, and an operand register loaded from X feeds eight matrix instructions.
//
// Activations.  The matrix instruction wants a lane to hold 8 consecutive k of one activation row, sixteen rows per
// operand; loaded straight from a row-major X that is one cache line per lane and 64 tag look-ups per load
// instruction, which is twice the time the matrix instructions of the step take.  A small kernel therefore first
// re-tiles X into operand order (k_prefill_xtile: the 1 KB of an operand consecutive in memory), and the main kernel
// reads whole operands with one fully coalesced load each, two K steps ahead of their use.
//
// Elements above level 1 (a fraction of a percent in these tensors).  Their values do not depend on the level-1
// decode: the e-th such element of a row unit is the element of rank (unit start - level-1 count before the unit) + e
// in bitmap 1's domain.  At its start the workgroup computes the values of all such elements of its rows and K slice
// (a few hundred, spread over the lanes, each a chain of a few dependent reads of the nested bitmaps) into a list in
// LDS; the decode phase writes the level-1 part of a row with zeros in their places and then stores the list's
// values over the zeros.  A workgroup with more such elements than the list holds computes each where it is needed.
//
// Memory pipeline of the decode phase: the bitmap words and the 3-bit stream range of a group of four row units reach
// LDS by LDS-DMA (two stages per wave); the first two groups of a column are requested before the multiply phase of
// the column before, the other two while the first two are decoded.
//
// Partial sums of the K slices go to an fp32 workspace [slice][m][n]; the reduction kernel of ixh_prefill.hip adds them
// in slice order and rounds to bf16.
#include "ixh_rows_common.h"

namespace ixh {

typedef __bf16 q_bf16x8 __attribute__((ext_vector_type(8)));
typedef float q_f32x4 __attribute__((ext_vector_type(4)));

constexpr int kQWaves = 8;
constexpr uint32_t kQRows = 128;       // weight rows per workgroup
constexpr uint32_t kQMaxM = 512;       // activation rows per launch
constexpr uint32_t kQMaxCols = 7;      // unit columns per K slice at most
constexpr uint32_t kQMaxSlices = 16;
constexpr uint32_t kQValueCap = 1024;  // values of elements above level 1 kept in LDS
constexpr uint32_t kQStage = 1280;     // 1024 stream + 256 bitmap
// LDS map.  The pair table sits at address 0: it is addressed with (index bits | lane bits).
constexpr uint32_t kQLut = 0;                                          // [64 pairs][16 copies] words
constexpr uint32_t kQSplice = kQLut + 64 * 16 * 4;                     // [33][2] x 16 bytes
constexpr uint32_t kQTq = kQSplice + 33 * 32;                          // [128 rows][8]: level-1 counts before the slice's columns
constexpr uint32_t kQRowBase = kQTq + kQRows * (kQMaxCols + 1) * 4;    // [129]: elements above level 1 before a row (in the slice)
constexpr uint32_t kQValues = kQRowBase + 132 * 4;                     // [kQValueCap] bf16
constexpr uint32_t kQRings = kQValues + kQValueCap * 2;                // [8 waves][2 stages]
constexpr uint32_t kQTile = (kQRings + kQWaves * 2 * kQStage + 1023u) & ~1023u;  // [128][64 pieces of 16 bytes], swizzled
constexpr uint32_t kQLdsBytes = kQTile + kQRows * 1024;
static_assert(kQLdsBytes <= 160 * 1024, "LDS of a CU");
static_assert(kQSplice % 16 == 0 && kQTq % 16 == 0 && kQValues % 16 == 0 && kQRings % 16 == 0, "alignment");

__device__ __forceinline__ void q_barrier_lds() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }
__device__ __forceinline__ void q_wait_lds() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }

// 16-byte piece p (0..63) of row r of the weight tile
__device__ __forceinline__ uint32_t q_tile_addr(uint32_t r, uint32_t p) { return kQTile + r * 1024u + ((p ^ (r & 15u)) << 4); }

// LDS stores issued outside the compiler's memory model: in front of a store it can see the compiler waits for every
// LDS-DMA copy in flight, which here are the copies for the groups decoded next.  Complete after s_waitcnt lgkmcnt(0).
__device__ __forceinline__ void q_store128(uint32_t addr, uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
    const u32x4 v = {a, b, c, d};
    asm volatile("ds_write_b128 %0, %1" ::"v"(addr), "v"(v) : "memory");
}
__device__ __forceinline__ void q_store16(uint32_t addr, uint32_t v) {
    asm volatile("ds_write_b16 %0, %1" ::"v"(addr), "v"(v) : "memory");
}

// Value of the element of rank r in bitmap 1's domain, which lies in table unit `unit` (whose first element has rank
// ru there): followed down the nested bitmaps, every count taken from the unit's start, where the table holds it.
__device__ __forceinline__ int q_value_at(const Dev &P, const int32_t *__restrict__ prefix, uint32_t entries, uint32_t unit,
                                          uint32_t ru, uint32_t r) {
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
            return (int)((uint32_t)((((uint64_t)hi << 32) | lo) >> sh) & ((1u << nb) - 1u)) - threshold_of((int)nb);
        }
        r -= qu + cnt;
        ru -= qu;
    }
    return r < P.last_bytes ? (int)P.last[r] - 127 : 0;
}

// X [m_rows, in_f] row-major -> operand order: block (K step kb of 32 k, block mb of 16 rows) is 1 KB, lane l's 16 bytes
// are row 16 mb + l % 16, k 32 kb + 8 (l / 16) .. + 8; rows past m_rows read as zero.  A workgroup writes the four
// blocks {kb, kb + 1} x {mb, mb + 1}, so that it reads whole 128-byte lines of X.
__global__ void __launch_bounds__(256)
k_prefill_xtile(const uint16_t *__restrict__ x, int64_t ldx, uint32_t m_rows, uint32_t n_kb, uint32_t n_mblk,
                u32x4 *__restrict__ xt) {
    const uint32_t lane = threadIdx.x & 63u, sub = threadIdx.x >> 6;
    const uint32_t pairs_m = n_mblk >> 1;
    const uint32_t kb = (blockIdx.x / pairs_m) * 2u + (sub & 1u), mb = (blockIdx.x % pairs_m) * 2u + (sub >> 1);
    if (kb >= n_kb) return;
    const uint32_t row = mb * 16u + (lane & 15u), k = kb * 32u + (lane >> 4) * 8u;
    u32x4 v = {0u, 0u, 0u, 0u};
    if (row < m_rows) v = *reinterpret_cast<const u32x4 *>(x + (int64_t)row * ldx + k);
    xt[((size_t)kb * n_mblk + mb) * 64u + lane] = v;
}

__global__ void __launch_bounds__(kWave *kQWaves, 2)
k_prefill358(Dev P, const int32_t *__restrict__ prefix, uint32_t n_chunks, const u32x4 *__restrict__ xt, uint32_t n_mblk,
             uint32_t m_rows, float *__restrict__ ws, uint32_t n_slices, uint32_t flags) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const uint32_t quarter = lane >> 4, li = lane & 15;
    const uint32_t slice = blockIdx.x % n_slices, tile = blockIdx.x / n_slices;
    const uint32_t n0 = tile * kQRows;
    const uint32_t c_begin = slice * n_chunks / n_slices, c_end = (slice + 1) * n_chunks / n_slices;
    const uint32_t cols = c_end - c_begin;  // 1..kQMaxCols (the launcher picks n_slices accordingly)
    const uint32_t entries = P.out_f * n_chunks + 1;

    // The pair table is addressed with (index bits | lane bits), which needs it at LDS address 0 (the kernel has no
    // other LDS).  Should that ever not hold, say so in the output instead of computing garbage.
    if ((uint32_t)(uintptr_t)(lds_ptr_t)smem != 0) {
        for (uint32_t i = tid; i < min(m_rows, kQMaxM) * kQRows; i += blockDim.x) {
            const uint32_t m = i / kQRows, n = n0 + i % kQRows;
            if (n < P.out_f) ws[((size_t)slice * m_rows + m) * P.out_f + n] = __uint_as_float(0x7FC00000u);
        }
        return;
    }
    uint32_t *const lut = reinterpret_cast<uint32_t *>(smem + kQLut);
    uint4 *const splice = reinterpret_cast<uint4 *>(smem + kQSplice);
    uint32_t *const tq = reinterpret_cast<uint32_t *>(smem + kQTq);
    uint32_t *const rowbase = reinterpret_cast<uint32_t *>(smem + kQRowBase);
    uint16_t *const values = reinterpret_cast<uint16_t *>(smem + kQValues);
    uint8_t *const ring = smem + kQRings + wave * 2 * kQStage;
    const uint32_t ring_addr = kQRings + wave * 2 * kQStage;

    // ---- set-up: the slice of the rank table (it waits on memory), the tables built here ----
    const uint16_t scale_bits = *P.scale;
    for (uint32_t i = tid; i < kQRows * (kQMaxCols + 1); i += blockDim.x) {
        const uint32_t r = i >> 3, j = i & 7u;
        tq[i] = (uint32_t)prefix[(size_t)min(n0 + r, P.out_f - 1) * n_chunks + c_begin + min(j, cols)];
    }
    const float scale = bf16_bits_to_f32(scale_bits);
    for (uint32_t i = tid; i < 64 * 16; i += blockDim.x) {
        const int c0 = (i >> 4) & 7, c1 = i >> 7;
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

    // group i (0..3) of unit column ci of this wave: rows 16 wave + 4 i + quarter; LDS-DMA into stage i % 2
    auto row_of = [&](uint32_t i) { return wave * 16u + i * 4u + quarter; };
    auto issue = [&](uint32_t i, uint32_t ci) {
        const uint32_t rl = row_of(i);
        const uint32_t q1u = lds_u32(kQTq + (rl * 8u + ci) * 4u);
        const uint32_t unit = min(n0 + rl, P.out_f - 1) * n_chunks + c_begin + ci;
        uint8_t *stage = ring + (i & 1u) * kQStage;
        asm volatile("" ::: "memory");
        if (li < 13)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(l1_rsrc, (lds_ptr_t)stage, 16,
                                                     (int)(((q1u * 3u) >> 5) * 4u + li * 16u), 0, 0, 0);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(b1_rsrc, (lds_ptr_t)(stage + 1024), 4, (int)((unit * 16u + li) * 4u), 0, 0, 0);
    };
    issue(0, 0);
    issue(1, 0);

    // ---- elements above level 1 of this workgroup's rows and slice: how many before each row, then their values ----
    if (wave == 0) {
        const uint32_t r0 = 2 * lane, r1 = 2 * lane + 1;
        const uint32_t v0 = cols * kFastChunk - (tq[r0 * 8 + cols] - tq[r0 * 8]);
        const uint32_t v1 = cols * kFastChunk - (tq[r1 * 8 + cols] - tq[r1 * 8]);
        const uint32_t incl = wave_scan(v0 + v1);
        rowbase[r0] = incl - v0 - v1;
        rowbase[r1] = incl - v1;
        if (lane == 63) rowbase[kQRows] = incl;
    }
    __syncthreads();
    const bool listed = rowbase[kQRows] <= kQValueCap && !(flags & 1u);  // flags & 1: never use the list (testing)
    if (listed) {
        for (uint32_t ru = tid; ru < kQRows * cols; ru += blockDim.x) {
            const uint32_t rl = ru / cols, cu = ru - rl * cols;
            const uint32_t q_lo = tq[rl * 8 + cu], q_hi = tq[rl * 8 + cu + 1];
            const uint32_t n_esc = kFastChunk - (q_hi - q_lo);
            const uint32_t off = rowbase[rl] + cu * kFastChunk - (q_lo - tq[rl * 8]);
            const uint32_t unit = min(n0 + rl, P.out_f - 1) * n_chunks + c_begin + cu;
            const uint32_t first = unit * kFastChunk - q_lo;
            for (uint32_t e = 0; e < n_esc; ++e)
                values[off + e] = (uint16_t)f32_to_bf16_bits((float)q_value_at(P, prefix, entries, unit, first, first + e) * scale);
        }
    }
    // (the barrier in front of the first decode phase makes the list visible)

    auto splice_once = [&](uint32_t &w0, uint32_t &w1, uint32_t &w2, uint32_t &zrem) {
        const uint32_t e = zrem != 0 ? (uint32_t)__builtin_ctz(zrem) : 32u;
        zrem &= zrem - 1;
        const u32x4 lm = lds_u128(kQSplice + e * 32), fm = lds_u128(kQSplice + e * 32 + 16);
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
    // code window of group i of column ci (its data is in the ring), every element above level 1 spliced out;
    // zeros: those elements; esc0: index in the list of the lane's first one
    auto open_window = [&](uint32_t i, uint32_t ci, uint32_t &w0, uint32_t &w1, uint32_t &w2, uint32_t &zeros, uint32_t &esc0) {
        const uint32_t rl = row_of(i);
        const uint32_t stage = ring_addr + (i & 1u) * kQStage;
        const uint32_t word = lds_u32(stage + 1024 + lane * 4);
        const uint32_t q1u = lds_u32(kQTq + (rl * 8u + ci) * 4u);
        const uint32_t q1r = lds_u32(kQTq + rl * 32u);
        const uint32_t c = __popc(word);
        const uint32_t excl = row_scan(c) - c;
        const uint32_t off = excl * 3u + ((q1u * 3u) & 31u);  // bit offset inside the staged stream piece
        const uint32_t wa = stage + quarter * 256 + (off >> 5) * 4;
        const uint32_t d0 = lds_u32(wa), d1 = lds_u32(wa + 4), d2 = lds_u32(wa + 8), d3 = lds_u32(wa + 12);
        w0 = __builtin_amdgcn_alignbit(d1, d0, off);
        w1 = __builtin_amdgcn_alignbit(d2, d1, off);
        w2 = __builtin_amdgcn_alignbit(d3, d2, off);
        zeros = ~word;
        // elements above level 1: before the row in the slice, before the column in the row, before the word in the unit
        esc0 = lds_u32(kQRowBase + rl * 4u) + ci * kFastChunk - (q1u - q1r) + li * 32u - excl;
        uint32_t zrem = zeros;
        while (__ballot(zrem != 0) != 0) splice_once(w0, w1, w2, zrem);
    };

    q_f32x4 acc[4][8];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int j = 0; j < 8; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[t][j][r] = 0.0f;

    const uint32_t n_kb = n_chunks * 16u;
    const __amdgpu_buffer_rsrc_t x_rs =
        __builtin_amdgcn_make_buffer_rsrc((void *)xt, 0, (int)(n_kb * n_mblk * 1024u), 0x00020000);
    const bool multiplies = wave * 64u < m_rows;  // wave-uniform
    const uint32_t lut_lane = (lane & 15u) << 2;
    const uint32_t b_lane = kQTile + li * 1024u;  // weight operand: row 16 nb + li, piece 4 kb + quarter

    for (uint32_t ci = 0; ci < cols; ++ci) {
        q_barrier_lds();  // the multiply phase of the column before is done with the weight tile; the value list is written
        wait_vmem<0>();    // groups 0 and 1 of this column have landed
        // ---- decode phase: this wave's 16 row units, four at a time ----
        uint32_t cw0, cw1, cw2, czeros, cesc;
        open_window(0, ci, cw0, cw1, cw2, czeros, cesc);
#pragma unroll
        for (uint32_t i = 0; i < 4; ++i) {
            uint32_t wp[16];
#pragma unroll
            for (int t = 0; t < 16; ++t) {
                const int bit = 6 * t, ob = bit & 31, d = bit >> 5;
                const uint32_t lo = d == 0 ? cw0 : (d == 1 ? cw1 : cw2);
                const uint32_t hi = d == 0 ? cw1 : cw2;
                uint32_t a;  // pair index at bits 11..6
                if (ob > 26) a = __builtin_amdgcn_alignbit(hi, lo, ob - 6);
                else if (ob >= 6) a = lo >> (ob - 6);
                else a = lo << (6 - ob);
                wp[t] = lds_u32((a & 0xFC0u) | lut_lane);
            }
            const uint32_t zeros_now = czeros, esc_now = cesc;
            // the stage group i was read from is free: group i + 2 goes there; then the window of group i + 1
            if (i + 2 < 4) {
                q_wait_lds();
                issue(i + 2, ci);
            }
            if (i + 1 < 4) {
                if (i == 1) wait_vmem<2>();       // group 2 has landed (group 3's two copies may be in flight)
                else if (i == 2) wait_vmem<0>();  // group 3
                open_window(i + 1, ci, cw0, cw1, cw2, czeros, cesc);
            }
            const uint32_t rl = row_of(i);
#pragma unroll
            for (uint32_t j = 0; j < 4; ++j)
                q_store128(q_tile_addr(rl, 4 * li + j), wp[4 * j], wp[4 * j + 1], wp[4 * j + 2], wp[4 * j + 3]);
            // the values of the elements above level 1 over the zeros just written (LDS executes a wave's
            // instructions in order)
            if (zeros_now != 0) {
                uint32_t zr = zeros_now, nth = 0;
                const uint32_t unit = min(n0 + rl, P.out_f - 1) * n_chunks + c_begin + ci;
                while (zr != 0) {
                    const uint32_t e = (uint32_t)__builtin_ctz(zr);
                    zr &= zr - 1;
                    uint32_t v;
                    if (listed) {
                        v = lds_u16(kQValues + (esc_now + nth) * 2u);
                    } else {
                        // rank of the lane's first such element in bitmap 1's domain: that of the unit's first, plus
                        // those before the word in the unit
                        const uint32_t q1u = lds_u32(kQTq + (rl * 8u + ci) * 4u);
                        const uint32_t first = unit * kFastChunk - q1u;
                        const uint32_t in_unit = esc_now - (lds_u32(kQRowBase + rl * 4u) + ci * kFastChunk - (q1u - lds_u32(kQTq + rl * 32u)));
                        v = f32_to_bf16_bits((float)q_value_at(P, prefix, entries, unit, first, first + in_unit + nth) * scale);
                    }
                    q_store16(q_tile_addr(rl, 4 * li + (e >> 3)) + (e & 7u) * 2u, v);
                    ++nth;
                }
            }
        }
        // the first two groups of the next column, to land during the multiply phase
        if (ci + 1 < cols) {
            q_wait_lds();
            issue(0, ci + 1);
            issue(1, ci + 1);
        }
        q_barrier_lds();  // weight tile complete

        // ---- multiply phase: 16 K steps of 32; operands of X two steps ahead, weight operands half a step ahead ----
        if (multiplies) {
            // scalar part of the X offsets: this column, this wave's four 16-row blocks; a K step is x_step further
            const uint32_t x_col = (((c_begin + ci) * 16u) * n_mblk + wave * 4u) * 1024u, x_step = n_mblk * 1024u;
            const uint32_t x_lane = lane * 16u;
            // weight operand of K step kb, rows 16 nb + li: piece (4 kb + quarter) ^ li = (quarter ^ li) ^ (kb << 2)
            const uint32_t bb = b_lane + ((quarter ^ li) << 4);
            u32x4 a[2][4], blo[4], bhi[4];
#pragma unroll
            for (int st = 0; st < 2; ++st)
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    a[st][t] = __builtin_amdgcn_raw_buffer_load_b128(x_rs, (int)(x_lane + t * 1024), (int)(x_col + st * x_step), 0);
#pragma unroll
            for (int j = 0; j < 4; ++j) blo[j] = lds_u128(bb + j * 16384u);
#pragma unroll 1
            for (uint32_t kp = 0; kp < 8; ++kp) {
#pragma unroll
                for (int st = 0; st < 2; ++st) {
                    const uint32_t kb = kp * 2u + st;
                    const uint32_t ba = bb ^ (kb << 6), ba_next = bb ^ ((kb + 1u) << 6);
#pragma unroll
                    for (int j = 0; j < 4; ++j) bhi[j] = lds_u128(ba + 65536u + j * 16384u);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int j = 0; j < 4; ++j)
#pragma unroll
                        for (int t = 0; t < 4; ++t)
                            acc[t][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(q_bf16x8, a[st][t]),
                                                                                __builtin_bit_cast(q_bf16x8, blo[j]), acc[t][j], 0, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
                    // (after the last step this reads a neighbouring row's pieces, which nobody uses)
#pragma unroll
                    for (int j = 0; j < 4; ++j) blo[j] = lds_u128(ba_next + j * 16384u);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int j = 0; j < 4; ++j)
#pragma unroll
                        for (int t = 0; t < 4; ++t)
                            acc[t][4 + j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(q_bf16x8, a[st][t]),
                                                                                    __builtin_bit_cast(q_bf16x8, bhi[j]), acc[t][4 + j], 0, 0, 0);
                    if (kp < 7) {
#pragma unroll
                        for (int t = 0; t < 4; ++t)
                            a[st][t] = __builtin_amdgcn_raw_buffer_load_b128(x_rs, (int)(x_lane + t * 1024),
                                                                             (int)(x_col + (kb + 2u) * x_step), 0);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
    }

    // ---- partial sums of this K slice: ws[slice][m][n]; lane l holds rows 4 (l / 16) + r, column l % 16 of a block ----
    if (multiplies) {
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int j = 0; j < 8; ++j)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const uint32_t m = 64 * wave + 16 * t + 4 * quarter + r;
                    const uint32_t n = n0 + j * 16 + li;
                    if (m < m_rows && n < P.out_f) ws[((size_t)slice * m_rows + m) * P.out_f + n] = acc[t][j][r];
                }
    }
}

// K slices for a shape: one workgroup per CU; the count that makes rounds x (columns per workgroup + a start-up
// share) smallest among those that leave a slice at most kQMaxCols columns.
static uint32_t q_pick_slices(uint32_t tiles, uint32_t n_chunks) {
    static int n_cu = 0;
    if (!n_cu) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n_cu <= 0)
            n_cu = 256;
    }
    uint32_t best = 0;
    double best_cost = 1e30;
    for (uint32_t s = 1; s <= kQMaxSlices && s <= n_chunks; ++s) {
        const uint32_t cols = (n_chunks + s - 1) / s, rounds = (tiles * s + (uint32_t)n_cu - 1) / (uint32_t)n_cu;
        if (cols > kQMaxCols) continue;
        const double cost = rounds * (cols + 0.6) + 0.15 * s;  // the partial sums are written and read once per slice
        if (cost < best_cost) best_cost = cost, best = s;
    }
    return best;
}

static uint32_t q_mblocks(uint32_t m_rows) { return ((min(m_rows, kQMaxM) + 63u) / 64u) * 4u; }

size_t prefill358_workspace_bytes(const Dev &P, uint32_t m_rows) {
    const uint32_t mb = min(m_rows, kQMaxM);
    return (size_t)kQMaxSlices * mb * P.out_f * sizeof(float) + (size_t)(P.in_f / 32u) * q_mblocks(mb) * 1024u;
}

bool prefill358_supports(const Dev &P, const uint16_t *x, int64_t ldx) {
    if (!(P.n_levels >= 2 && P.bits[0] == 3 && P.in_f % kFastChunk == 0 && P.in_f != 0 && P.out_f != 0 && P.n < (1u << 30) &&
          ((uintptr_t)x & 15u) == 0 && (ldx & 7) == 0))
        return false;
    const uint32_t n_chunks = P.in_f / kFastChunk;
    return (n_chunks + kQMaxSlices - 1) / kQMaxSlices <= kQMaxCols &&
           (uint64_t)(P.in_f / 32u) * q_mblocks(kQMaxM) * 1024u < (1ull << 31);
}

int launch_prefill358(const Dev &P, const int32_t *prefix, const uint16_t *x, uint32_t m_rows, int64_t ldx, uint16_t *y,
                      int64_t ldy, float *ws, uint32_t flags, hipStream_t s) {
    static bool raised = false;
    if (!raised) {
        if (hipFuncSetAttribute(reinterpret_cast<const void *>(k_prefill358), hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)kQLdsBytes) != hipSuccess)
            return IXH_EUNSUPPORTED;
        raised = true;
    }
    const uint32_t n_chunks = P.in_f / kFastChunk, n_kb = P.in_f / 32u;
    const uint32_t tiles = (P.out_f + kQRows - 1) / kQRows;
    const uint32_t n_slices = q_pick_slices(tiles, n_chunks);
    if (n_slices == 0) return IXH_EUNSUPPORTED;
    // workspace: the partial sums first, the re-tiled activations behind them
    u32x4 *const xt = reinterpret_cast<u32x4 *>(ws + (size_t)kQMaxSlices * min(m_rows, kQMaxM) * P.out_f);
    for (uint32_t m0 = 0; m0 < m_rows; m0 += kQMaxM) {
        const uint32_t mb = min(kQMaxM, m_rows - m0), n_mblk = q_mblocks(mb);
        hipLaunchKernelGGL(k_prefill_xtile, dim3((n_kb / 2u) * (n_mblk / 2u)), dim3(256), 0, s, x + (int64_t)m0 * ldx, ldx, mb,
                           n_kb, n_mblk, xt);
        hipLaunchKernelGGL(k_prefill358, dim3(tiles * n_slices), dim3(kWave * kQWaves), kQLdsBytes, s, P, prefix, n_chunks,
                           (const u32x4 *)xt, n_mblk, mb, ws, n_slices, flags);
        if (hipGetLastError() != hipSuccess) return IXH_ELAUNCH;
        const int rc = launch_prefill_reduce(ws, mb, P.out_f, n_slices, y + (int64_t)m0 * ldy, ldy, s);
        if (rc) return rc;
    }
    return IXH_OK;
}

}  // namespace ixh
