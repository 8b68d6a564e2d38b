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
//            tile (rows 1 KB apart, the 16-byte pieces of a row swizzled so that neither the sixteen rows of an
//            operand nor the sixteen lanes that store a row unit collide on a bank), the activation operand from global memory.
// The 128-row tile is what makes the activations affordable: a workgroup reads its K slice of X once per 128 weight
// rows, and an operand register loaded from X feeds eight matrix instructions.
//
// Activations.  The matrix instruction wants a lane to hold 8 consecutive k of one activation row, sixteen rows per
// operand; loaded straight from a row-major X that is one cache line per lane and 64 tag look-ups per load
// instruction, which is twice the time the matrix instructions of the step take.  A small kernel therefore first
// re-tiles X into operand order (k_prefill_xtile: the 1 KB of an operand consecutive in memory), and the main kernel
// reads whole operands with one fully coalesced load each, two K steps ahead of their use.
//
// Elements above level 1 (up to a few percent in these tensors).  Their values do not depend on the level-1 decode:
// the e-th such element of a row unit is the element of rank (unit start - level-1 count before the unit) + e in
// bitmap 1's domain.  At its start the workgroup computes the values (int8) of all such elements of its rows and K
// slice, one element per lane and round (each a chain of a few dependent reads of the nested bitmaps), into one list
// per unit column in global memory, rows in order; a column's list (at most 2048 values) is copied to LDS by LDS-DMA
// during the multiply phase of the column before, together with the count of such elements before each row in that
// column.  The decode phase writes the level-1 part of a row with zeros in their places and then stores the
// dequantised list values over the zeros.  A column with more such elements than the list holds computes each where
// it is needed.
//
// Memory pipeline of the decode phase: the bitmap words and the 3-bit stream range of a group of four row units reach
// LDS by LDS-DMA (two stages per wave); the first two groups of a column are requested before the multiply phase of
// the column before, the other two while the first two are decoded.
//
// Partial sums of the K slices go to an fp32 workspace in accumulator order (whole 1 KB stores); a second kernel adds
// them in slice order and rounds to bf16.
#include "ixh_prefill358.h"
#include "ixh_rows_common.h"

namespace ixh {

typedef __bf16 q_bf16x8 __attribute__((ext_vector_type(8)));
typedef float q_f32x4 __attribute__((ext_vector_type(4)));

constexpr int kQWaves = 8;
constexpr uint32_t kQRows = 128;       // weight rows per workgroup
constexpr uint32_t kQMaxM = 512;       // activation rows per launch
constexpr uint32_t kQMaxCols = 7;      // unit columns per K slice at most
constexpr uint32_t kQMaxSlices = 16;
constexpr uint32_t kQValueCap = 2048;  // values (int8) of a unit column's elements above level 1 kept in LDS
constexpr uint32_t kQStage = 1280;     // 1024 stream + 256 bitmap
// LDS map.  The pair table sits at address 0: it is addressed with (index bits | lane bits).
constexpr uint32_t kQLut = 0;                                          // [64 pairs][16 copies] words
constexpr uint32_t kQSplice = kQLut + 64 * 16 * 4;                     // [33][2] x 16 bytes
constexpr uint32_t kQTq = kQSplice + 33 * 32;                          // [128 rows][8]: level-1 counts before the slice's columns
constexpr uint32_t kQRowBase = kQTq + kQRows * (kQMaxCols + 1) * 4;    // [2][132] u16: elements above level 1 before a row in a column (saturated), for the column being decoded and the next
constexpr uint32_t kQValues = kQRowBase + 132 * 4;                     // [kQValueCap] int8
constexpr uint32_t kQRings = kQValues + kQValueCap;                    // [8 waves][2 stages]
constexpr uint32_t kQTile = (kQRings + kQWaves * 2 * kQStage + 1023u) & ~1023u;  // [128][64 pieces of 16 bytes], swizzled
constexpr uint32_t kQLdsBytes = kQTile + kQRows * 1024;
constexpr uint32_t kQListBytes = kQMaxCols * kQValueCap;  // a workgroup's value lists in global memory, one per column
static_assert(kQLdsBytes <= 160 * 1024, "LDS of a CU");
static_assert(kQSplice % 16 == 0 && kQTq % 16 == 0 && kQValues % 16 == 0 && kQRings % 16 == 0, "alignment");

struct QReload { static constexpr bool value = true; };
struct QLast { static constexpr bool value = false; };

__device__ __forceinline__ void q_barrier_lds() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }
__device__ __forceinline__ void q_wait_lds() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }
// "at most N vector-memory operations outstanding", as an instruction the compiler sees: it keeps its own count of
// what is in flight and, not knowing about a wait written in assembly, would later wait again for copies that have
// long landed, at a point where that also waits for the ones issued since.
template <int N>
__device__ __forceinline__ void q_wait_vmem() {
    static_assert(N >= 0 && N < 16, "low four bits of vmcnt");
    __builtin_amdgcn_s_waitcnt(0x0F70 | N);  // expcnt and lgkmcnt at their maxima: no wait on them
    asm volatile("" ::: "memory");
}

// 16-byte piece p (0..63) of row r of the weight tile sits at slot p ^ (p >> 4) ^ (r & 15) of the row's 1 KB: the
// sixteen rows of a weight operand (same p) then hit sixteen different groups of four banks, and so do the sixteen
// lanes of a row unit when each stores the j-th of its four consecutive pieces (p = 4 lane + j).
__device__ __forceinline__ uint32_t q_tile_addr(uint32_t r, uint32_t p) {
    return kQTile + r * 1024u + ((p ^ (p >> 4) ^ (r & 15u)) << 4);
}

// LDS stores issued outside the compiler's memory model: in front of a store it can see the compiler waits for every
// LDS-DMA copy in flight, which here are the copies for the groups decoded next.  Complete after s_waitcnt lgkmcnt(0).
__device__ __forceinline__ void q_store128(uint32_t addr, uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
    const u32x4 v = {a, b, c, d};
    asm volatile("ds_write_b128 %0, %1" ::"v"(addr), "v"(v) : "memory");
}
__device__ __forceinline__ void q_store16(uint32_t addr, uint32_t v) {
    asm volatile("ds_write_b16 %0, %1" ::"v"(addr), "v"(v) : "memory");
}

// LDS reads issued outside the compiler's memory model, for the part of the decode phase that runs while the copies
// for the groups decoded later are in flight: in front of a read it can see, the compiler waits for those copies.
// Eight table look-ups in place (the address register receives the data), without the wait: the results are there
// after q_release16 of the same registers (which the compiler must see as redefining them, or it may copy a register
// before its read has returned).
__device__ __forceinline__ void q_issue8(uint32_t (&r)[16], int h) {
    asm volatile(
        "ds_read_b32 %0, %0\n\t"
        "ds_read_b32 %1, %1\n\t"
        "ds_read_b32 %2, %2\n\t"
        "ds_read_b32 %3, %3\n\t"
        "ds_read_b32 %4, %4\n\t"
        "ds_read_b32 %5, %5\n\t"
        "ds_read_b32 %6, %6\n\t"
        "ds_read_b32 %7, %7"
        : "+v"(r[8 * h]), "+v"(r[8 * h + 1]), "+v"(r[8 * h + 2]), "+v"(r[8 * h + 3]), "+v"(r[8 * h + 4]), "+v"(r[8 * h + 5]),
          "+v"(r[8 * h + 6]), "+v"(r[8 * h + 7])
        :
        : "memory");
}
__device__ __forceinline__ void q_release16(uint32_t (&r)[16]) {
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]), "+v"(r[4]), "+v"(r[5]), "+v"(r[6]), "+v"(r[7]), "+v"(r[8]),
                   "+v"(r[9]), "+v"(r[10]), "+v"(r[11]), "+v"(r[12]), "+v"(r[13]), "+v"(r[14]), "+v"(r[15])
                 :
                 : "memory");
}
__device__ __forceinline__ void q_issue_i8(uint32_t addr, int &out) {
    asm volatile("ds_read_i8 %0, %1" : "=&v"(out) : "v"(addr) : "memory");
}
__device__ __forceinline__ void q_release2(int &a, int &b) {
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a), "+v"(b) : : "memory");
}
__device__ __forceinline__ int q_read_i8(uint32_t addr) {
    int v;
    asm volatile("ds_read_i8 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(addr) : "memory");
    return v;
}
__device__ __forceinline__ uint32_t q_read_u32(uint32_t addr) {
    uint32_t v;
    asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(addr) : "memory");
    return v;
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
             uint32_t m_rows, float *__restrict__ ws, int8_t *__restrict__ lists, uint32_t n_slices, uint32_t flags) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    // (not const: re-derived from an opaque copy of the lane number at the top of every column, so that the compiler
    // does not carry the dozens of lane-dependent addresses of the decode phase in registers through the multiply phase)
    uint32_t lane_v = lane, quarter = lane >> 4, li = lane & 15;
    const uint32_t slice = blockIdx.x % n_slices, tile = blockIdx.x / n_slices;
    const uint32_t n0 = tile * kQRows;
    const uint32_t c_begin = slice * n_chunks / n_slices, c_end = (slice + 1) * n_chunks / n_slices;
    const uint32_t cols = c_end - c_begin;  // 1..kQMaxCols (the launcher picks n_slices accordingly)
    const uint32_t entries = P.out_f * n_chunks + 1;

    // The pair table is addressed with (index bits | lane bits), which needs it at LDS address 0 (the kernel has no
    // other LDS).  Should that ever not hold, say so in the output instead of computing garbage.
    if ((uint32_t)(uintptr_t)(lds_ptr_t)smem != 0) {
        float *const mine = ws + ((size_t)slice * (gridDim.x / n_slices) + tile) * (kQMaxM * kQRows);
        for (uint32_t i = tid; i < kQMaxM * kQRows; i += blockDim.x) mine[i] = __uint_as_float(0x7FC00000u);
        return;
    }
    uint32_t *const lut = reinterpret_cast<uint32_t *>(smem + kQLut);
    uint4 *const splice = reinterpret_cast<uint4 *>(smem + kQSplice);
    uint32_t *const tq = reinterpret_cast<uint32_t *>(smem + kQTq);
    uint16_t *const rowbase = reinterpret_cast<uint16_t *>(smem + kQRowBase);
    int8_t *const values = reinterpret_cast<int8_t *>(smem + kQValues);
    int8_t *const my_lists = lists + (size_t)blockIdx.x * kQListBytes;
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

    // ---- elements above level 1 of this workgroup's rows and slice ----
    // Per column: how many before each row (a scan over the 128 rows by one wave; the counts of all columns go to
    // the weight tile's memory, which is free until the first decode phase), and the column totals.
    uint32_t *const offs = reinterpret_cast<uint32_t *>(smem + kQTile);  // [cols][132]
    auto scan_column = [&](uint32_t cu, uint32_t *dst32, uint16_t *dst16) {  // one wave; either destination may be null
        const uint32_t r0 = 2 * lane, r1 = 2 * lane + 1;
        const uint32_t v0 = kFastChunk - (tq[r0 * 8 + cu + 1] - tq[r0 * 8 + cu]);
        const uint32_t v1 = kFastChunk - (tq[r1 * 8 + cu + 1] - tq[r1 * 8 + cu]);
        const uint32_t incl = wave_scan(v0 + v1);
        if (dst32) {
            dst32[r0] = incl - v0 - v1;
            dst32[r1] = incl - v1;
            if (lane == 63) dst32[kQRows] = incl;
        }
        if (dst16) {
            dst16[r0] = (uint16_t)min(incl - v0 - v1, 0xFFFFu);
            dst16[r1] = (uint16_t)min(incl - v1, 0xFFFFu);
            if (lane == 63) dst16[kQRows] = (uint16_t)min(incl, 0xFFFFu);
        }
    };
    if (wave < cols) scan_column(wave, offs + wave * 132, wave == 0 ? rowbase : nullptr);
    __syncthreads();
    // The values: one element per lane and round over all columns' lists; entry idx of column cu is the idx-th such
    // element of the column, rows in order: its row by bisection of the rows' first indices.
    if (!(flags & 1u)) {  // flags & 1: no lists, every element is computed where it is needed (testing)
        uint32_t cbase[kQMaxCols + 1];  // first item of each column's list in the workgroup's run of items
        cbase[0] = 0;
#pragma unroll
        for (uint32_t cu = 0; cu < kQMaxCols; ++cu) {
            const uint32_t n = cu < cols ? offs[cu * 132 + kQRows] : 0u;
            cbase[cu + 1] = cbase[cu] + (n <= kQValueCap ? n : 0u);  // a column that does not fit has no list
        }
        for (uint32_t g = tid; g < cbase[kQMaxCols]; g += blockDim.x) {
            uint32_t cu = 0;
#pragma unroll
            for (uint32_t j = 1; j < kQMaxCols; ++j)
                if (cbase[j] <= g) cu = j;
            uint32_t idx = g;
#pragma unroll
            for (uint32_t j = 1; j < kQMaxCols; ++j)
                if (cu == j) idx = g - cbase[j];
            const uint32_t *const off = offs + cu * 132;
            uint32_t lo = 0, hi = kQRows;
            while (hi - lo > 1) {
                const uint32_t mid = (lo + hi) >> 1;
                if (off[mid] <= idx) lo = mid;
                else hi = mid;
            }
            const uint32_t rl = lo, e = idx - off[rl], q_lo = tq[rl * 8 + cu];
            const uint32_t unit = min(n0 + rl, P.out_f - 1) * n_chunks + c_begin + cu;
            const uint32_t first = unit * kFastChunk - q_lo;
            const int8_t v = (int8_t)q_value_at(P, prefix, entries, unit, first, first + e);
            my_lists[cu * kQValueCap + idx] = v;
            if (cu == 0) values[idx] = v;
        }
    }
    // (the wait and the barrier in front of the first decode phase complete the stores and make column 0's list
    // visible)

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
    // One group's decode state: the code window (every element above level 1 spliced out), those elements, and the
    // index in the value list of the lane's first one.
    struct Window {
        uint32_t w0, w1, w2, zeros, esc;
    };
    // Windows of groups i and i + 1 of column ci (their data is in the ring), in lockstep, so that every trip to LDS
    // serves both.
    auto open_pair = [&](uint32_t i, uint32_t ci, Window &A, Window &B) {
        const uint32_t rl_a = row_of(i), rl_b = row_of(i + 1);
        const uint32_t stage_a = ring_addr + (i & 1u) * kQStage, stage_b = ring_addr + ((i + 1) & 1u) * kQStage;
        const uint32_t word_a = lds_u32(stage_a + 1024 + lane_v * 4), word_b = lds_u32(stage_b + 1024 + lane_v * 4);
        const uint32_t q1u_a = lds_u32(kQTq + (rl_a * 8u + ci) * 4u), q1u_b = lds_u32(kQTq + (rl_b * 8u + ci) * 4u);
        const uint32_t rb = kQRowBase + (ci & 1u) * 264u;
        const uint32_t rb_a = lds_u16(rb + rl_a * 2u), rb_b = lds_u16(rb + rl_b * 2u);
        const uint32_t c_a = __popc(word_a), c_b = __popc(word_b);
        const uint32_t excl_a = row_scan(c_a) - c_a, excl_b = row_scan(c_b) - c_b;
        const uint32_t off_a = excl_a * 3u + ((q1u_a * 3u) & 31u), off_b = excl_b * 3u + ((q1u_b * 3u) & 31u);
        const uint32_t wa = stage_a + quarter * 256 + (off_a >> 5) * 4, wb = stage_b + quarter * 256 + (off_b >> 5) * 4;
        const uint32_t a0 = lds_u32(wa), a1 = lds_u32(wa + 4), a2 = lds_u32(wa + 8), a3 = lds_u32(wa + 12);
        const uint32_t b0 = lds_u32(wb), b1 = lds_u32(wb + 4), b2 = lds_u32(wb + 8), b3 = lds_u32(wb + 12);
        A.w0 = __builtin_amdgcn_alignbit(a1, a0, off_a);
        A.w1 = __builtin_amdgcn_alignbit(a2, a1, off_a);
        A.w2 = __builtin_amdgcn_alignbit(a3, a2, off_a);
        B.w0 = __builtin_amdgcn_alignbit(b1, b0, off_b);
        B.w1 = __builtin_amdgcn_alignbit(b2, b1, off_b);
        B.w2 = __builtin_amdgcn_alignbit(b3, b2, off_b);
        A.zeros = ~word_a;
        B.zeros = ~word_b;
        // elements above level 1 of the column: before the row, before the word in the unit
        A.esc = rb_a + li * 32u - excl_a;
        B.esc = rb_b + li * 32u - excl_b;
        uint32_t zrem_a = A.zeros, zrem_b = B.zeros;
        while (__ballot((zrem_a | zrem_b) != 0) != 0) {
            splice_once(A.w0, A.w1, A.w2, zrem_a);
            splice_once(B.w0, B.w1, B.w2, zrem_b);
        }
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
    uint32_t lut_lane, b_lane;

    const __amdgpu_buffer_rsrc_t list_rs =
        __builtin_amdgcn_make_buffer_rsrc((void *)my_lists, 0, (int)kQListBytes, 0x00020000);
    for (uint32_t ci = 0; ci < cols; ++ci) {
        // What this wave asked for has arrived: groups 0 and 1 of this column; from waves 0 and 1 the column's value
        // list; at the first column the stores of the lists.
        q_wait_vmem<0>();
        asm volatile("" : "+v"(lane_v));
        quarter = lane_v >> 4, li = lane_v & 15u;
        lut_lane = li << 2;
        b_lane = kQTile + li * 1024u;  // weight operand: row 16 nb + li, piece 4 kb + quarter
        // the next column's counts, while none of this wave's copies is in flight (the buffer they go to was last read
        // in the decode phase of the column before)
        if (wave == 0 && ci + 1 < cols) scan_column(ci + 1, nullptr, rowbase + ((ci + 1) & 1u) * 132u);
        // ---- decode phase: this wave's 16 row units, four at a time, two groups of four in lockstep ----
        Window A, B;
        bool listed = false;  // this column has its value list in LDS (set behind the barrier)
        auto lut_addresses = [&](const Window &W, uint32_t (&la)[16]) {
#pragma unroll
            for (int t = 0; t < 16; ++t) {
                const int bit = 6 * t, ob = bit & 31, d = bit >> 5;
                const uint32_t lo = d == 0 ? W.w0 : (d == 1 ? W.w1 : W.w2);
                const uint32_t hi = d == 0 ? W.w1 : W.w2;
                uint32_t a;  // pair index at bits 11..6
                if (ob > 26) a = __builtin_amdgcn_alignbit(hi, lo, ob - 6);
                else if (ob >= 6) a = lo >> (ob - 6);
                else a = lo << (6 - ob);
                la[t] = (a & 0xFC0u) | lut_lane;
            }
        };
        // the values of a lane's elements above level 1 over the zeros the lane has just written (LDS executes a wave's
        // instructions in order); `first` is the list's value for the first of them, already read
        auto patch = [&](uint32_t i, const Window &W, int first) {
            if (W.zeros == 0) return;
            const uint32_t rl = row_of(i);
            const uint32_t unit = min(n0 + rl, P.out_f - 1) * n_chunks + c_begin + ci;
            uint32_t zr = W.zeros, nth = 0;
            while (zr != 0) {
                const uint32_t e = (uint32_t)__builtin_ctz(zr);
                zr &= zr - 1;
                int v = first;
                if (!listed) {
                    // rank of the lane's first such element in bitmap 1's domain: that of the unit's first, plus
                    // those before the word in the unit
                    const uint32_t first_rank = unit * kFastChunk - q_read_u32(kQTq + (rl * 8u + ci) * 4u);
                    const uint32_t in_unit = W.esc - (q_read_u32(kQRowBase + (ci & 1u) * 264u + (rl & ~1u) * 2u) >> ((rl & 1u) * 16u) & 0xFFFFu);
                    v = q_value_at(P, prefix, entries, unit, first_rank, first_rank + in_unit + nth);
                } else if (nth != 0) {
                    v = q_read_i8(kQValues + W.esc + nth);
                }
                q_store16(q_tile_addr(rl, 4 * li + (e >> 3)) + (e & 7u) * 2u, f32_to_bf16_bits((float)v * scale));
                ++nth;
            }
        };
        // groups i and i + 1, in lockstep: the pairs of dequantised weights from the table, then into the weight tile
        uint32_t wa[16], wb[16];  // table addresses, then the pairs read from them
        auto look_up_pair = [&]() {
            lut_addresses(A, wa);
            lut_addresses(B, wb);
            q_issue8(wa, 0);
            q_issue8(wa, 1);
            q_issue8(wb, 0);
            q_issue8(wb, 1);
            q_release16(wa);
            q_release16(wb);
        };
        auto store_pair = [&](uint32_t i) {
            int va, vb;
            // (a lane without such elements reads a neighbour's value, or a byte behind the list, and drops it; a
            // column without a list has indices beyond it)
            q_issue_i8(kQValues + min(A.esc, kQValueCap), va);
            q_issue_i8(kQValues + min(B.esc, kQValueCap), vb);
            const uint32_t rl_a = row_of(i), rl_b = row_of(i + 1);
#pragma unroll
            for (uint32_t j = 0; j < 4; ++j)
                q_store128(q_tile_addr(rl_a, 4 * li + j), wa[4 * j], wa[4 * j + 1], wa[4 * j + 2], wa[4 * j + 3]);
#pragma unroll
            for (uint32_t j = 0; j < 4; ++j)
                q_store128(q_tile_addr(rl_b, 4 * li + j), wb[4 * j], wb[4 * j + 1], wb[4 * j + 2], wb[4 * j + 3]);
            q_release2(va, vb);
            patch(i, A, va);
            patch(i + 1, B, vb);
        };
        // Groups 0 and 1 are in the ring: opening their windows frees the two stages for groups 2 and 3, whose copies
        // then run under the table look-ups and tile stores of groups 0 and 1.  Everything up to the first store into
        // the weight tile is done in front of the barrier: a wave that leaves the multiply phase early uses the wait.
        open_pair(0, ci, A, B);
        q_wait_lds();
        issue(2, ci);
        issue(3, ci);
        look_up_pair();
        q_barrier_lds();  // the multiply phase of the column before is done with the weight tile; this column's list is in LDS
        listed = lds_u16(kQRowBase + (ci & 1u) * 264u + kQRows * 2u) <= kQValueCap && !(flags & 1u);
        store_pair(0);
        q_wait_vmem<0>();  // groups 2 and 3 have landed
        open_pair(2, ci, A, B);
        // the first two groups of the next column, to land during the multiply phase
        if (ci + 1 < cols) {
            q_wait_lds();
            issue(0, ci + 1);
            issue(1, ci + 1);
        }
        look_up_pair();
        store_pair(2);
        // the activation operands of the first two K steps, requested in front of the barrier
        const uint32_t x_col = (((c_begin + ci) * 16u) * n_mblk + wave * 4u) * 1024u, x_step = n_mblk * 1024u;
        const uint32_t x_lane = lane_v * 16u;
        u32x4 a[2][4];
        if (multiplies) {
            // (first all of step 0, then all of step 1: the order in which the loop below reloads them, so that
            // "all but the newest four have arrived" is the wait in front of every step)
#pragma unroll
            for (int st = 0; st < 2; ++st) {
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    a[st][t] = __builtin_amdgcn_raw_buffer_load_b128(x_rs, (int)(x_lane + t * 1024), (int)(x_col + st * x_step), 0);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        q_barrier_lds();  // weight tile complete; nobody reads this column's counts and list any more
        if (ci + 1 < cols) {
            // the next column's list (waves 0 and 1 copy 1 KB each), in place during the multiply phase
            if (wave < 2)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(list_rs, (lds_ptr_t)(smem + kQValues + wave * 1024u), 16,
                                                         (int)((ci + 1) * kQValueCap + wave * 1024u + lane * 16u), 0, 0, 0);
        }

        // ---- multiply phase: 16 K steps of 32; operands of X two steps ahead, weight operands half a step ahead ----
        if (multiplies) {
            // weight operand of K step kb, rows 16 nb + li: piece p = 4 kb + quarter at slot p ^ (p >> 4) ^ li, which is
            // (quarter ^ li) ^ (kb << 2 | kb >> 2)
            const uint32_t bb = b_lane + ((quarter ^ li) << 4);
            u32x4 blo[4], bhi[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) blo[j] = lds_u128(bb + j * 16384u);
            // K step kb with the operands a[st]; `reload`: fetch the operands of step kb + 2 into a[st] afterwards
            auto step = [&](uint32_t kb, int st, auto reload) {
                const uint32_t kn = kb + 1u;
                const uint32_t ba = bb ^ (((kb << 2) | (kb >> 2)) << 4), ba_next = bb ^ (((kn << 2) | ((kn >> 2) & 3u)) << 4);
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
                if (decltype(reload)::value) {
#pragma unroll
                    for (int t = 0; t < 4; ++t)
                        a[st][t] = __builtin_amdgcn_raw_buffer_load_b128(x_rs, (int)(x_lane + t * 1024),
                                                                         (int)(x_col + (kb + 2u) * x_step), 0);
                }
                __builtin_amdgcn_sched_barrier(0);
            };
            // no branch around the reloads inside the loop: with one, the compiler's count of what is in flight
            // differs between the paths and it waits for everything, the operands just requested included
#pragma unroll 1
            for (uint32_t kp = 0; kp < 7; ++kp) {
                step(kp * 2u, 0, QReload{});
                step(kp * 2u + 1u, 1, QReload{});
            }
            step(14u, 0, QLast{});
            step(15u, 1, QLast{});
        }
    }

    // ---- partial sums of this K slice, in accumulator order: [slice][tile][wave][t][j][lane] x 4 floats, so that a
    // store instruction writes 1 KB of consecutive memory (lane l of block (t, j) holds rows 64 wave + 16 t + 4 (l / 16)
    // + r, column 16 j + l % 16 of the tile) ----
    if (multiplies) {
        q_f32x4 *const dst = reinterpret_cast<q_f32x4 *>(ws) +
                             ((((size_t)slice * (gridDim.x / n_slices) + tile) * kQWaves + wave) * 32u) * 64u + lane;
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int j = 0; j < 8; ++j) dst[(t * 8 + j) * 64] = acc[t][j];
    }
}

// y[m][n] = bf16(sum over the K slices, in slice order) from the partial sums in accumulator order; a thread takes one
// lane's four floats of one block.
__global__ void __launch_bounds__(256)
k_prefill358_reduce(const q_f32x4 *__restrict__ ws, uint32_t m_rows, uint32_t out_f, uint32_t tiles, uint32_t n_slices,
                    uint16_t *__restrict__ y, int64_t ldy) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;  // ((tile * 8 + wave) * 32 + t * 8 + j) * 64 + lane
    const uint32_t lane = i & 63u, blk = (i >> 6) & 31u, wave = (i >> 11) & 7u, tile = i >> 14;
    if (tile >= tiles) return;
    const uint32_t m0 = 64u * wave + 16u * (blk >> 3) + 4u * (lane >> 4), n = tile * kQRows + 16u * (blk & 7u) + (lane & 15u);
    if (m0 >= m_rows || n >= out_f) return;
    const size_t per_slice = (size_t)tiles * kQWaves * 32u * 64u;
    q_f32x4 sum = ws[i];
    for (uint32_t sl = 1; sl < n_slices; ++sl) {
        const q_f32x4 v = ws[sl * per_slice + i];
#pragma unroll
        for (int r = 0; r < 4; ++r) sum[r] += v[r];
    }
#pragma unroll
    for (int r = 0; r < 4; ++r)
        if (m0 + r < m_rows) y[(int64_t)(m0 + r) * ldy + n] = (uint16_t)f32_to_bf16_bits(sum[r]);
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

// partial sums of the most slices, whole tiles of 512 x 128
static size_t q_sums_bytes(size_t tiles) { return (size_t)kQMaxSlices * tiles * kQMaxM * kQRows * sizeof(float); }
static uint32_t q_mblocks(uint32_t m_rows) { return ((min(m_rows, kQMaxM) + 63u) / 64u) * 4u; }

size_t prefill358_workspace_bytes(const Dev &P, uint32_t m_rows) {
    const uint32_t mb = min(m_rows, kQMaxM);
    const size_t tiles = (P.out_f + kQRows - 1) / kQRows;
    return q_sums_bytes(tiles) + (size_t)(P.in_f / 32u) * q_mblocks(mb) * 1024u + tiles * kQMaxSlices * kQListBytes;
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
    // workspace: the partial sums first, the re-tiled activations behind them, then the workgroups' value lists
    u32x4 *const xt = reinterpret_cast<u32x4 *>(reinterpret_cast<uint8_t *>(ws) + q_sums_bytes(tiles));
    int8_t *const lists = reinterpret_cast<int8_t *>(xt) + (size_t)n_kb * q_mblocks(min(m_rows, kQMaxM)) * 1024u;
    for (uint32_t m0 = 0; m0 < m_rows; m0 += kQMaxM) {
        const uint32_t mb = min(kQMaxM, m_rows - m0), n_mblk = q_mblocks(mb);
        hipLaunchKernelGGL(k_prefill_xtile, dim3((n_kb / 2u) * (n_mblk / 2u)), dim3(256), 0, s, x + (int64_t)m0 * ldx, ldx, mb,
                           n_kb, n_mblk, xt);
        hipLaunchKernelGGL(k_prefill358, dim3(tiles * n_slices), dim3(kWave * kQWaves), kQLdsBytes, s, P, prefix, n_chunks,
                           (const u32x4 *)xt, n_mblk, mb, ws, lists, n_slices, flags);
        if (hipGetLastError() != hipSuccess) return IXH_ELAUNCH;
        hipLaunchKernelGGL(k_prefill358_reduce, dim3(tiles * 64u), dim3(256), 0, s, (const q_f32x4 *)ws, mb, P.out_f, tiles,
                           n_slices, y + (int64_t)m0 * ldy, ldy);
        if (hipGetLastError() != hipSuccess) return IXH_ELAUNCH;
    }
    return IXH_OK;
}

}  // namespace ixh
