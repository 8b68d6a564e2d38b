// (3,5,8) fused decode + GEMV / skinny GEMM for gfx950, built around table
// units of 512 flat elements.
//
// Work split.  A wave owns one 512-wide column block of the weight matrix and
// walks down a block of rows, four rows per step: each 16-lane DPP row of the
// wave takes one matrix row, each lane 32 consecutive elements of it, i.e. one
// word of bitmap 0.  The lane's slice of x (32 bf16 per activation row) stays
// in registers for the whole walk.
//
// Level-1 elements (the common case).  The lane's level-1 rank is the unit's
// table entry plus a 4-step DPP scan of the popcounts of its row.  From it the
// lane loads its own 96-bit window of the 3-bit stream (one bounds-checked
// 128-bit buffer load) and aligns it with three v_alignbit.  If the bitmap word
// is all ones the window now holds the codes of elements 0..31 at bit 3*j.
// Two neighbouring codes (6 bits) index a 64-entry table spread over the
// wave's lanes (ds_bpermute), which returns the two dequantised weights
// bf16(v*scale) as one packed pair; v_dot2_f32_bf16 multiplies them with the
// matching x pair and accumulates in fp32.
//
// Other elements.  For every zero bit of the bitmap word the window is spliced:
// the codes above the zero move up by one field and the freed field is set to
// the code of value 0, so the level-1 path above stays branch-free.  The
// element itself (level 2 or 3) is described by a 16-byte record appended to a
// per-wave queue in LDS; records are resolved 64 at a time, one per lane
// (popcount of bitmap 1 from the unit's start, then a 5-bit or 8-bit code), and
// their products are added to the row's partial sum in LDS.
//
// Output.  Per (row, column block) partial sums leave through one of three
// doors: straight to bf16 y when a row has a single block, fp32 atomics into
// y32, or a [block][m][row] fp32 workspace that k_reduce_chunks sums in block
// order.
#include <stdlib.h>

#include "ixh_fast358.h"

namespace ixh {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

constexpr int kFWaves = 4;      // waves per workgroup
constexpr int kFRowSlots = 64;  // most rows one wave walks
constexpr int kFQueue = 128;    // records per wave queue

// 96-bit pattern whose every 3-bit field is code 3 (= value 0)
constexpr uint32_t kZeroCodes0 = 0xDB6DB6DBu, kZeroCodes1 = 0xB6DB6DB6u, kZeroCodes2 = 0x6DB6DB6Du;

enum : int { kOutDirect = 0, kOutAtomic = 1, kOutWorkspace = 2 };

__device__ __forceinline__ uint32_t dpp_row_shr(uint32_t v, int n) {
    switch (n) {
        case 1: return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x111, 0xf, 0xf, true);
        case 2: return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x112, 0xf, 0xf, true);
        case 4: return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x114, 0xf, 0xf, true);
        default: return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x118, 0xf, 0xf, true);
    }
}

// inclusive sum over the lanes of a 16-lane row at or below this lane
__device__ __forceinline__ uint32_t row_scan_u32(uint32_t v) {
    v += dpp_row_shr(v, 1);
    v += dpp_row_shr(v, 2);
    v += dpp_row_shr(v, 4);
    v += dpp_row_shr(v, 8);
    return v;
}

// after this, lane 15 of every 16-lane row holds the row's sum
__device__ __forceinline__ float row_sum_f32(float v) {
    v += __uint_as_float(dpp_row_shr(__float_as_uint(v), 1));
    v += __uint_as_float(dpp_row_shr(__float_as_uint(v), 2));
    v += __uint_as_float(dpp_row_shr(__float_as_uint(v), 4));
    v += __uint_as_float(dpp_row_shr(__float_as_uint(v), 8));
    return v;
}

// Resolve queued level-2/3 elements, one record per lane, and add x*w to the row sums.
template <int MT>
__device__ __forceinline__ void resolve_queue(const Dev &P, const uint4 *queue, uint32_t count, float *rowacc,
                                              const uint16_t *__restrict__ xcol, int m, int64_t ldx,
                                              float scale, uint32_t lane) {
    const uint32_t *__restrict__ b2 = P.bm[1];
    const uint32_t b2_words = P.bm_words[1];
    for (uint32_t base = 0; base < count; base += kWave) {
        const uint32_t idx = base + lane;
        if (idx < count) {
            const uint4 rec = queue[idx];
            const uint32_t r = rec.x, r0u = rec.y, q2u = rec.z;
            const uint32_t slot = rec.w >> 16, koff = rec.w & 0xFFFFu;
            // level-2 elements among bitmap-1 bits [r0u, r), and the bit at r
            // (a unit has 512 elements, so a well-formed record spans at most 17 words)
            const uint32_t wf = r0u >> 5, wl = min(r >> 5, wf + 17u);
            const uint32_t first_mask = ~0u << (r0u & 31);
            uint32_t cnt = 0;
            for (uint32_t w = wf; w < wl; ++w) {
                uint32_t bits = w < b2_words ? b2[w] : 0u;
                if (w == wf) bits &= first_mask;
                cnt += __popc(bits);
            }
            const uint32_t bits = wl < b2_words ? b2[wl] : 0u;
            uint32_t low = (1u << (r & 31)) - 1u;
            if (wl == wf) low &= first_mask;
            cnt += __popc(bits & low);
            int v = 0;
            if ((bits >> (r & 31)) & 1u) {
                const uint64_t bitpos = (uint64_t)(q2u + cnt) * 5u;
                const uint32_t wi = (uint32_t)(bitpos >> 5), s = (uint32_t)bitpos & 31u;
                const uint32_t lo = wi < P.st_words[1] ? P.st[1][wi] : 0u;
                const uint32_t hi = (s > 27 && wi + 1 < P.st_words[1]) ? P.st[1][wi + 1] : 0u;
                v = (int)((uint32_t)((((uint64_t)hi << 32) | lo) >> s) & 31u) - 15;
            } else {
                const uint32_t i3 = r - (q2u + cnt);
                v = i3 < P.last_bytes ? (int)P.last[i3] - 127 : 0;
            }
            const float w = dequant(v, scale);
#pragma unroll
            for (int j = 0; j < MT; ++j)
                if (j < m) atomicAdd(&rowacc[slot * MT + j], bf16_bits_to_f32(xcol[(int64_t)j * ldx + koff]) * w);
        }
    }
}

// what stage A of the pipeline brings in for one step: bitmap word and table entries
struct StepIn {
    uint32_t word, q1, q2, unit;
    bool valid;
};

// what stage B adds: the stream window (in flight) and the lane's ranks
struct StepWin {
    u32x4 win;
    uint32_t zeros, sh, r0_lane, r0_unit, q2;
};

template <int MT>
__global__ void __launch_bounds__(kWave *kFWaves)
k_gemv358(Dev P, const int32_t *__restrict__ prefix, uint32_t n_chunks, uint32_t rows_per_wave,
          uint32_t n_rowblocks, const uint16_t *__restrict__ x, int m, int64_t ldx, uint16_t *__restrict__ y,
          int64_t ldy, float *__restrict__ y32, float *__restrict__ ws, int out_mode) {
    __shared__ uint4 s_splice[32 * 2];
    __shared__ uint4 s_queue[kFWaves][kFQueue];
    __shared__ float s_rowacc[kFWaves][kFRowSlots * MT];

    const uint32_t tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const uint32_t quarter = lane >> 4, li = lane & 15;

    // splice table: for a zero at element e (code bit 3e) the mask of the bits
    // below it and the mask of its own field, both over the 96-bit window
    if (tid < 32) {
        const uint32_t pos = 3 * tid;
        uint32_t lm[3], f[3];
#pragma unroll
        for (int d = 0; d < 3; ++d) {
            const uint32_t base = 32u * d;
            lm[d] = pos <= base ? 0u : (pos >= base + 32 ? ~0u : (1u << (pos - base)) - 1u);
            f[d] = (pos + 3 <= base || pos >= base + 32) ? 0u : (pos >= base ? 7u << (pos - base) : 7u >> (base - pos));
        }
        s_splice[2 * tid] = make_uint4(lm[0], lm[1], lm[2], 0u);
        s_splice[2 * tid + 1] = make_uint4(f[0], f[1], f[2], 0u);
    }
    float *rowacc = s_rowacc[wave];
    for (uint32_t j = lane; j < kFRowSlots * MT; j += kWave) rowacc[j] = 0.0f;
    __syncthreads();

    const uint32_t wid = blockIdx.x * kFWaves + wave;
    if (wid >= n_chunks * n_rowblocks) return;
    const uint32_t cj = wid % n_chunks, rb = wid / n_chunks;
    const uint32_t r_begin = rb * rows_per_wave;
    const uint32_t r_end = min(r_begin + rows_per_wave, P.out_f);
    const uint32_t n_steps = (r_end - r_begin + 3) >> 2;
    const uint32_t entries = P.out_f * n_chunks + 1;
    uint4 *queue = s_queue[wave];

    // this lane's 32 activations per x row, as 16 packed bf16 pairs
    const uint16_t *xcol = x + (size_t)cj * kFastChunk;
    uint32_t xr[MT][16];
#pragma unroll
    for (int j = 0; j < MT; ++j) {
        if (j < m) {
            const uint4 *src = reinterpret_cast<const uint4 *>(xcol + (int64_t)j * ldx + li * 32);
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const uint4 v = src[t];
                xr[j][4 * t] = v.x; xr[j][4 * t + 1] = v.y; xr[j][4 * t + 2] = v.z; xr[j][4 * t + 3] = v.w;
            }
        } else {
#pragma unroll
            for (int t = 0; t < 16; ++t) xr[j][t] = 0u;
        }
    }

    // pair table: lane L holds the dequantised weights of codes (L & 7, L >> 3)
    const float scale = bf16_bits_to_f32(*P.scale);
    uint32_t pair_lut;
    {
        const int c0 = lane & 7, c1 = lane >> 3;
        const uint32_t w0 = c0 < 7 ? f32_to_bf16_bits((float)(c0 - 3) * scale) : 0u;
        const uint32_t w1 = c1 < 7 ? f32_to_bf16_bits((float)(c1 - 3) * scale) : 0u;
        pair_lut = w0 | (w1 << 16);
    }

    const __amdgpu_buffer_rsrc_t l1_rsrc =
        __builtin_amdgcn_make_buffer_rsrc((void *)P.st[0], 0, (int)(P.st_words[0] * 4u), 0x00020000);
    const uint32_t *__restrict__ b1 = P.bm[0];

    auto fetch = [&](uint32_t step) -> StepIn {
        StepIn a;
        const uint32_t row_raw = r_begin + 4 * step + quarter;
        a.valid = row_raw < r_end;
        const uint32_t row = min(row_raw, r_end - 1);
        a.unit = row * n_chunks + cj;
        a.word = b1[a.unit * 16 + li];
        a.q1 = (uint32_t)prefix[a.unit];
        a.q2 = (uint32_t)prefix[entries + a.unit];
        return a;
    };

    auto open_window = [&](const StepIn &a) -> StepWin {
        StepWin b;
        const uint32_t c = __popc(a.word);
        const uint32_t r1 = a.q1 + row_scan_u32(c) - c;
        const uint32_t bitpos = r1 * 3u;
        b.sh = bitpos & 31u;
        b.win = __builtin_amdgcn_raw_buffer_load_b128(l1_rsrc, (int)((bitpos >> 5) * 4u), 0, 0);
        b.zeros = a.valid ? ~a.word : 0u;
        b.r0_lane = a.unit * kFastChunk + li * 32u - r1;
        b.r0_unit = a.unit * kFastChunk - a.q1;
        b.q2 = a.q2;
        if (!a.valid) b.sh = 0xFFFFFFFFu;  // marks a lane whose row does not exist
        return b;
    };

    uint32_t qcount = 0;  // wave-uniform

    StepIn a_next = fetch(0);
    StepWin cur = open_window(a_next);
    a_next = fetch(1 < n_steps ? 1 : 0);

    for (uint32_t step = 0; step < n_steps; ++step) {
        const StepIn a_after = fetch(step + 2 < n_steps ? step + 2 : n_steps - 1);
        const StepWin nxt = open_window(a_next);
        a_next = a_after;

        // ---- level-1 window of this step ----
        uint32_t w0, w1, w2;
        if (cur.sh == 0xFFFFFFFFu) {
            w0 = kZeroCodes0; w1 = kZeroCodes1; w2 = kZeroCodes2;
        } else {
            w0 = __builtin_amdgcn_alignbit(cur.win.y, cur.win.x, cur.sh);
            w1 = __builtin_amdgcn_alignbit(cur.win.z, cur.win.y, cur.sh);
            w2 = __builtin_amdgcn_alignbit(cur.win.w, cur.win.z, cur.sh);
        }

        // ---- splice out the elements that are not level 1, queue them ----
        uint32_t zrem = cur.zeros, nth = 0;
        while (__ballot(zrem != 0) != 0) {
            if (qcount + kWave > kFQueue) {
                resolve_queue<MT>(P, queue, qcount, rowacc, xcol, m, ldx, scale, lane);
                qcount = 0;
            }
            const bool has = zrem != 0;
            const uint64_t has_mask = __ballot(has);
            if (has) {
                const uint32_t e = __builtin_ctz(zrem);
                zrem &= zrem - 1;
                const uint4 lm = s_splice[2 * e], fm = s_splice[2 * e + 1];
                const uint32_t s0 = w0 << 3;
                const uint32_t s1 = __builtin_amdgcn_alignbit(w1, w0, 29);
                const uint32_t s2 = __builtin_amdgcn_alignbit(w2, w1, 29);
                w0 = (w0 & lm.x) | (s0 & ~lm.x);
                w1 = (w1 & lm.y) | (s1 & ~lm.y);
                w2 = (w2 & lm.z) | (s2 & ~lm.z);
                w0 = (w0 & ~fm.x) | (kZeroCodes0 & fm.x);
                w1 = (w1 & ~fm.y) | (kZeroCodes1 & fm.y);
                w2 = (w2 & ~fm.z) | (kZeroCodes2 & fm.z);
                const uint32_t slot = qcount + lanes_below(has_mask);
                queue[slot] = make_uint4(cur.r0_lane + nth, cur.r0_unit, cur.q2,
                                         ((4 * step + quarter) << 16) | (li * 32u + e));
                ++nth;
            }
            qcount += (uint32_t)__popcll(has_mask);
        }

        // ---- 16 code pairs -> packed bf16 weights -> dot2 with the x pairs ----
        float acc[MT];
#pragma unroll
        for (int j = 0; j < MT; ++j) acc[j] = 0.0f;
#pragma unroll
        for (int t = 0; t < 16; ++t) {
            const int bit = 6 * t;  // first bit of the pair in the 96-bit window
            uint32_t addr;          // byte address for ds_bpermute: bits 7..2 = the 6-bit pair
            if (bit == 0) addr = w0 << 2;
            else if (bit == 30) addr = __builtin_amdgcn_alignbit(w1, w0, 28);
            else if (bit == 60) addr = __builtin_amdgcn_alignbit(w2, w1, 26);
            else if (bit < 32) addr = w0 >> (bit - 2);
            else if (bit < 64) addr = w1 >> (bit - 32 - 2);
            else addr = (bit - 64 - 2) == 0 ? w2 : w2 >> (bit - 64 - 2);
            const uint32_t wp = (uint32_t)__builtin_amdgcn_ds_bpermute((int)(addr & 0xFCu), (int)pair_lut);
#pragma unroll
            for (int j = 0; j < MT; ++j)
                acc[j] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, wp),
                                                         __builtin_bit_cast(bf16x2, xr[j][t]), acc[j], false);
        }
#pragma unroll
        for (int j = 0; j < MT; ++j) {
            const float total = row_sum_f32(acc[j]);
            if (li == 15) rowacc[(4 * step + quarter) * MT + j] += total;
        }
        cur = nxt;
    }

    resolve_queue<MT>(P, queue, qcount, rowacc, xcol, m, ldx, scale, lane);
    __builtin_amdgcn_wave_barrier();

    // ---- hand the row sums over ----
    const uint32_t row = r_begin + lane;
    if (row < r_end) {
#pragma unroll
        for (int j = 0; j < MT; ++j) {
            if (j >= m) break;
            const float v = rowacc[lane * MT + j];
            if (out_mode == kOutDirect)
                y[(int64_t)j * ldy + row] = (uint16_t)f32_to_bf16_bits(v);
            else if (out_mode == kOutAtomic)
                atomicAdd(&y32[(size_t)j * P.out_f + row], v);
            else
                ws[((size_t)cj * m + j) * P.out_f + row] = v;
        }
    }
}

bool fast358_supports(const Dev &P, uint32_t chunk, int m) {
    return chunk == kFastChunk && P.in_f % kFastChunk == 0 && P.n < (1u << 30) && m >= 1 && m <= 16;
}

static uint32_t pick_rows_per_wave(const Dev &P, uint32_t n_chunks) {
    // aim for at least ~4 waves per SIMD of a 256-CU part
    uint32_t rows = kFRowSlots;
    while (rows > 8 && (uint64_t)n_chunks * ((P.out_f + rows - 1) / rows) < 4096) rows >>= 1;
    return rows;
}

template <int MT>
static void launch358(const Dev &P, const int32_t *prefix, uint32_t n_chunks, uint32_t rows, const uint16_t *x,
                      int m, int64_t ldx, uint16_t *y, int64_t ldy, float *y32, float *ws, int out_mode,
                      hipStream_t s) {
    const uint32_t n_rowblocks = (P.out_f + rows - 1) / rows;
    const uint32_t waves = n_chunks * n_rowblocks;
    hipLaunchKernelGGL(k_gemv358<MT>, dim3((waves + kFWaves - 1) / kFWaves), dim3(kWave * kFWaves), 0, s, P, prefix,
                       n_chunks, rows, n_rowblocks, x, m, ldx, y, ldy, y32, ws, out_mode);
}

int launch_gemv_358(const Dev &P, const int32_t *prefix, uint32_t chunk, const uint16_t *x, int m, int64_t ldx,
                    uint16_t *y, int64_t ldy, float *y32, float *ws, bool atomic, hipStream_t s) {
    (void)chunk;
    if (((uintptr_t)x & 15u) != 0 || (m > 1 && (ldx & 7) != 0)) return IXH_EUNSUPPORTED;
    const uint32_t n_chunks = P.in_f / kFastChunk;
    const uint32_t rows = pick_rows_per_wave(P, n_chunks);
    const int out_mode = atomic ? kOutAtomic : (n_chunks == 1 ? kOutDirect : kOutWorkspace);
    if (m == 1) launch358<1>(P, prefix, n_chunks, rows, x, m, ldx, y, ldy, y32, ws, out_mode, s);
    else if (m == 2) launch358<2>(P, prefix, n_chunks, rows, x, m, ldx, y, ldy, y32, ws, out_mode, s);
    else if (m <= 4) launch358<4>(P, prefix, n_chunks, rows, x, m, ldx, y, ldy, y32, ws, out_mode, s);
    else if (m <= 8) launch358<8>(P, prefix, n_chunks, rows, x, m, ldx, y, ldy, y32, ws, out_mode, s);
    else launch358<16>(P, prefix, n_chunks, rows, x, m, ldx, y, ldy, y32, ws, out_mode, s);
    if (hipGetLastError() != hipSuccess) return IXH_ELAUNCH;
    if (out_mode == kOutWorkspace) return launch_reduce_chunks(ws, n_chunks, m, P.out_f, y, ldy, s);
    return IXH_OK;
}

}  // namespace ixh
