// (3,5,8) fused decode + GEMV for one activation row when every level is well populated (e.g. the 55 / 40 / 5 %
// mix of real LLM weights), where decoding element by element costs ~45 instructions per weight and lane.
//
// This kernel does not decode by position.  The codes of a level are dense in their stream, so the dot product of
// a run of weights is taken level by level over whole codes at fixed positions:
//     sum_k w_k x_k = sum_{k in level 1} w_k x_k + sum_{k in level 2} w_k x_k + sum_{k in level 3} w_k x_k
// and what depends on the bitmaps is moved to the activations: the x values of a span are scattered ("compacted")
// into three arrays in LDS, one per level, in the order of that level's codes.  Scattering costs an LDS write per
// weight and about nine integer instructions (two elements per step, with the running slot addresses in packed
// 16-bit halves); the three dense passes then cost about one instruction per weight.
//
// A wave takes spans of up to 2048 consecutive elements of one weight row (four 512-element table units).  The
// rank table gives the span's first code in every stream and its level counts.  Lane l owns bitmap word l (32
// elements, 16 x pairs in registers): popcount + wave prefix sums give the lane's first slot in each compacted array
// (bitmap 1 is read at the lane's first element not in level 1).  The dense passes split each level's codes evenly over
// the 64 lanes (E codes per lane, a multiple of four, wave-uniform), read them through buffer descriptors at addresses
// that depend only on the table, and meet the compacted x pairs in v_dot2_f32_bf16: level 1 through the table of
// dequantised pairs (two 3-bit codes -> one LDS read), levels 2 and 3 by arithmetic, each weight rounded to bf16 as
// the reference's decoder does (ixrun/triton_kernels.py:168-177).  The array of each level is padded with zeros up
// to 64 * E slots, so codes read past a level's end meet a zero.
//
// No LDS-DMA and no hand-counted waits here: the kernel is bound by instruction issue (about 520 vector instructions
// per 2048 weights), five waves per SIMD cover the load latency.  A wave sums whole rows when rows spread evenly over
// the launch; otherwise partial sums of the spans of a row are combined through the workspace in span order (or
// added to y32 with atomics).
#include "ixh_dense_tiles.h"
#include "ixh_fast358.h"

namespace ixh {

typedef uint32_t d_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t d_u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t d_u32x3 __attribute__((ext_vector_type(3)));
typedef uint16_t dn_u16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 d_bf16x2 __attribute__((ext_vector_type(2)));
typedef float d_f32x2 __attribute__((ext_vector_type(2)));

constexpr int kDnWaves = 4;                  // waves per workgroup
constexpr uint32_t kDnSpan = 2048;           // elements per span: four table units of one row
constexpr uint32_t kDnSlots = kDnSpan + 3 * 256;  // compacted x slots per wave: three arrays, each padded to 64 * E
static_assert(kDnSlots * 2 >= 64 * 80 && (kDnSlots * 2) % 16 == 0, "the decode kernel re-uses a wave's slots as 64 rows of 80 bytes");
constexpr uint32_t kDnLutBytes = 64 * 32 * 4;     // pair table: 64 code pairs x 32 lane copies

enum : int { kDnDirect = 0, kDnAtomic = 1, kDnWorkspace = 2 };

// sum over the wave, valid in lane 63 (DPP: shifts inside the 16-lane rows, then the two row broadcasts)
#define IXH_DN_DPP_ADD(v, ctrl, row_mask, bound) \
    v += __uint_as_float((uint32_t)__builtin_amdgcn_update_dpp(0, (int)__float_as_uint(v), ctrl, row_mask, 0xf, bound))
__device__ __forceinline__ float dn_wave_sum(float v) {
    IXH_DN_DPP_ADD(v, 0x111, 0xf, true);
    IXH_DN_DPP_ADD(v, 0x112, 0xf, true);
    IXH_DN_DPP_ADD(v, 0x114, 0xf, true);
    IXH_DN_DPP_ADD(v, 0x118, 0xf, true);
    IXH_DN_DPP_ADD(v, 0x142, 0xa, false);
    IXH_DN_DPP_ADD(v, 0x143, 0xc, false);
    return v;
}
#undef IXH_DN_DPP_ADD

__device__ __forceinline__ uint32_t dn_pack(float lo, float hi) {
    const d_f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, d_bf16x2));
}

__device__ __forceinline__ float dn_dot2(uint32_t w, uint32_t x, float acc) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(d_bf16x2, w), __builtin_bit_cast(d_bf16x2, x), acc, false);
}

__global__ void __launch_bounds__(kWave *kDnWaves)
k_gemv358_dense(Dev P, const int32_t *__restrict__ prefix, uint32_t n_chunks, uint32_t spans_per_row, uint32_t n_spans,
                const uint16_t *__restrict__ x, uint16_t *__restrict__ y,
                float *__restrict__ y32, float *__restrict__ ws, int out_mode, bool by_rows) {
    __shared__ __attribute__((aligned(16))) uint32_t lut[kDnLutBytes / 4];
    __shared__ __attribute__((aligned(16))) uint16_t xc_all[kDnWaves][kDnSlots];
    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const float scale = bf16_bits_to_f32(*P.scale);
    const float m15 = -15.0f * scale, m127 = -127.0f * scale;  // exact: 7 + 8 significant bits at most

    // pair table: entry (c0 | c1 << 3) = the two dequantised level-1 weights, one copy per bank
    for (uint32_t e = tid; e < 64 * 32; e += kWave * kDnWaves) {
        const uint32_t idx = e >> 5;
        lut[e] = dn_pack(dequant((int)(idx & 7u) - 3, scale), dequant((int)(idx >> 3) - 3, scale));
    }
    __syncthreads();

    uint16_t *const xc = xc_all[wave];
    const uint32_t lut_lane = (lane & 31u) << 2;
    const uint32_t entries = P.out_f * n_chunks + 1;
    const uint32_t *__restrict__ b1 = P.bm[0];
    const __amdgpu_buffer_rsrc_t l1_rsrc =
        __builtin_amdgcn_make_buffer_rsrc((void *)P.st[0], 0, (int)(P.st_words[0] * 4u), 0x00020000);
    const __amdgpu_buffer_rsrc_t l2_rsrc =
        __builtin_amdgcn_make_buffer_rsrc((void *)P.st[1], 0, (int)(P.st_words[1] * 4u), 0x00020000);
    // whole dwords of the byte stream (device allocations are 256-byte granular, the last dword is there to read)
    const __amdgpu_buffer_rsrc_t l3_rsrc =
        __builtin_amdgcn_make_buffer_rsrc((void *)P.last, 0, (int)((P.last_bytes + 3u) & ~3u), 0x00020000);
    const __amdgpu_buffer_rsrc_t b2_rsrc =
        __builtin_amdgcn_make_buffer_rsrc((void *)P.bm[1], 0, (int)(P.bm_words[1] * 4u), 0x00020000);

    // Work is dealt to the waves of the launch in turn; the launch is resident as a whole, so every wave gets the
    // same number of items (give or take one).  An item is a whole row (its spans are summed in the wave and the
    // result leaves as it is) or, when rows would not spread evenly, one span (partial sums meet in the workspace).
    const uint32_t n_waves = gridDim.x * kDnWaves;
    const uint32_t n_items = by_rows ? P.out_f : n_spans;
    for (uint32_t item = blockIdx.x * kDnWaves + wave; item < n_items; item += n_waves) {
      const uint32_t row = by_rows ? item : item / spans_per_row;
      const uint32_t k_first = by_rows ? 0u : item - row * spans_per_row;
      const uint32_t k_end = by_rows ? spans_per_row : k_first + 1u;
      float row_total = 0.0f;  // meaningful in lane 63
      for (uint32_t k = k_first; k < k_end; ++k) {
        // The waves that share a SIMD take turns at the issue priority, one span each: all of them start their rows
        // together, and this keeps them from meeting at the same phase (scatter, dense passes) span after span.
        {
            const uint32_t turn = (wave + k) % 3u;  // s_setprio takes an immediate
            if (turn == 0) __builtin_amdgcn_s_setprio(0);
            else if (turn == 1) __builtin_amdgcn_s_setprio(1);
            else __builtin_amdgcn_s_setprio(2);
        }
        const uint32_t c0 = 4 * k, nb = min(4u, n_chunks - c0);
        const uint32_t u0 = row * n_chunks + c0;
        const uint32_t n_el = nb * kFastChunk, p0 = u0 * kFastChunk;
        const uint32_t q1a = (uint32_t)prefix[u0], q1b = (uint32_t)prefix[u0 + nb];
        const uint32_t q2a = (uint32_t)prefix[entries + u0], q2b = (uint32_t)prefix[entries + u0 + nb];
        const uint32_t n1 = q1b - q1a, n2 = q2b - q2a, n3 = n_el - n1 - n2;
        // codes per lane in the dense passes (a multiple of four: the passes run in groups of two pairs), and the
        // padded sizes of the compacted arrays
        const uint32_t e1 = 4 * ((n1 + 255) / 256), e2 = 4 * ((n2 + 255) / 256), e3 = 4 * ((n3 + 255) / 256);
        const uint32_t base2 = 64 * e1, base3 = base2 + 64 * e2;

        // ---- loads whose addresses follow from the table alone ----
        const bool valid = 32 * lane < n_el;
        const uint32_t w1 = valid ? b1[(p0 >> 5) + lane] : 0u;
        uint32_t xr[16];
        if (valid) {
            const uint4 *xp = reinterpret_cast<const uint4 *>(x + c0 * kFastChunk + 32 * lane);
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const uint4 v = xp[t];
                xr[4 * t] = v.x; xr[4 * t + 1] = v.y; xr[4 * t + 2] = v.z; xr[4 * t + 3] = v.w;
            }
        } else {
#pragma unroll
            for (int t = 0; t < 16; ++t) xr[t] = 0u;
        }
        // The code streams, read through buffer descriptors: a dword past a stream's end reads as zero, so no lane
        // needs a bounds test; lanes whose share lies past the level's last code read codes of the next span, which
        // then meet the zero pads of the compacted arrays.
        // level-1 codes of this lane: e1 of them from code q1a + lane * e1 on (96 bits at most)
        uint32_t c1w[3];
        {
            const uint64_t bit = (uint64_t)(q1a + lane * e1) * 3u;
            const uint32_t wi = (uint32_t)(bit >> 5), sh = (uint32_t)bit & 31u;
            const d_u32x4 d = __builtin_amdgcn_raw_buffer_load_b128(l1_rsrc, (int)(wi * 4u), 0, 0);
            c1w[0] = __builtin_amdgcn_alignbit(d[1], d[0], sh);
            c1w[1] = __builtin_amdgcn_alignbit(d[2], d[1], sh);
            c1w[2] = __builtin_amdgcn_alignbit(d[3], d[2], sh);
        }
        // level-2 codes: e2 of them from code q2a + lane * e2 on (160 bits at most)
        uint32_t c2w[5];
        {
            const uint64_t bit = (uint64_t)(q2a + lane * e2) * 5u;
            const uint32_t wi = (uint32_t)(bit >> 5), sh = (uint32_t)bit & 31u;
            const d_u32x4 da = __builtin_amdgcn_raw_buffer_load_b128(l2_rsrc, (int)(wi * 4u), 0, 0);
            const d_u32x2 db = __builtin_amdgcn_raw_buffer_load_b64(l2_rsrc, (int)(wi * 4u + 16u), 0, 0);
            const uint32_t d[6] = {da[0], da[1], da[2], da[3], db[0], db[1]};
#pragma unroll
            for (int j = 0; j < 5; ++j) c2w[j] = __builtin_amdgcn_alignbit(d[j + 1], d[j], sh);
        }
        // level-3 bytes: e3 of them from byte (p0 - q1a - q2a) + lane * e3 on (32 bytes at most), read as dwords
        uint32_t c3w[8];
        {
            const uint32_t at = (p0 - q1a - q2a) + lane * e3;
            const uint32_t wi = at >> 2, sh = (at & 3u) * 8u;
            const d_u32x4 da = __builtin_amdgcn_raw_buffer_load_b128(l3_rsrc, (int)(wi * 4u), 0, 0);
            const d_u32x4 db = __builtin_amdgcn_raw_buffer_load_b128(l3_rsrc, (int)(wi * 4u + 16u), 0, 0);
            const uint32_t dc = __builtin_amdgcn_raw_buffer_load_b32(l3_rsrc, (int)(wi * 4u + 32u), 0, 0);
            const uint32_t d[9] = {da[0], da[1], da[2], da[3], db[0], db[1], db[2], db[3], dc};
#pragma unroll
            for (int j = 0; j < 8; ++j) c3w[j] = __builtin_amdgcn_alignbit(d[j + 1], d[j], sh);
        }

        // ---- clear the compacted arrays (the pads must read as zero) ----
        for (uint32_t j = lane; j < kDnSlots / 8; j += kWave) reinterpret_cast<d_u32x4 *>(xc)[j] = d_u32x4{0, 0, 0, 0};

        // ---- ranks: first slot of this lane in each array ----
        const uint32_t cnt1 = (uint32_t)__popc(w1);
        const uint32_t alive = valid ? 32u - cnt1 : 0u;
        const uint32_t packed = wave_scan_inclusive(cnt1 | (alive << 16));
        const uint32_t first1 = (packed & 0xffffu) - cnt1;          // level-1 elements in the lanes below
        const uint32_t first_a = (packed >> 16) - alive;            // elements above level 1 in the lanes below
        uint32_t bits2;  // bit j: the lane's j-th element above level 1 is level 2
        {
            const uint32_t g = (p0 - q1a) + first_a;
            const d_u32x2 w = __builtin_amdgcn_raw_buffer_load_b64(b2_rsrc, (int)((g >> 5) * 4u), 0, 0);
            // alive = 0 shifts the mask out entirely (a 64-bit shift: 32 is a legal count)
            bits2 = __builtin_amdgcn_alignbit(w[1], w[0], g & 31u) & (uint32_t)(0xFFFFFFFFull >> (32u - alive));
        }
        const uint32_t cnt2 = (uint32_t)__popc(bits2);
        const uint32_t first2 = wave_scan_inclusive(cnt2) - cnt2;
        const uint32_t first3 = first_a - first2;

        // ---- scatter the lane's 32 activations to their levels' arrays ----
        // Two elements per step, t and t + 16, with their counters in the two halves of one register (packed
        // 16-bit arithmetic): each half holds "LDS byte address / 2" of the next slot of its level, which fits
        // 16 bits.  The second half starts where the first one will end: behind the level counts of the lane's
        // first 16 elements.  in1 / in2 / in3 are 0 or 1 per half; the slot is picked by multiply-add.
        {
            const uint32_t xc_half = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint16_t *)xc >> 1;
            const uint32_t low1 = (uint32_t)__popc(w1 & 0xffffu);               // level-1 elements among the first 16
            const uint32_t low_a = valid ? 16u - low1 : 0u;                       // elements above level 1 among them
            const uint32_t low2 = (uint32_t)__popc(bits2 & ((1u << low_a) - 1u));  // of which level 2
            const uint32_t a1 = xc_half + first1, a2 = xc_half + base2 + first2, a3 = xc_half + base3 + first3;
            dn_u16x2 s1 = __builtin_bit_cast(dn_u16x2, a1 | ((a1 + low1) << 16));
            dn_u16x2 s2 = __builtin_bit_cast(dn_u16x2, a2 | ((a2 + low2) << 16));
            dn_u16x2 s3 = __builtin_bit_cast(dn_u16x2, a3 | ((a3 + low_a - low2) << 16));
            // the level-2 flags each half walks through: bits2 from bit 0, and from bit low_a
            const dn_u16x2 flags = __builtin_bit_cast(dn_u16x2, (bits2 & 0xffffu) | ((bits2 >> low_a) << 16));
            dn_u16x2 ja = {0, 0};
            const dn_u16x2 one = {1, 1};
#pragma unroll
            for (int t = 0; t < 16; ++t) {
                const dn_u16x2 in1 = __builtin_bit_cast(dn_u16x2, (w1 >> t) & 0x00010001u);
                const dn_u16x2 out1 = in1 ^ one;
                const dn_u16x2 in2 = (flags >> ja) & out1;
                const dn_u16x2 in3 = out1 ^ in2;
                const dn_u16x2 at = in1 * (s1 - s3) + (in2 * (s2 - s3) + s3);
                const uint32_t at32 = __builtin_bit_cast(uint32_t, at);
                const uint32_t x_lo = xr[t >> 1], x_hi = xr[8 + (t >> 1)];
                // lanes past the span scatter zeros behind the last array's entries
                *reinterpret_cast<__attribute__((address_space(3))) uint16_t *>((uintptr_t)((at32 & 0xffffu) << 1)) =
                    (uint16_t)((t & 1) ? x_lo >> 16 : x_lo);
                *reinterpret_cast<__attribute__((address_space(3))) uint16_t *>((uintptr_t)((at32 >> 16) << 1)) =
                    (uint16_t)((t & 1) ? x_hi >> 16 : x_hi);
                s1 += in1; s2 += in2; s3 += in3; ja += out1;
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();

        // ---- dense passes ----
        float acc = 0.0f;
        // Each pass runs in groups of two pairs; a group is entered only if the level has codes for it.  (The empty
        // asm statements keep the group tests branches: as selects, all 24 groups would run for every span.)
        {   // level 1: pairs of 3-bit codes through the pair table
            const uint32_t *xp = reinterpret_cast<const uint32_t *>(xc) + (lane * e1) / 2;
#pragma unroll
            for (int g = 0; g < 8; ++g) {
                if (e1 > 4u * g) {
                    asm volatile("");
#pragma unroll
                    for (int t = 2 * g; t < 2 * g + 2; ++t) {
                        const int bit = 6 * t, ob = bit & 31, d = bit >> 5;
                        const uint32_t lo = c1w[d];
                        const uint32_t hi = d < 2 ? c1w[d + 1] : 0u;
                        uint32_t a;  // pair index at bits 12..7
                        if (ob > 26) a = __builtin_amdgcn_alignbit(hi, lo, ob - 7);
                        else if (ob >= 7) a = lo >> (ob - 7);
                        else a = lo << (7 - ob);
                        const uint32_t wp = lut[((a & 0x1F80u) | lut_lane) >> 2];
                        acc = dn_dot2(wp, xp[t], acc);
                    }
                }
            }
        }
        {   // level 2: pairs of 5-bit codes, dequantised by arithmetic
            const uint32_t *xp = reinterpret_cast<const uint32_t *>(xc) + (base2 + lane * e2) / 2;
#pragma unroll
            for (int g = 0; g < 8; ++g) {
                if (e2 > 4u * g) {
                    asm volatile("");
#pragma unroll
                    for (int t = 2 * g; t < 2 * g + 2; ++t) {
                        uint32_t c[2];
#pragma unroll
                        for (int h = 0; h < 2; ++h) {
                            const int bit = 10 * t + 5 * h, ob = bit & 31, d = bit >> 5;
                            c[h] = ob <= 27 ? (c2w[d] >> ob) & 31u
                                            : __builtin_amdgcn_alignbit(d < 4 ? c2w[d + 1] : 0u, c2w[d], ob) & 31u;
                        }
                        // (c - 15) * scale as c * scale - 15 * scale: both products and their difference are exact in
                        // fp32 (codes and 15 have at most 5 significant bits, the bf16 scale 8): nothing is rounded twice
                        const uint32_t wp = dn_pack(__fmaf_rn((float)c[0], scale, m15), __fmaf_rn((float)c[1], scale, m15));
                        acc = dn_dot2(wp, xp[t], acc);
                    }
                }
            }
        }
        {   // level 3: pairs of bytes
            const uint32_t *xp = reinterpret_cast<const uint32_t *>(xc) + (base3 + lane * e3) / 2;
#pragma unroll
            for (int g = 0; g < 8; ++g) {
                if (e3 > 4u * g) {
                    asm volatile("");
#pragma unroll
                    for (int t = 2 * g; t < 2 * g + 2; ++t) {
                        const uint32_t word = c3w[t >> 1];
                        const uint32_t ca = (word >> (16 * (t & 1))) & 255u, cb = (word >> (16 * (t & 1) + 8)) & 255u;
                        const uint32_t wp = dn_pack(__fmaf_rn((float)ca, scale, m127), __fmaf_rn((float)cb, scale, m127));
                        acc = dn_dot2(wp, xp[t], acc);
                    }
                }
            }
        }
        row_total += dn_wave_sum(acc);
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
      }
      if (lane == 63) {
          if (out_mode == kDnDirect) y[row] = (uint16_t)f32_to_bf16_bits(row_total);
          else if (out_mode == kDnAtomic) atomicAdd(y32 + row, row_total);
          else ws[(size_t)k_first * P.out_f + row] = row_total;
      }
    }
}

// ---------------------------------------------------------------------------------------------------------------
// The weights of a span in position order, by the same route turned round (for dense mixes): the codes of each level
// are dequantised where they lie (dense, fixed positions) into three LDS arrays of weights, and every lane then
// gathers the weights of its 32 positions from the slots that the scatter above would have written to.
// dn_walk_spans does this for every span that `spans` deals to the wave and hands the lane's 16 packed pairs to
// `sink` (the full decode stores them, the several-row product multiplies them with its activations).
// A lane's rows of the three arrays hold a number of codes that is twice an odd number, and the passes work in groups
// of two pairs, so a lane's last group decodes one pair that is the next lane's first: both write the same value.
// With group scales (GS: one fp16 scale per 2^group_shift >= 32 consecutive elements, so one per lane) the arrays
// hold the integer values as bf16, exact, and the lane multiplies what it gathered by its scale.
// ---------------------------------------------------------------------------------------------------------------
struct DnSpan {
    uint32_t p0, n_el;   // first flat element, elements (a multiple of 32 except at the tensor's end)
    uint32_t u0, u1;     // rank-table entries at its start and end
    uint32_t a, b, c;    // the enumerator's own: span index, or row / span of the row / item
};

// flat spans of 2048 elements, dealt to the waves of the launch in turn
struct DnFlatSpans {
    uint32_t n_units, n_spans, n, first, stride;
    __device__ __forceinline__ DnSpan at(uint32_t s) const {
        DnSpan sp;
        sp.u0 = 4 * s;
        sp.u1 = min(sp.u0 + 4, n_units);
        sp.p0 = sp.u0 * kFastChunk;
        sp.n_el = min(kDnSpan, n - sp.p0);
        sp.a = s; sp.b = 0; sp.c = 0;
        return sp;
    }
    __device__ __forceinline__ bool first_span(DnSpan &sp) const {
        if (first >= n_spans) return false;
        sp = at(first);
        return true;
    }
    __device__ __forceinline__ bool next(const DnSpan &cur, DnSpan &nx) const {
        if (cur.a + stride >= n_spans) return false;
        nx = at(cur.a + stride);
        return true;
    }
};

template <bool GS, class Spans, class Sink, bool TAKE_TURNS = true>
__device__ __forceinline__ void dn_walk_spans(const Dev &P, const int32_t *__restrict__ prefix, uint32_t entries,
                                              const uint16_t *__restrict__ group_scales, uint32_t group_shift,
                                              const uint32_t *lut, uint16_t *wc, float scale, uint32_t lane,
                                              const Spans &spans, Sink &sink, uint32_t wave_turn) {
    const float m15 = -15.0f * scale, m127 = -127.0f * scale;
    uint32_t *const wc32 = reinterpret_cast<uint32_t *>(wc);
    const uint32_t lut_lane = (lane & 31u) << 2;
    const uint32_t *__restrict__ b1 = P.bm[0];
    const __amdgpu_buffer_rsrc_t l1_rsrc =
        __builtin_amdgcn_make_buffer_rsrc((void *)P.st[0], 0, (int)(P.st_words[0] * 4u), 0x00020000);
    const __amdgpu_buffer_rsrc_t l2_rsrc =
        __builtin_amdgcn_make_buffer_rsrc((void *)P.st[1], 0, (int)(P.st_words[1] * 4u), 0x00020000);
    const __amdgpu_buffer_rsrc_t l3_rsrc =
        __builtin_amdgcn_make_buffer_rsrc((void *)P.last, 0, (int)((P.last_bytes + 3u) & ~3u), 0x00020000);
    const __amdgpu_buffer_rsrc_t b2_rsrc =
        __builtin_amdgcn_make_buffer_rsrc((void *)P.bm[1], 0, (int)(P.bm_words[1] * 4u), 0x00020000);

    // What a span needs from memory before any arithmetic: four table entries (scalars), the lane's bitmap word and
    // its window of each code stream.  They are fetched one span ahead (the table entries two), so that a wave's
    // chain table -> windows -> arithmetic does not wait on memory twice per span.
    struct Ranks { uint32_t q1a, q1b, q2a, q2b; };
    struct Loads { uint32_t w1; d_u32x4 l1a; uint32_t l1b; d_u32x4 l2a; d_u32x3 l2b; d_u32x4 l3a, l3b; d_u32x2 l3c; uint32_t group_scale; };
    struct Shape { uint32_t p0, n_el, e1, e2, e3; };
    // Codes of a level per lane: enough for all of them, and twice an odd number, so that the lanes' rows of the LDS
    // array start an odd number of dwords apart (no two of 32 neighbouring lanes on one bank).  2, 6, ... 34.
    auto codes_per_lane = [](uint32_t n) { return (((n + 63) / 64 + 1) & ~3u) + 2; };
    auto table_of = [&](const DnSpan &sp) {
        return Ranks{(uint32_t)prefix[sp.u0], (uint32_t)prefix[sp.u1], (uint32_t)prefix[entries + sp.u0],
                     (uint32_t)prefix[entries + sp.u1]};
    };
    auto shape_of = [&](const DnSpan &sp, const Ranks &q) {
        const uint32_t p0 = sp.p0, n_el = sp.n_el;
        const uint32_t n1 = q.q1b - q.q1a, n2 = q.q2b - q.q2a, n3 = n_el - n1 - n2;
        return Shape{p0, n_el, codes_per_lane(n1), codes_per_lane(n2), codes_per_lane(n3)};
    };
    auto fetch = [&](const DnSpan &sp, const Ranks &q) {
        const Shape g = shape_of(sp, q);
        Loads r;
        r.w1 = 32 * lane < g.n_el ? b1[(g.p0 >> 5) + lane] : 0u;
        r.group_scale = GS && 32 * lane < g.n_el ? group_scales[(g.p0 + 32 * lane) >> group_shift] : 0u;
        {
            const uint64_t bit = (uint64_t)(q.q1a + lane * g.e1) * 3u;
            const uint32_t at = (uint32_t)(bit >> 5) * 4u;
            r.l1a = __builtin_amdgcn_raw_buffer_load_b128(l1_rsrc, (int)at, 0, 0);
            r.l1b = __builtin_amdgcn_raw_buffer_load_b32(l1_rsrc, (int)(at + 16u), 0, 0);
        }
        {
            const uint64_t bit = (uint64_t)(q.q2a + lane * g.e2) * 5u;
            const uint32_t at = (uint32_t)(bit >> 5) * 4u;
            r.l2a = __builtin_amdgcn_raw_buffer_load_b128(l2_rsrc, (int)at, 0, 0);
            r.l2b = __builtin_amdgcn_raw_buffer_load_b96(l2_rsrc, (int)(at + 16u), 0, 0);
        }
        {
            const uint32_t at = (((g.p0 - q.q1a - q.q2a) + lane * g.e3) >> 2) * 4u;
            r.l3a = __builtin_amdgcn_raw_buffer_load_b128(l3_rsrc, (int)at, 0, 0);
            r.l3b = __builtin_amdgcn_raw_buffer_load_b128(l3_rsrc, (int)(at + 16u), 0, 0);
            r.l3c = __builtin_amdgcn_raw_buffer_load_b64(l3_rsrc, (int)(at + 32u), 0, 0);
        }
        return r;
    };


    DnSpan sp_now, sp_next, sp_after;
    if (!spans.first_span(sp_now)) return;
    bool has_next = spans.next(sp_now, sp_next);
    if (!has_next) sp_next = sp_now;  // at the end the last span is fetched once more: loads that nobody uses
    bool has_after = has_next && spans.next(sp_next, sp_after);
    if (!has_after) sp_after = sp_next;
    Ranks q_now = table_of(sp_now);
    Loads in_now = fetch(sp_now, q_now);
    Ranks q_next = table_of(sp_next);
    for (uint32_t turn = wave_turn;; ++turn) {
        // the waves that share a SIMD take turns at the issue priority, one span each, so that they do not meet at the
        // same phase (dequantise, gather, store or multiply) span after span
        if (TAKE_TURNS) {  // (not where the waves meet at a barrier every span: there they should keep pace)
            const uint32_t pr = turn % 3u;  // s_setprio takes an immediate
            if (pr == 0) __builtin_amdgcn_s_setprio(0);
            else if (pr == 1) __builtin_amdgcn_s_setprio(1);
            else __builtin_amdgcn_s_setprio(2);
        }
        const Loads in_next = fetch(sp_next, q_next);
        const Ranks q_after = table_of(sp_after);
        sink.begin(sp_now);
        const Shape g = shape_of(sp_now, q_now);
        const uint32_t p0 = g.p0, n_el = g.n_el, e1 = g.e1, e2 = g.e2, e3 = g.e3;
        const uint32_t q1a = q_now.q1a, q2a = q_now.q2a;
        const uint32_t base2 = 64 * e1, base3 = base2 + 64 * e2;

        // positions of this lane inside the span, and its bitmap word
        const uint32_t n_here = 32 * lane < n_el ? min(32u, n_el - 32 * lane) : 0u;
        const uint32_t here = (uint32_t)(0xFFFFFFFFull >> (32u - n_here));  // n_here = 0 gives an empty mask
        const uint32_t w1 = in_now.w1 & here;

        // ---- dequantise every level where its codes lie ----
        {
            const uint32_t sh = (uint32_t)((uint64_t)(q1a + lane * e1) * 3u) & 31u;
            const d_u32x4 d = in_now.l1a;
            const uint32_t c1w[4] = {__builtin_amdgcn_alignbit(d[1], d[0], sh), __builtin_amdgcn_alignbit(d[2], d[1], sh),
                                     __builtin_amdgcn_alignbit(d[3], d[2], sh), __builtin_amdgcn_alignbit(in_now.l1b, d[3], sh)};
            uint32_t *dst = wc32 + (lane * e1) / 2;
#pragma unroll
            for (int g = 0; g < 9; ++g) {
                if (e1 > 4u * g) {
                    asm volatile("");
#pragma unroll
                    for (int t = 2 * g; t < 2 * g + 2; ++t) {
                        const int bt = 6 * t, ob = bt & 31, dd = bt >> 5;
                        const uint32_t lo = c1w[dd];
                        const uint32_t hi = dd < 3 ? c1w[dd + 1] : 0u;
                        uint32_t a;
                        if (ob > 26) a = __builtin_amdgcn_alignbit(hi, lo, ob - 7);
                        else if (ob >= 7) a = lo >> (ob - 7);
                        else a = lo << (7 - ob);
                        dst[t] = lut[((a & 0x1F80u) | lut_lane) >> 2];
                    }
                }
            }
        }
        {
            const uint32_t sh = (uint32_t)((uint64_t)(q2a + lane * e2) * 5u) & 31u;
            const uint32_t d[7] = {in_now.l2a[0], in_now.l2a[1], in_now.l2a[2], in_now.l2a[3],
                                   in_now.l2b[0], in_now.l2b[1], in_now.l2b[2]};
            uint32_t c2w[6];
#pragma unroll
            for (int j = 0; j < 6; ++j) c2w[j] = __builtin_amdgcn_alignbit(d[j + 1], d[j], sh);
            uint32_t *dst = wc32 + (base2 + lane * e2) / 2;
#pragma unroll
            for (int g = 0; g < 9; ++g) {
                if (e2 > 4u * g) {
                    asm volatile("");
#pragma unroll
                    for (int t = 2 * g; t < 2 * g + 2; ++t) {
                        uint32_t c[2];
#pragma unroll
                        for (int h = 0; h < 2; ++h) {
                            const int bt = 10 * t + 5 * h, ob = bt & 31, dd = bt >> 5;
                            c[h] = ob <= 27 ? (c2w[dd] >> ob) & 31u
                                            : __builtin_amdgcn_alignbit(dd < 5 ? c2w[dd + 1] : 0u, c2w[dd], ob) & 31u;
                        }
                        dst[t] = dn_pack(__fmaf_rn((float)c[0], scale, m15), __fmaf_rn((float)c[1], scale, m15));
                    }
                }
            }
        }
        {
            const uint32_t sh = (((p0 - q1a - q2a) + lane * e3) & 3u) * 8u;
            const uint32_t d[10] = {in_now.l3a[0], in_now.l3a[1], in_now.l3a[2], in_now.l3a[3], in_now.l3b[0],
                                    in_now.l3b[1], in_now.l3b[2], in_now.l3b[3], in_now.l3c[0], in_now.l3c[1]};
            uint32_t c3w[9];
#pragma unroll
            for (int j = 0; j < 9; ++j) c3w[j] = __builtin_amdgcn_alignbit(d[j + 1], d[j], sh);
            uint32_t *dst = wc32 + (base3 + lane * e3) / 2;
#pragma unroll
            for (int g = 0; g < 9; ++g) {
                if (e3 > 4u * g) {
                    asm volatile("");
#pragma unroll
                    for (int t = 2 * g; t < 2 * g + 2; ++t) {
                        const uint32_t word = c3w[t >> 1];
                        const uint32_t ca = (word >> (16 * (t & 1))) & 255u, cb = (word >> (16 * (t & 1) + 8)) & 255u;
                        dst[t] = dn_pack(__fmaf_rn((float)ca, scale, m127), __fmaf_rn((float)cb, scale, m127));
                    }
                }
            }
        }

        // ---- ranks: first slot of this lane in each array ----
        const uint32_t cnt1 = (uint32_t)__popc(w1);
        const uint32_t alive = n_here - cnt1;
        const uint32_t packed = wave_scan_inclusive(cnt1 | (alive << 16));
        const uint32_t first1 = (packed & 0xffffu) - cnt1;
        const uint32_t first_a = (packed >> 16) - alive;
        uint32_t bits2;
        {
            const uint32_t g = (p0 - q1a) + first_a;
            const d_u32x2 w = __builtin_amdgcn_raw_buffer_load_b64(b2_rsrc, (int)((g >> 5) * 4u), 0, 0);
            bits2 = __builtin_amdgcn_alignbit(w[1], w[0], g & 31u) & (uint32_t)(0xFFFFFFFFull >> (32u - alive));
        }
        const uint32_t cnt2 = (uint32_t)__popc(bits2);
        const uint32_t first2 = wave_scan_inclusive(cnt2) - cnt2;
        const uint32_t first3 = first_a - first2;
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();

        // ---- gather: the same walk as the scatter of the product kernel, reading instead of writing ----
        uint32_t o[16];  // the lane's 32 weights, in position order
        {
            const uint32_t wc_half = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint16_t *)wc >> 1;
            const uint32_t low1 = (uint32_t)__popc(w1 & 0xffffu);
            const uint32_t low_a = min(n_here, 16u) - low1;
            const uint32_t low2 = (uint32_t)__popc(bits2 & ((1u << low_a) - 1u));
            const uint32_t a1 = wc_half + first1, a2 = wc_half + base2 + first2, a3 = wc_half + base3 + first3;
            dn_u16x2 s1 = __builtin_bit_cast(dn_u16x2, a1 | ((a1 + low1) << 16));
            dn_u16x2 s2 = __builtin_bit_cast(dn_u16x2, a2 | ((a2 + low2) << 16));
            dn_u16x2 s3 = __builtin_bit_cast(dn_u16x2, a3 | ((a3 + low_a - low2) << 16));
            const dn_u16x2 flags = __builtin_bit_cast(dn_u16x2, (bits2 & 0xffffu) | ((bits2 >> low_a) << 16));
            dn_u16x2 ja = {0, 0};
            const dn_u16x2 one = {1, 1};
#pragma unroll
            for (int t = 0; t < 16; ++t) {
                const dn_u16x2 in1 = __builtin_bit_cast(dn_u16x2, (w1 >> t) & 0x00010001u);
                const dn_u16x2 out1 = in1 ^ one;
                const dn_u16x2 in2 = (flags >> ja) & out1;
                const dn_u16x2 in3 = out1 ^ in2;
                const dn_u16x2 at = in1 * (s1 - s3) + (in2 * (s2 - s3) + s3);
                const uint32_t at32 = __builtin_bit_cast(uint32_t, at);
                // positions past the end of the tensor walk on through the last array; what they read is not stored
                const uint32_t va = *reinterpret_cast<const __attribute__((address_space(3))) uint16_t *>((uintptr_t)((at32 & 0xffffu) << 1));
                const uint32_t vb = *reinterpret_cast<const __attribute__((address_space(3))) uint16_t *>((uintptr_t)((at32 >> 16) << 1));
                if (t & 1) {
                    o[t >> 1] |= va << 16;
                    o[8 + (t >> 1)] |= vb << 16;
                } else {
                    o[t >> 1] = va;
                    o[8 + (t >> 1)] = vb;
                }
                s1 += in1; s2 += in2; s3 += in3; ja += out1;
            }
        }
        if (GS) {
            const float sc = fp16_bits_to_f32((uint16_t)in_now.group_scale);
#pragma unroll
            for (int j = 0; j < 16; ++j)
                o[j] = dn_pack(__uint_as_float(o[j] << 16) * sc, __uint_as_float(o[j] & 0xffff0000u) * sc);
        }
        sink.end(sp_now, o, n_here);
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
        if (!has_next) break;
        sp_now = sp_next;
        in_now = in_next;
        q_now = q_next;
        q_next = q_after;
        sp_next = sp_after;
        has_next = has_after;
        has_after = has_next && spans.next(sp_next, sp_after);
        if (!has_after) sp_after = sp_next;
    }
}

// the full decode's end of a span: the lane's 64 bytes to their place in the output
struct DnStoreSink {
    uint16_t *__restrict__ out;
    uint16_t *wc;
    uint32_t lane;
    __device__ __forceinline__ void begin(const DnSpan &) {}
    __device__ __forceinline__ void end(const DnSpan &sp, const uint32_t (&o)[16], uint32_t n_here) {
        const uint32_t p0 = sp.p0, n_el = sp.n_el;
        uint16_t *dst = out + (size_t)p0 + 32 * lane;
        if (n_el == kDnSpan) {
            // Whole span: through LDS once more, so that a store instruction writes 1 KB of consecutive bytes
            // (lane rows 80 bytes apart keep the 16-byte accesses of eight neighbouring lanes on distinct banks).
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
            __builtin_amdgcn_wave_barrier();
            d_u32x4 *const rows = reinterpret_cast<d_u32x4 *>(wc);
#pragma unroll
            for (int j = 0; j < 4; ++j) rows[lane * 5 + j] = d_u32x4{o[4 * j], o[4 * j + 1], o[4 * j + 2], o[4 * j + 3]};
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
            __builtin_amdgcn_wave_barrier();
            d_u32x4 *const line = reinterpret_cast<d_u32x4 *>(out + (size_t)p0);
#pragma unroll
            for (int j = 0; j < 4; ++j) line[64 * j + lane] = rows[(16 * j + (lane >> 2)) * 5 + (lane & 3u)];
        } else if (n_here == 32) {
#pragma unroll
            for (int j = 0; j < 4; ++j)
                reinterpret_cast<d_u32x4 *>(dst)[j] = d_u32x4{o[4 * j], o[4 * j + 1], o[4 * j + 2], o[4 * j + 3]};
        } else {
            for (uint32_t t = 0; t < n_here; ++t) {
                uint32_t v = 0;
#pragma unroll
                for (int j = 0; j < 16; ++j) v = (t >> 1) == (uint32_t)j ? o[j] : v;
                dst[t] = (uint16_t)((t & 1u) ? v >> 16 : v);
            }
        }
    }
};

template <bool GS>
__global__ void __launch_bounds__(kWave *kDnWaves, 5)  // five waves per SIMD: what the LDS allows
k_decode358_dense(Dev P, const int32_t *__restrict__ prefix, uint32_t n_units, uint32_t n_spans, uint16_t *__restrict__ out,
                  const uint16_t *__restrict__ group_scales, uint32_t group_shift) {
    __shared__ __attribute__((aligned(16))) uint32_t lut[kDnLutBytes / 4];
    __shared__ __attribute__((aligned(16))) uint16_t wc_all[kDnWaves][kDnSlots];
    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const float scale = GS ? 1.0f : bf16_bits_to_f32(*P.scale);
    for (uint32_t e = tid; e < 64 * 32; e += kWave * kDnWaves) {
        const uint32_t idx = e >> 5;
        lut[e] = dn_pack(dequant((int)(idx & 7u) - 3, scale), dequant((int)(idx >> 3) - 3, scale));
    }
    __syncthreads();
    const DnFlatSpans spans{n_units, n_spans, P.n, blockIdx.x * kDnWaves + wave, gridDim.x * kDnWaves};
    DnStoreSink sink{out, wc_all[wave], lane};
    dn_walk_spans<GS>(P, prefix, n_units + 1, group_scales, group_shift, lut, wc_all[wave], scale, lane, spans, sink, wave);
}

// ---------------------------------------------------------------------------------------------------------------
// Product with 2..8 activation rows for dense mixes (more than four: in two passes over the gathered weights): the span walker above with a sink that multiplies.  (With one
// row it is cheaper to move the activations to the codes, k_gemv358_dense; with several rows the weights are
// brought to position order once and meet every row's activations there.)
// ---------------------------------------------------------------------------------------------------------------
// spans of up to four units of one row; an item of the deal is a whole row (by_rows) or one span
struct DnRowSpans {
    uint32_t n_chunks, spans_per_row, n_items, first, stride, stride_rows, stride_spans;  // stride = rows * spans_per_row + spans
    bool by_rows;
    __device__ __forceinline__ DnSpan at(uint32_t row, uint32_t k, uint32_t item) const {
        DnSpan sp;
        const uint32_t nb = min(4u, n_chunks - 4 * k);
        sp.u0 = row * n_chunks + 4 * k;
        sp.u1 = sp.u0 + nb;
        sp.p0 = sp.u0 * kFastChunk;
        sp.n_el = nb * kFastChunk;
        sp.a = row; sp.b = k; sp.c = item;
        return sp;
    }
    __device__ __forceinline__ bool first_span(DnSpan &sp) const {
        if (first >= n_items) return false;
        sp = by_rows ? at(first, 0, first) : at(first / spans_per_row, first % spans_per_row, first);
        return true;
    }
    __device__ __forceinline__ bool next(const DnSpan &cur, DnSpan &nx) const {
        if (by_rows) {
            if (cur.b + 1 < spans_per_row) { nx = at(cur.a, cur.b + 1, cur.c); return true; }
            if (cur.a + stride >= n_items) return false;
            nx = at(cur.a + stride, 0, cur.a + stride);
            return true;
        }
        if (cur.c + stride >= n_items) return false;
        uint32_t row = cur.a + stride_rows, k = cur.b + stride_spans;
        if (k >= spans_per_row) { k -= spans_per_row; ++row; }
        nx = at(row, k, cur.c + stride);
        return true;
    }
};

template <int MT>
struct DnDotSink {
    const uint16_t *__restrict__ x;
    int64_t ldx;
    int m;
    uint16_t *__restrict__ y;
    int64_t ldy;
    float *__restrict__ ws;
    uint32_t out_f, spans_per_row, lane;
    bool by_rows;
    uint32_t xr[MT][16];
    float row_total[2 * MT];  // meaningful in lane 63

    // the lane's activations of rows j0 .. j0 + MT - 1 for this span
    __device__ __forceinline__ void load_x(const DnSpan &sp, int j0) {
        const bool valid = 32 * lane < sp.n_el;
#pragma unroll
        for (int j = 0; j < MT; ++j) {
            if (valid && j0 + j < m) {
                const uint4 *xp =
                    reinterpret_cast<const uint4 *>(x + (int64_t)(j0 + j) * ldx + (size_t)sp.b * kDnSpan + 32 * lane);
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const uint4 v = xp[t];
                    xr[j][4 * t] = v.x; xr[j][4 * t + 1] = v.y; xr[j][4 * t + 2] = v.z; xr[j][4 * t + 3] = v.w;
                }
            } else {
#pragma unroll
                for (int t = 0; t < 16; ++t) xr[j][t] = 0u;  // lanes past the row's end gathered stale weights
            }
        }
    }
    // the first MT rows are requested before the span's arithmetic starts; rows MT .. 2 MT - 1 (if any) take their
    // place after the first rows' products
    __device__ __forceinline__ void begin(const DnSpan &sp) { load_x(sp, 0); }
    __device__ __forceinline__ void end(const DnSpan &sp, const uint32_t (&o)[16], uint32_t) {
        dots(sp, o, 0);
        if (m > MT) {
            load_x(sp, MT);
            dots(sp, o, MT);
        }
    }
    __device__ __forceinline__ void dots(const DnSpan &sp, const uint32_t (&o)[16], int j0) {
#pragma unroll
        for (int j = 0; j < MT; ++j) {
            float a0 = 0.0f, a1 = 0.0f;
#pragma unroll
            for (int t = 0; t < 16; t += 2) {
                a0 = dn_dot2(o[t], xr[j][t], a0);
                a1 = dn_dot2(o[t + 1], xr[j][t + 1], a1);
            }
            const float total = dn_wave_sum(a0 + a1);
            if (by_rows) {
                float &sum = j0 == 0 ? row_total[j] : row_total[MT + j];
                sum = (sp.b == 0 ? 0.0f : sum) + total;
                if (sp.b + 1 == spans_per_row && lane == 63 && j0 + j < m)
                    y[(int64_t)(j0 + j) * ldy + sp.a] = (uint16_t)f32_to_bf16_bits(sum);
            } else if (lane == 63 && j0 + j < m) {
                ws[((size_t)sp.b * m + j0 + j) * out_f + sp.a] = total;
            }
        }
    }
};

template <int MT>
__global__ void __launch_bounds__(kWave *kDnWaves, MT == 4 ? 3 : 4)  // waves per SIMD that the registers should allow
k_gemv358_dense_rows(Dev P, const int32_t *__restrict__ prefix, uint32_t n_chunks, uint32_t spans_per_row, uint32_t n_items,
                     const uint16_t *__restrict__ x, int m, int64_t ldx, uint16_t *__restrict__ y, int64_t ldy,
                     float *__restrict__ ws, bool by_rows) {
    __shared__ __attribute__((aligned(16))) uint32_t lut[kDnLutBytes / 4];
    __shared__ __attribute__((aligned(16))) uint16_t wc_all[kDnWaves][kDnSlots];
    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const float scale = bf16_bits_to_f32(*P.scale);
    for (uint32_t e = tid; e < 64 * 32; e += kWave * kDnWaves) {
        const uint32_t idx = e >> 5;
        lut[e] = dn_pack(dequant((int)(idx & 7u) - 3, scale), dequant((int)(idx >> 3) - 3, scale));
    }
    // Lanes past a row's end gather from wherever their walk leads, inside the wave's arrays; their activations are
    // zero, so what they find only has to be finite: start from zeros (later contents are weights).
    for (uint32_t j = lane; j < kDnSlots / 8; j += kWave) reinterpret_cast<d_u32x4 *>(wc_all[wave])[j] = d_u32x4{0, 0, 0, 0};
    __syncthreads();
    const uint32_t stride = gridDim.x * kDnWaves;
    const DnRowSpans spans{n_chunks, spans_per_row, n_items, blockIdx.x * kDnWaves + wave, stride, stride / spans_per_row,
                           stride % spans_per_row, by_rows};
    DnDotSink<MT> sink;
    sink.x = x; sink.ldx = ldx; sink.m = m; sink.y = y; sink.ldy = ldy; sink.ws = ws;
    sink.out_f = P.out_f; sink.spans_per_row = spans_per_row; sink.lane = lane; sink.by_rows = by_rows;
#pragma unroll
    for (int j = 0; j < 2 * MT; ++j) sink.row_total[j] = 0.0f;
    dn_walk_spans<false>(P, prefix, P.out_f * n_chunks + 1, nullptr, 0u, lut, wc_all[wave], scale, lane, spans, sink, wave);
}

// ---------------------------------------------------------------------------------------------------------------
// Product with 2..16 activation rows for dense mixes on the matrix pipe: the walker above, 16 waves to a workgroup,
// with the sink of ixh_dense_tiles.h (the 16 waves' spans as a tile in LDS, v_mfma_f32_16x16x32_bf16, pieces of partial
// sums for k_reduce_chunks).  The decode costs what it costs the full decoder, whatever the number of activation rows.
// ---------------------------------------------------------------------------------------------------------------
constexpr uint32_t kDtRegion = kDnSlots * 2 + 16;  // bytes between the waves' arrays
constexpr size_t kDtLdsBytes = kDnLutBytes + (size_t)kDtWaves * kDtRegion + kDtSumsBytes;

// the workgroup's steps [step_begin, step_end) of the sequence (row block, span); this wave's row of every block
struct DnTileSpans {
    uint32_t n_chunks, spans_per_row, out_f, wave, step_begin, step_end;
    __device__ __forceinline__ DnSpan at(uint32_t step) const {
        DnSpan sp;
        const uint32_t rb = step / spans_per_row, k = step - rb * spans_per_row;
        const uint32_t row = min(rb * (uint32_t)kDtWaves + wave, out_f - 1u);  // a wave past the last row decodes it again
        const uint32_t nb = min(4u, n_chunks - 4 * k);
        sp.u0 = row * n_chunks + 4 * k;
        sp.u1 = sp.u0 + nb;
        sp.p0 = sp.u0 * kFastChunk;
        sp.n_el = nb * kFastChunk;
        sp.a = rb; sp.b = k; sp.c = step;
        return sp;
    }
    __device__ __forceinline__ bool first_span(DnSpan &sp) const {
        if (step_begin >= step_end) return false;
        sp = at(step_begin);
        return true;
    }
    __device__ __forceinline__ bool next(const DnSpan &cur, DnSpan &nx) const {
        if (cur.c + 1 >= step_end) return false;
        nx = at(cur.c + 1);
        return true;
    }
};

struct DnMfmaSink {
    DtMfmaSink<kDtRegion> t;
    __device__ __forceinline__ void begin(const DnSpan &sp) { t.begin(DtStep{sp.a, sp.b, sp.c}); }
    __device__ __forceinline__ void end(const DnSpan &sp, const uint32_t (&o)[16], uint32_t) { t.end(DtStep{sp.a, sp.b, sp.c}, o); }
};

__global__ void __launch_bounds__(kWave *kDtWaves)
k_gemv358_dense_tiles(Dev P, const int32_t *__restrict__ prefix, uint32_t n_chunks, uint32_t spans_per_row, uint32_t total_steps,
                      const uint16_t *__restrict__ x, int m, int64_t ldx, float *__restrict__ ws, uint32_t n_pieces) {
    extern __shared__ __attribute__((aligned(16))) uint8_t dt_smem[];
    uint32_t *const lut = reinterpret_cast<uint32_t *>(dt_smem);
    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    uint16_t *const wc = reinterpret_cast<uint16_t *>(dt_smem + kDnLutBytes + wave * kDtRegion);
    const float scale = bf16_bits_to_f32(*P.scale);
    for (uint32_t e = tid; e < 64 * 32; e += kWave * kDtWaves) {
        const uint32_t idx = e >> 5;
        lut[e] = dn_pack(dequant((int)(idx & 7u) - 3, scale), dequant((int)(idx >> 3) - 3, scale));
    }
    // Lanes past a row's end gather from wherever their walk leads, inside the wave's array; their activations are
    // zero, so what they find only has to be finite: start from zeros (later contents are weights).
    for (uint32_t j = lane; j < kDtRegion / 16; j += kWave) reinterpret_cast<d_u32x4 *>(wc)[j] = d_u32x4{0, 0, 0, 0};
    __syncthreads();
    const uint32_t step_begin = (uint32_t)((uint64_t)blockIdx.x * total_steps / gridDim.x);
    const uint32_t step_end = (uint32_t)(((uint64_t)blockIdx.x + 1u) * total_steps / gridDim.x);
    const DnTileSpans spans{n_chunks, spans_per_row, P.out_f, wave, step_begin, step_end};
    DnMfmaSink sink;
    sink.t.x = x; sink.t.ldx = ldx; sink.t.m = m; sink.t.ws = ws;
    sink.t.out_f = P.out_f; sink.t.in_f = P.in_f; sink.t.spans_per_row = spans_per_row; sink.t.n_pieces = n_pieces;
    sink.t.total_steps = total_steps; sink.t.step_end = step_end;
    sink.t.wave = wave; sink.t.lane = lane; sink.t.wc = wc;
    sink.t.tile_addr = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t *)(dt_smem + kDnLutBytes);
    sink.t.red = reinterpret_cast<float *>(dt_smem + kDnLutBytes + (size_t)kDtWaves * kDtRegion);
    sink.t.acc = dt_f32x4{0.f, 0.f, 0.f, 0.f};
    dn_walk_spans<false, DnTileSpans, DnMfmaSink, false>(P, prefix, P.out_f * n_chunks + 1, nullptr, 0u, lut, wc, scale, lane,
                                                         spans, sink, wave);
}

bool gemv_dense358_tiles_supports(const Dev &P, uint32_t chunk, int m, const uint16_t *x, int64_t ldx) {
    return P.n_levels == 3 && P.bits[0] == 3 && P.bits[1] == 5 && P.bits[2] == 8 && chunk == kFastChunk && m >= 2 && m <= 16 &&
           P.in_f % kFastChunk == 0 && P.in_f >= 2 * kFastChunk && ((uintptr_t)x & 15u) == 0 && (ldx & 7) == 0 &&
           ((uintptr_t)P.last & 3u) == 0 && P.out_f != 0;
}

static uint32_t dt_cu_count() {
    static const uint32_t n_cu = [] {
        int dev = 0, v = 256;
        if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev);
        return (uint32_t)v;
    }();
    return n_cu;
}

// The workspace holds n_pieces x m x out_f partial sums (n_pieces <= in_f / 512, what ixh_gemv_workspace_bytes asks for).
int launch_gemv_dense358_tiles(const Dev &P, const int32_t *prefix, const uint16_t *x, int m, int64_t ldx, uint16_t *y,
                               int64_t ldy, float *ws, hipStream_t s) {
    static const bool raised = hipFuncSetAttribute(reinterpret_cast<const void *>(k_gemv358_dense_tiles),
                                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)kDtLdsBytes) == hipSuccess;
    if (!raised) return IXH_EUNSUPPORTED;
    const DtPlan plan = dt_plan(P.out_f, P.in_f, dt_cu_count());
    if (plan.groups == 0) return IXH_EUNSUPPORTED;
    hipLaunchKernelGGL(k_gemv358_dense_tiles, dim3(plan.groups), dim3(kWave * kDtWaves), kDtLdsBytes, s, P, prefix,
                       plan.n_chunks, plan.spans_per_row, plan.total_steps, x, m, ldx, ws, plan.n_pieces);
    if (hipGetLastError() != hipSuccess) return IXH_ELAUNCH;
    return launch_reduce_chunks(ws, plan.n_pieces, m, P.out_f, y, ldy, s);
}

bool gemv_dense358_rows_supports(const Dev &P, uint32_t chunk, int m, const uint16_t *x, int64_t ldx) {
    return P.n_levels == 3 && P.bits[0] == 3 && P.bits[1] == 5 && P.bits[2] == 8 && chunk == kFastChunk && m >= 2 && m <= 8 &&
           P.in_f % kFastChunk == 0 && P.in_f != 0 && ((uintptr_t)x & 15u) == 0 && (ldx & 7) == 0 &&
           ((uintptr_t)P.last & 3u) == 0;
}

template <int MT>
static int launch_dense_rows(const Dev &P, const int32_t *prefix, const uint16_t *x, int m, int64_t ldx, uint16_t *y,
                             int64_t ldy, float *ws, hipStream_t s) {
    const uint32_t n_chunks = P.in_f / kFastChunk;
    const uint32_t spans_per_row = (n_chunks + 3) / 4;
    const uint32_t n_spans = P.out_f * spans_per_row;
    if (n_spans == 0) return IXH_OK;
    static const uint32_t resident = [] {
        int dev = 0, n_cu = 256, per_cu = 0;
        if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev);
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, k_gemv358_dense_rows<MT>, kWave * kDnWaves, 0) != hipSuccess ||
            per_cu < 1)
            per_cu = 3;
        return (uint32_t)n_cu * (uint32_t)per_cu;
    }();
    // whole rows per wave when they spread over the resident waves within 12 % (one launch, no workspace); otherwise
    // spans are dealt out and a second kernel adds a row's partial sums in span order
    const uint32_t waves_res = resident * kDnWaves;
    const uint32_t rounds = (P.out_f + waves_res - 1) / waves_res;
    const bool by_rows = spans_per_row == 1 || (uint64_t)rounds * waves_res * 100u <= (uint64_t)P.out_f * 112u;
    const uint32_t n_items = by_rows ? P.out_f : n_spans;
    const uint32_t blocks = min(resident, (n_items + kDnWaves - 1) / kDnWaves);
    hipLaunchKernelGGL(k_gemv358_dense_rows<MT>, dim3(blocks), dim3(kWave * kDnWaves), 0, s, P, prefix, n_chunks, spans_per_row,
                       n_items, x, m, ldx, y, ldy, ws, by_rows);
    if (hipGetLastError() != hipSuccess) return IXH_ELAUNCH;
    if (!by_rows) return launch_reduce_chunks(ws, spans_per_row, m, P.out_f, y, ldy, s);
    return IXH_OK;
}

int launch_gemv_dense358_rows(const Dev &P, const int32_t *prefix, const uint16_t *x, int m, int64_t ldx, uint16_t *y,
                              int64_t ldy, float *ws, hipStream_t s) {
    return m <= 2 ? launch_dense_rows<2>(P, prefix, x, m, ldx, y, ldy, ws, s)
                  : launch_dense_rows<4>(P, prefix, x, m, ldx, y, ldy, ws, s);
}

bool decode_dense358_supports(const Dev &P, uint32_t chunk, const int8_t *o8, const uint16_t *o16, GroupScales gs) {
    if (gs.fp16 && (gs.group < 32 || (gs.group & (gs.group - 1)) != 0)) return false;  // one scale per lane, by a shift
    return P.n_levels == 3 && P.bits[0] == 3 && P.bits[1] == 5 && P.bits[2] == 8 && chunk == kFastChunk && !o8 && o16 &&
           ((uintptr_t)o16 & 15u) == 0 && ((uintptr_t)P.last & 3u) == 0 && P.n != 0;
}

int launch_decode_dense358(const Dev &P, const int32_t *prefix, uint16_t *o16, GroupScales gs, hipStream_t s) {
    const uint32_t n_units = (P.n + kFastChunk - 1) / kFastChunk;
    const uint32_t n_spans = (n_units + 3) / 4;
    static const uint32_t resident = [] {
        int dev = 0, n_cu = 256, per_cu = 0;
        if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev);
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, k_decode358_dense<true>, kWave * kDnWaves, 0) != hipSuccess || per_cu < 1)
            per_cu = 4;
        return (uint32_t)n_cu * (uint32_t)per_cu;
    }();
    const uint32_t blocks = min(resident, (n_spans + kDnWaves - 1) / kDnWaves);
    if (gs.fp16)
        hipLaunchKernelGGL(k_decode358_dense<true>, dim3(blocks), dim3(kWave * kDnWaves), 0, s, P, prefix, n_units, n_spans, o16,
                           gs.fp16, (uint32_t)__builtin_ctz(gs.group));
    else
        hipLaunchKernelGGL(k_decode358_dense<false>, dim3(blocks), dim3(kWave * kDnWaves), 0, s, P, prefix, n_units, n_spans, o16,
                           (const uint16_t *)nullptr, 0u);
    return hipGetLastError() == hipSuccess ? IXH_OK : IXH_ELAUNCH;
}

bool gemv_dense358_supports(const Dev &P, uint32_t chunk, int m, const uint16_t *x) {
    return P.n_levels == 3 && P.bits[0] == 3 && P.bits[1] == 5 && P.bits[2] == 8 && chunk == kFastChunk && m == 1 &&
           P.in_f % kFastChunk == 0 && P.in_f != 0 && ((uintptr_t)x & 15u) == 0 && ((uintptr_t)P.last & 3u) == 0;
}

uint32_t gemv_dense358_pieces(const Dev &P) { return (P.in_f / kFastChunk + 3) / 4; }

int launch_gemv_dense358(const Dev &P, const int32_t *prefix, const uint16_t *x, uint16_t *y, float *y32, float *ws,
                         bool atomic, hipStream_t s) {
    const uint32_t n_chunks = P.in_f / kFastChunk;
    const uint32_t spans_per_row = (n_chunks + 3) / 4;
    const uint32_t n_spans = P.out_f * spans_per_row;
    if (n_spans == 0) return IXH_OK;
    // one resident set of workgroups; each wave walks the spans with the stride of the launch
    static const uint32_t resident = [] {
        int dev = 0, n_cu = 256, per_cu = 0;
        if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev);
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, k_gemv358_dense, kWave * kDnWaves, 0) != hipSuccess || per_cu < 1)
            per_cu = 4;
        return (uint32_t)n_cu * (uint32_t)per_cu;
    }();
    // Whole rows per wave when they spread over the resident waves within 12 %: one launch, no workspace, each
    // output summed in one register.  Otherwise spans are dealt out and a second kernel adds a row's partial sums.
    const uint32_t waves_res = resident * kDnWaves;
    const uint32_t rounds = (P.out_f + waves_res - 1) / waves_res;
    const bool by_rows = spans_per_row == 1 || (uint64_t)rounds * waves_res * 100u <= (uint64_t)P.out_f * 112u;
    const uint32_t n_items = by_rows ? P.out_f : n_spans;
    const uint32_t blocks = min(resident, (n_items + kDnWaves - 1) / kDnWaves);
    const int out_mode = atomic ? kDnAtomic : (by_rows ? kDnDirect : kDnWorkspace);
    hipLaunchKernelGGL(k_gemv358_dense, dim3(blocks), dim3(kWave * kDnWaves), 0, s, P, prefix, n_chunks, spans_per_row,
                       n_spans, x, y, y32, ws, out_mode, by_rows);
    if (hipGetLastError() != hipSuccess) return IXH_ELAUNCH;
    if (out_mode == kDnWorkspace) return launch_reduce_chunks(ws, spans_per_row, 1, P.out_f, y, P.out_f, s);
    return IXH_OK;
}

}  // namespace ixh
