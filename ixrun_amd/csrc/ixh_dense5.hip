// (3,4,5,6,8) fused decode + GEMV for one activation row when the levels above the first are well populated (the
// reference's five-level scheme on real weights: about 5.3 bits per weight): the level-by-level method of
// ixh_dense358.hip with five levels.
//
//     sum_k w_k x_k = sum over the levels of (sum_{k in level} w_k x_k)
// The codes of a level are dense in their stream, so each level's sum is taken over whole codes at fixed positions,
// and what depends on the bitmaps is moved to the activations: the x values of a span are scattered into five arrays
// in LDS, one per level, in the order of that level's codes.
//
// A wave takes spans of up to 2048 consecutive elements of one weight row (four 512-element table units).  The rank
// table gives the span's first code in every stream and its level counts.  Lane l owns word l of the first bitmap (32
// elements, 16 x pairs in registers).  The nested bitmaps of the span (at most 2048 bits each) are copied to LDS from
// addresses that follow from the table alone; a lane's window into each of them starts at its number of elements that
// no earlier level claimed, which comes from one wave prefix sum per level.  The scatter walks two elements per step
// (t and t + 16) with all running slots and bitmap cursors in packed 16-bit halves.  The dense passes split each
// level's codes evenly over the 64 lanes (a multiple of four per lane), read them through buffer descriptors, and
// meet the compacted x pairs in v_dot2_f32_bf16: level 1 through the table of dequantised pairs, the others as
// fma(code, scale, -T * scale), exact in fp32, rounded to bf16 as the reference's decoder does
// (ixrun/triton_kernels.py:168-177).  Every array is padded with zeros up to 64 x codes-per-lane.
#include "ixh_dense_tiles.h"
#include "ixh_fast358.h"

namespace ixh {

typedef uint32_t e_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t e_u32x3 __attribute__((ext_vector_type(3)));
typedef uint32_t e_u32x2 __attribute__((ext_vector_type(2)));
typedef uint16_t e_u16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 e_bf16x2 __attribute__((ext_vector_type(2)));
typedef float e_f32x2 __attribute__((ext_vector_type(2)));

constexpr int kD5Waves = 4;                       // waves per workgroup
constexpr uint32_t kD5Span = 2048;                // elements per span: four table units of one row
constexpr uint32_t kD5Slots = kD5Span + 5 * 256;  // compacted x slots per wave: five arrays, each padded to 64 * E
constexpr uint32_t kD5BmWords = 68;               // staged words of a nested bitmap: 2048 bits from any bit of a word on
constexpr uint32_t kD5LutBytes = 64 * 32 * 4;     // pair table: 64 code pairs x 32 lane copies

enum : int { kD5Direct = 0, kD5Atomic = 1, kD5Workspace = 2 };

#define IXH_D5_DPP_ADD(v, ctrl, row_mask, bound) \
    v += __uint_as_float((uint32_t)__builtin_amdgcn_update_dpp(0, (int)__float_as_uint(v), ctrl, row_mask, 0xf, bound))
// sum over the wave, valid in lane 63
__device__ __forceinline__ float d5_wave_sum(float v) {
    IXH_D5_DPP_ADD(v, 0x111, 0xf, true);
    IXH_D5_DPP_ADD(v, 0x112, 0xf, true);
    IXH_D5_DPP_ADD(v, 0x114, 0xf, true);
    IXH_D5_DPP_ADD(v, 0x118, 0xf, true);
    IXH_D5_DPP_ADD(v, 0x142, 0xa, false);
    IXH_D5_DPP_ADD(v, 0x143, 0xc, false);
    return v;
}
#undef IXH_D5_DPP_ADD

__device__ __forceinline__ uint32_t d5_pack(float lo, float hi) {
    const e_f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, e_bf16x2));
}

__device__ __forceinline__ float d5_dot2(uint32_t w, uint32_t x, float acc) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(e_bf16x2, w), __builtin_bit_cast(e_bf16x2, x), acc, false);
}

// the low `n` bits set (n = 0 .. 32)
__device__ __forceinline__ uint32_t d5_low_mask(uint32_t n) { return (uint32_t)(0xFFFFFFFFull >> (32u - n)); }

// A lane's window of a code stream: B + 1 dwords from the dword that holds the bit `first_bit` on (d5_fetch), shifted
// so that the bit lands at bit 0 of w[0] (d5_align).  A dword past the stream's end reads as zero.
template <int B>
__device__ __forceinline__ void d5_fetch(__amdgpu_buffer_rsrc_t rsrc, uint64_t first_bit, uint32_t (&d)[B + 1]) {
    const uint32_t at = (uint32_t)(first_bit >> 5) * 4u;
#pragma unroll
    for (int j = 0; j + 4 <= B + 1; j += 4) {
        const e_u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)(at + 4u * j), 0, 0);
        d[j] = v[0]; d[j + 1] = v[1]; d[j + 2] = v[2]; d[j + 3] = v[3];
    }
    constexpr int done = ((B + 1) / 4) * 4, rest = B + 1 - done;
    if constexpr (rest == 1) {
        d[done] = __builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)(at + 4u * done), 0, 0);
    } else if constexpr (rest == 2) {
        const e_u32x2 v = __builtin_amdgcn_raw_buffer_load_b64(rsrc, (int)(at + 4u * done), 0, 0);
        d[done] = v[0]; d[done + 1] = v[1];
    } else if constexpr (rest == 3) {
        const e_u32x3 v = __builtin_amdgcn_raw_buffer_load_b96(rsrc, (int)(at + 4u * done), 0, 0);
        d[done] = v[0]; d[done + 1] = v[1]; d[done + 2] = v[2];
    }
}

template <int B>
__device__ __forceinline__ void d5_align(const uint32_t (&d)[B + 1], uint64_t first_bit, uint32_t (&w)[B]) {
    const uint32_t sh = (uint32_t)first_bit & 31u;
#pragma unroll
    for (int j = 0; j < B; ++j) w[j] = __builtin_amdgcn_alignbit(d[j + 1], d[j], sh);
}

template <int B>
__device__ __forceinline__ void d5_window(__amdgpu_buffer_rsrc_t rsrc, uint64_t first_bit, uint32_t (&w)[B]) {
    uint32_t d[B + 1];
    d5_fetch<B>(rsrc, first_bit, d);
    d5_align<B>(d, first_bit, w);
}

// code t (a compile-time index) of a window of B-bit codes
template <int B>
__device__ __forceinline__ uint32_t d5_code(const uint32_t (&w)[B], int t) {
    const int bit = B * t, ob = bit & 31, d = bit >> 5;
    constexpr uint32_t mask = (1u << B) - 1u;
    if (ob + B <= 32) return (w[d] >> ob) & mask;
    return __builtin_amdgcn_alignbit(d + 1 < B ? w[d + 1] : 0u, w[d], ob) & mask;
}

// one level's dense pass: e codes of this lane (a multiple of four, at most 32) against its row of compacted x pairs.
// Groups of two pairs; a group is entered only if the level has codes for it (the empty asm statements keep the
// group tests branches: as selects, all eight groups would run for every span).
template <int B>
__device__ __forceinline__ float d5_pass(const uint32_t (&w)[B], const uint32_t *xp, uint32_t e, float scale,
                                         float minus_t_scale, float acc) {
#pragma unroll
    for (int g = 0; g < 8; ++g) {
        if (e > 4u * g) {
            asm volatile("");
#pragma unroll
            for (int t = 2 * g; t < 2 * g + 2; ++t) {
                // (c - T) * scale as c * scale - T * scale: both products and their difference are exact in fp32
                // (codes and T have at most 8 significant bits, the bf16 scale 8): nothing is rounded twice
                const uint32_t c0 = d5_code<B>(w, 2 * t), c1 = d5_code<B>(w, 2 * t + 1);
                const uint32_t wp = d5_pack(__fmaf_rn((float)c0, scale, minus_t_scale), __fmaf_rn((float)c1, scale, minus_t_scale));
                acc = d5_dot2(wp, xp[t], acc);
            }
        }
    }
    return acc;
}

__global__ void __launch_bounds__(kWave *kD5Waves)
k_gemv34568_dense(Dev P, const int32_t *__restrict__ prefix, uint32_t n_chunks, uint32_t spans_per_row, uint32_t n_spans,
                  const uint16_t *__restrict__ x, uint16_t *__restrict__ y, float *__restrict__ y32,
                  float *__restrict__ ws, int out_mode, bool by_rows) {
    __shared__ __attribute__((aligned(16))) uint32_t lut[kD5LutBytes / 4];
    __shared__ __attribute__((aligned(16))) uint16_t xc_all[kD5Waves][kD5Slots];
    __shared__ uint32_t bm_all[kD5Waves][3][kD5BmWords];
    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const float scale = bf16_bits_to_f32(*P.scale);
    const float m7 = -7.0f * scale, m15 = -15.0f * scale, m31 = -31.0f * scale, m127 = -127.0f * scale;  // exact

    // pair table: entry (c0 | c1 << 3) = the two dequantised level-1 weights, one copy per bank
    for (uint32_t e = tid; e < 64 * 32; e += kWave * kD5Waves) {
        const uint32_t idx = e >> 5;
        lut[e] = d5_pack(dequant((int)(idx & 7u) - 3, scale), dequant((int)(idx >> 3) - 3, scale));
    }
    __syncthreads();

    uint16_t *const xc = xc_all[wave];
    uint32_t(*const bmw)[kD5BmWords] = bm_all[wave];
    const uint32_t lut_lane = (lane & 31u) << 2;
    const uint32_t entries = P.out_f * n_chunks + 1;
    const uint32_t *__restrict__ b1 = P.bm[0];
    const __amdgpu_buffer_rsrc_t st_rsrc[4] = {
        __builtin_amdgcn_make_buffer_rsrc((void *)P.st[0], 0, (int)(P.st_words[0] * 4u), 0x00020000),
        __builtin_amdgcn_make_buffer_rsrc((void *)P.st[1], 0, (int)(P.st_words[1] * 4u), 0x00020000),
        __builtin_amdgcn_make_buffer_rsrc((void *)P.st[2], 0, (int)(P.st_words[2] * 4u), 0x00020000),
        __builtin_amdgcn_make_buffer_rsrc((void *)P.st[3], 0, (int)(P.st_words[3] * 4u), 0x00020000)};
    // whole dwords of the byte stream (device allocations are 256-byte granular, the last dword is there to read)
    const __amdgpu_buffer_rsrc_t last_rsrc =
        __builtin_amdgcn_make_buffer_rsrc((void *)P.last, 0, (int)((P.last_bytes + 3u) & ~3u), 0x00020000);
    const __amdgpu_buffer_rsrc_t bm_rsrc[3] = {
        __builtin_amdgcn_make_buffer_rsrc((void *)P.bm[1], 0, (int)(P.bm_words[1] * 4u), 0x00020000),
        __builtin_amdgcn_make_buffer_rsrc((void *)P.bm[2], 0, (int)(P.bm_words[2] * 4u), 0x00020000),
        __builtin_amdgcn_make_buffer_rsrc((void *)P.bm[3], 0, (int)(P.bm_words[3] * 4u), 0x00020000)};

    // Work is dealt to the waves of the launch in turn; the launch is resident as a whole.  An item is a whole row (its
    // spans are summed in the wave and the result leaves as it is) or, when rows would not spread evenly, one span
    // (partial sums meet in the workspace).
    const uint32_t n_waves = gridDim.x * kD5Waves;
    const uint32_t n_items = by_rows ? P.out_f : n_spans;
    for (uint32_t item = blockIdx.x * kD5Waves + wave; item < n_items; item += n_waves) {
      const uint32_t row = by_rows ? item : item / spans_per_row;
      const uint32_t k_first = by_rows ? 0u : item - row * spans_per_row;
      const uint32_t k_end = by_rows ? spans_per_row : k_first + 1u;
      float row_total = 0.0f;  // meaningful in lane 63
      for (uint32_t k = k_first; k < k_end; ++k) {
        {   // the waves that share a SIMD take turns at the issue priority, one span each
            const uint32_t turn = (wave + k) % 3u;  // s_setprio takes an immediate
            if (turn == 0) __builtin_amdgcn_s_setprio(0);
            else if (turn == 1) __builtin_amdgcn_s_setprio(1);
            else __builtin_amdgcn_s_setprio(2);
        }
        const uint32_t c0 = 4 * k, nb = min(4u, n_chunks - c0);
        const uint32_t u0 = row * n_chunks + c0;
        const uint32_t n_el = nb * kFastChunk, p0 = u0 * kFastChunk;
        // codes of each level before the span, and in it
        uint32_t qa[4], cnt[5];
        {
            uint32_t rest = n_el;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                qa[i] = (uint32_t)prefix[(size_t)i * entries + u0];
                cnt[i] = (uint32_t)prefix[(size_t)i * entries + u0 + nb] - qa[i];
                rest -= cnt[i];
            }
            cnt[4] = rest;
        }
        // codes per lane in the dense passes (a multiple of four), and where each level's compacted array starts
        uint32_t e[5], base[5];
        {
            uint32_t at = 0;
#pragma unroll
            for (int i = 0; i < 5; ++i) {
                e[i] = 4 * ((cnt[i] + 255) / 256);
                base[i] = at;
                at += 64 * e[i];
            }
        }
        // first bit of the span in each nested bitmap's domain: its elements that no earlier level claimed
        const uint32_t g1 = p0 - qa[0], g2 = g1 - qa[1], g3 = g2 - qa[2], at_last = g3 - qa[3];

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
        // the span's part of the nested bitmaps: 65 words each from the word that holds its first bit
        {
            const uint32_t gs[3] = {g1, g2, g3};
#pragma unroll
            for (int j = 0; j < 3; ++j) {
                const uint32_t w0 = gs[j] >> 5;
                bmw[j][lane] = __builtin_amdgcn_raw_buffer_load_b32(bm_rsrc[j], (int)((w0 + lane) * 4u), 0, 0);
                if (lane < 4) bmw[j][64 + lane] = __builtin_amdgcn_raw_buffer_load_b32(bm_rsrc[j], (int)((w0 + 64u + lane) * 4u), 0, 0);
            }
        }
        // The code streams, read through buffer descriptors: a dword past a stream's end reads as zero, so no lane
        // needs a bounds test; lanes whose share lies past the level's last code read codes of the next span, which
        // then meet the zero pads of the compacted arrays.
        uint32_t c1w[3], c2w[4], c3w[5], c4w[6], c5w[8];
        d5_window<3>(st_rsrc[0], (uint64_t)(qa[0] + lane * e[0]) * 3u, c1w);
        d5_window<4>(st_rsrc[1], (uint64_t)(qa[1] + lane * e[1]) * 4u, c2w);
        d5_window<5>(st_rsrc[2], (uint64_t)(qa[2] + lane * e[2]) * 5u, c3w);
        d5_window<6>(st_rsrc[3], (uint64_t)(qa[3] + lane * e[3]) * 6u, c4w);
        d5_window<8>(last_rsrc, (uint64_t)(at_last + lane * e[4]) * 8u, c5w);

        // ---- clear the compacted arrays (the pads must read as zero) ----
        for (uint32_t j = lane; j < kD5Slots / 8; j += kWave) reinterpret_cast<e_u32x4 *>(xc)[j] = e_u32x4{0, 0, 0, 0};

        // ---- ranks: first slot of this lane in each array ----
        // a lane's window into nested bitmap j starts at the span's first bit there plus the elements of the lanes
        // below that no earlier level claimed
        auto window = [&](int j, uint32_t g, uint32_t first, uint32_t alive) {
            const uint32_t o = (g & 31u) + first;
            const uint32_t lo = bmw[j][o >> 5], hi = bmw[j][(o >> 5) + 1];
            return __builtin_amdgcn_alignbit(hi, lo, o & 31u) & d5_low_mask(alive);
        };
        const uint32_t cnt1 = (uint32_t)__popc(w1);
        const uint32_t alive1 = valid ? 32u - cnt1 : 0u;
        const uint32_t sc1 = wave_scan_inclusive(cnt1 | (alive1 << 16));
        const uint32_t first1 = (sc1 & 0xffffu) - cnt1, first_a1 = (sc1 >> 16) - alive1;
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
        const uint32_t bits2 = window(0, g1, first_a1, alive1);  // bit j: the lane's j-th element above level 1 is level 2
        const uint32_t cnt2 = (uint32_t)__popc(bits2), alive2 = alive1 - cnt2;
        const uint32_t sc2 = wave_scan_inclusive(cnt2 | (alive2 << 16));
        const uint32_t first2 = (sc2 & 0xffffu) - cnt2, first_a2 = (sc2 >> 16) - alive2;
        const uint32_t bits3 = window(1, g2, first_a2, alive2);
        const uint32_t cnt3 = (uint32_t)__popc(bits3), alive3 = alive2 - cnt3;
        const uint32_t sc3 = wave_scan_inclusive(cnt3 | (alive3 << 16));
        const uint32_t first3 = (sc3 & 0xffffu) - cnt3, first_a3 = (sc3 >> 16) - alive3;
        const uint32_t bits4 = window(2, g3, first_a3, alive3);
        const uint32_t cnt4 = (uint32_t)__popc(bits4);
        const uint32_t first4 = wave_scan_inclusive(cnt4) - cnt4;
        const uint32_t first5 = first_a3 - first4;

        // ---- scatter the lane's 32 activations to their levels' arrays ----
        // Two elements per step, t and t + 16, with their counters in the two halves of one register (packed 16-bit
        // arithmetic): each half holds "LDS byte address / 2" of the next slot of its level.  The second half starts
        // where the first one will end: behind the level counts of the lane's first 16 elements.  in1 .. in5 are 0 or
        // 1 per half; the slot is picked by multiply-add.  ja, jb, jc count the elements that levels 1, 1..2 and 1..3
        // have passed on: the cursors into the three nested windows.
        {
            const uint32_t xc_half = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint16_t *)xc >> 1;
            const uint32_t low1 = (uint32_t)__popc(w1 & 0xffffu);  // level-1 elements among the first 16
            const uint32_t low_a1 = valid ? 16u - low1 : 0u;          // elements above level 1 among them
            const uint32_t low2 = (uint32_t)__popc(bits2 & d5_low_mask(low_a1)), low_a2 = low_a1 - low2;
            const uint32_t low3 = (uint32_t)__popc(bits3 & d5_low_mask(low_a2)), low_a3 = low_a2 - low3;
            const uint32_t low4 = (uint32_t)__popc(bits4 & d5_low_mask(low_a3)), low5 = low_a3 - low4;
            const uint32_t a1 = xc_half + base[0] + first1, a2 = xc_half + base[1] + first2, a3 = xc_half + base[2] + first3;
            const uint32_t a4 = xc_half + base[3] + first4, a5 = xc_half + base[4] + first5;
            e_u16x2 s1 = __builtin_bit_cast(e_u16x2, a1 | ((a1 + low1) << 16));
            e_u16x2 s2 = __builtin_bit_cast(e_u16x2, a2 | ((a2 + low2) << 16));
            e_u16x2 s3 = __builtin_bit_cast(e_u16x2, a3 | ((a3 + low3) << 16));
            e_u16x2 s4 = __builtin_bit_cast(e_u16x2, a4 | ((a4 + low4) << 16));
            e_u16x2 s5 = __builtin_bit_cast(e_u16x2, a5 | ((a5 + low5) << 16));
            // the flags each half walks through: from bit 0, and from where the first 16 elements will have got to
            // (a 64-bit shift: 32 is a legal count when no element of the first half gets that far)
            const e_u16x2 f2 = __builtin_bit_cast(e_u16x2, (bits2 & 0xffffu) | ((uint32_t)((uint64_t)bits2 >> low_a1) << 16));
            const e_u16x2 f3 = __builtin_bit_cast(e_u16x2, (bits3 & 0xffffu) | ((uint32_t)((uint64_t)bits3 >> low_a2) << 16));
            const e_u16x2 f4 = __builtin_bit_cast(e_u16x2, (bits4 & 0xffffu) | ((uint32_t)((uint64_t)bits4 >> low_a3) << 16));
            e_u16x2 ja = {0, 0}, jb = {0, 0}, jc = {0, 0};
            const e_u16x2 one = {1, 1};
#pragma unroll
            for (int t = 0; t < 16; ++t) {
                const e_u16x2 in1 = __builtin_bit_cast(e_u16x2, (w1 >> t) & 0x00010001u);
                const e_u16x2 out1 = in1 ^ one;
                const e_u16x2 in2 = (f2 >> ja) & out1;
                const e_u16x2 out2 = out1 ^ in2;
                const e_u16x2 in3 = (f3 >> jb) & out2;
                const e_u16x2 out3 = out2 ^ in3;
                const e_u16x2 in4 = (f4 >> jc) & out3;
                const e_u16x2 in5 = out3 ^ in4;
                const e_u16x2 at = in1 * (s1 - s5) + (in2 * (s2 - s5) + (in3 * (s3 - s5) + (in4 * (s4 - s5) + s5)));
                const uint32_t at32 = __builtin_bit_cast(uint32_t, at);
                const uint32_t x_lo = xr[t >> 1], x_hi = xr[8 + (t >> 1)];
                // lanes past the span scatter zeros behind the last array's entries
                *reinterpret_cast<__attribute__((address_space(3))) uint16_t *>((uintptr_t)((at32 & 0xffffu) << 1)) =
                    (uint16_t)((t & 1) ? x_lo >> 16 : x_lo);
                *reinterpret_cast<__attribute__((address_space(3))) uint16_t *>((uintptr_t)((at32 >> 16) << 1)) =
                    (uint16_t)((t & 1) ? x_hi >> 16 : x_hi);
                s1 += in1; s2 += in2; s3 += in3; s4 += in4; s5 += in5;
                ja += out1; jb += out2; jc += out3;
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();

        // ---- dense passes ----
        float acc = 0.0f;
        {   // level 1: pairs of 3-bit codes through the pair table
            const uint32_t *xp = reinterpret_cast<const uint32_t *>(xc) + (lane * e[0]) / 2;
#pragma unroll
            for (int g = 0; g < 8; ++g) {
                if (e[0] > 4u * g) {
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
                        acc = d5_dot2(wp, xp[t], acc);
                    }
                }
            }
        }
        acc = d5_pass<4>(c2w, reinterpret_cast<const uint32_t *>(xc) + (base[1] + lane * e[1]) / 2, e[1], scale, m7, acc);
        acc = d5_pass<5>(c3w, reinterpret_cast<const uint32_t *>(xc) + (base[2] + lane * e[2]) / 2, e[2], scale, m15, acc);
        acc = d5_pass<6>(c4w, reinterpret_cast<const uint32_t *>(xc) + (base[3] + lane * e[3]) / 2, e[3], scale, m31, acc);
        acc = d5_pass<8>(c5w, reinterpret_cast<const uint32_t *>(xc) + (base[4] + lane * e[4]) / 2, e[4], scale, m127, acc);
        row_total += d5_wave_sum(acc);
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
      }
      if (lane == 63) {
          if (out_mode == kD5Direct) y[row] = (uint16_t)f32_to_bf16_bits(row_total);
          else if (out_mode == kD5Atomic) atomicAdd(y32 + row, row_total);
          else ws[(size_t)k_first * P.out_f + row] = row_total;
      }
    }
}

// ---------------------------------------------------------------------------------------------------------------
// The full decode by the same route turned round (for dense mixes): the codes of each level are dequantised where they
// lie (dense, fixed positions) into five LDS arrays of bf16 weights, and every lane then gathers the weights of its 32
// positions from the slots that the scatter above would have written to.  Spans are 2048 consecutive flat elements,
// dealt to the waves of the launch in turn.  A lane's 64 output bytes go through LDS once more (rows 80 bytes apart),
// so that a store instruction writes 1 KB of consecutive bytes.
// ---------------------------------------------------------------------------------------------------------------
template <int B>
__device__ __forceinline__ void d5_dequant(const uint32_t (&w)[B], uint32_t *dst, uint32_t e, float scale, float minus_t_scale) {
#pragma unroll
    for (int g = 0; g < 8; ++g) {
        if (e > 4u * g) {
            asm volatile("");
#pragma unroll
            for (int t = 2 * g; t < 2 * g + 2; ++t) {
                const uint32_t c0 = d5_code<B>(w, 2 * t), c1 = d5_code<B>(w, 2 * t + 1);
                dst[t] = d5_pack(__fmaf_rn((float)c0, scale, minus_t_scale), __fmaf_rn((float)c1, scale, minus_t_scale));
            }
        }
    }
}

// TILE: the product with 2..16 activation rows on the matrix pipe instead of the store (ixh_dense_tiles.h): 16 waves
// to a workgroup, wave w on row 16 rb + w of every step (row block rb, span k of the row) of the workgroup's share.
struct D5TileArgs {
    uint32_t n_chunks, spans_per_row, total_steps, n_pieces;
    const uint16_t *x;
    int m;
    int64_t ldx;
    float *ws;
};
constexpr uint32_t kD5Region = kD5Slots * 2 + 16;  // bytes between the waves' arrays in the tile kernel
constexpr size_t kD5TileLds = kD5LutBytes + (size_t)kDtWaves * kD5Region + (size_t)kDtWaves * 3 * kD5BmWords * 4 + kDtSumsBytes;

template <bool TILE>
__global__ void __launch_bounds__(kWave *(TILE ? kDtWaves : kD5Waves))
k_decode34568_dense(Dev P, const int32_t *__restrict__ prefix, uint32_t n_units, uint32_t n_spans, uint16_t *__restrict__ out,
                    D5TileArgs ta) {
    constexpr int kWaves = TILE ? kDtWaves : kD5Waves;
    extern __shared__ __attribute__((aligned(16))) uint8_t d5_smem[];  // the tile kernel's (more than a static array may hold)
    __shared__ __attribute__((aligned(16))) uint32_t lut_s[TILE ? 4 : kD5LutBytes / 4];
    __shared__ __attribute__((aligned(16))) uint16_t wc_s[TILE ? 1 : kD5Waves][TILE ? 8 : kD5Slots];
    __shared__ uint32_t bm_s[TILE ? 1 : kD5Waves][3][TILE ? 1 : kD5BmWords];
    static_assert(kD5Slots * 2 >= 64 * 80 && (kD5Slots * 2) % 16 == 0, "a wave's slots are re-used as 64 rows of 80 bytes");
    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    uint32_t *const lut = TILE ? reinterpret_cast<uint32_t *>(d5_smem) : lut_s;
    uint16_t *const wc = TILE ? reinterpret_cast<uint16_t *>(d5_smem + kD5LutBytes + wave * kD5Region) : wc_s[TILE ? 0 : wave];
    uint32_t(*const bmw)[kD5BmWords] =
        TILE ? reinterpret_cast<uint32_t(*)[kD5BmWords]>(d5_smem + kD5LutBytes + (size_t)kDtWaves * kD5Region) + wave * 3
             : reinterpret_cast<uint32_t(*)[kD5BmWords]>(&bm_s[TILE ? 0 : wave][0][0]);
    const float scale = bf16_bits_to_f32(*P.scale);
    const float m7 = -7.0f * scale, m15 = -15.0f * scale, m31 = -31.0f * scale, m127 = -127.0f * scale;  // exact
    for (uint32_t e = tid; e < 64 * 32; e += kWave * kWaves) {
        const uint32_t idx = e >> 5;
        lut[e] = d5_pack(dequant((int)(idx & 7u) - 3, scale), dequant((int)(idx >> 3) - 3, scale));
    }
    // Positions past the tensor's (or the row's) end walk on through the arrays; what they read is not stored (or meets
    // activations that are zero) but must be there to read, and finite: start from zeros.
    for (uint32_t j = lane; j < kD5Slots / 8; j += kWave) reinterpret_cast<e_u32x4 *>(wc)[j] = e_u32x4{0, 0, 0, 0};
    __syncthreads();

    uint32_t *const wc32 = reinterpret_cast<uint32_t *>(wc);
    const uint32_t lut_lane = (lane & 31u) << 2;
    const uint32_t entries = n_units + 1;
    const uint32_t *__restrict__ b1 = P.bm[0];
    const __amdgpu_buffer_rsrc_t st_rsrc[4] = {
        __builtin_amdgcn_make_buffer_rsrc((void *)P.st[0], 0, (int)(P.st_words[0] * 4u), 0x00020000),
        __builtin_amdgcn_make_buffer_rsrc((void *)P.st[1], 0, (int)(P.st_words[1] * 4u), 0x00020000),
        __builtin_amdgcn_make_buffer_rsrc((void *)P.st[2], 0, (int)(P.st_words[2] * 4u), 0x00020000),
        __builtin_amdgcn_make_buffer_rsrc((void *)P.st[3], 0, (int)(P.st_words[3] * 4u), 0x00020000)};
    const __amdgpu_buffer_rsrc_t last_rsrc =
        __builtin_amdgcn_make_buffer_rsrc((void *)P.last, 0, (int)((P.last_bytes + 3u) & ~3u), 0x00020000);
    const __amdgpu_buffer_rsrc_t bm_rsrc[3] = {
        __builtin_amdgcn_make_buffer_rsrc((void *)P.bm[1], 0, (int)(P.bm_words[1] * 4u), 0x00020000),
        __builtin_amdgcn_make_buffer_rsrc((void *)P.bm[2], 0, (int)(P.bm_words[2] * 4u), 0x00020000),
        __builtin_amdgcn_make_buffer_rsrc((void *)P.bm[3], 0, (int)(P.bm_words[3] * 4u), 0x00020000)};

    // What a span needs from memory before any arithmetic: its table entries (scalars), the lane's word of the first
    // bitmap, the span's part of the nested bitmaps and the lane's window of every code stream.  They are asked for one
    // span ahead (the table entries two), so that a wave's chain table -> windows -> arithmetic waits for memory once.
    struct Ranks { uint32_t qa[4], qb[4]; };
    struct Shape { uint32_t p0, n_el, e[5], base[5], g1, g2, g3, at_last; };
    struct Loads { uint32_t w1, bm[3], bmx[3], d1[4], d2[5], d3[6], d4[7], d5[9]; };
    // table units [u0, u1) of span (or step) sp: four of the flat tensor, or up to four of the wave's row
    auto units_of = [&](uint32_t sp, uint32_t &u0, uint32_t &u1) {
        if (TILE) {
            const uint32_t rb = sp / ta.spans_per_row, k = sp - rb * ta.spans_per_row;
            const uint32_t row = min(rb * (uint32_t)kDtWaves + wave, P.out_f - 1u);  // a wave past the last row: it again
            u0 = row * ta.n_chunks + 4 * k;
            u1 = u0 + min(4u, ta.n_chunks - 4 * k);
        } else {
            u0 = 4 * sp;
            u1 = min(u0 + 4, n_units);
        }
    };
    auto table_of = [&](uint32_t sp) {
        Ranks q;
        uint32_t u0, u1;
        units_of(sp, u0, u1);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            q.qa[i] = (uint32_t)prefix[(size_t)i * entries + u0];
            q.qb[i] = (uint32_t)prefix[(size_t)i * entries + u1];
        }
        return q;
    };
    auto shape_of = [&](uint32_t sp, const Ranks &q) {
        Shape g;
        uint32_t u0, u1;
        units_of(sp, u0, u1);
        g.p0 = u0 * kFastChunk;
        g.n_el = min((u1 - u0) * kFastChunk, P.n - g.p0);
        uint32_t rest = g.n_el, at = 0;
#pragma unroll
        for (int i = 0; i < 5; ++i) {
            const uint32_t cnt = i < 4 ? q.qb[i < 4 ? i : 0] - q.qa[i < 4 ? i : 0] : rest;
            rest -= i < 4 ? cnt : 0u;
            g.e[i] = 4 * ((cnt + 255) / 256);
            g.base[i] = at;
            at += 64 * g.e[i];
        }
        g.g1 = g.p0 - q.qa[0]; g.g2 = g.g1 - q.qa[1]; g.g3 = g.g2 - q.qa[2]; g.at_last = g.g3 - q.qa[3];
        return g;
    };
    auto fetch = [&](const Shape &g, const Ranks &q) {
        Loads r;
        const uint32_t n_here = 32 * lane < g.n_el ? min(32u, g.n_el - 32 * lane) : 0u;
        r.w1 = n_here ? b1[(g.p0 >> 5) + lane] & d5_low_mask(n_here) : 0u;
        const uint32_t gs[3] = {g.g1, g.g2, g.g3};
#pragma unroll
        for (int j = 0; j < 3; ++j) {
            const uint32_t w0 = gs[j] >> 5;
            r.bm[j] = __builtin_amdgcn_raw_buffer_load_b32(bm_rsrc[j], (int)((w0 + lane) * 4u), 0, 0);
            r.bmx[j] = lane < 4 ? __builtin_amdgcn_raw_buffer_load_b32(bm_rsrc[j], (int)((w0 + 64u + lane) * 4u), 0, 0) : 0u;
        }
        d5_fetch<3>(st_rsrc[0], (uint64_t)(q.qa[0] + lane * g.e[0]) * 3u, r.d1);
        d5_fetch<4>(st_rsrc[1], (uint64_t)(q.qa[1] + lane * g.e[1]) * 4u, r.d2);
        d5_fetch<5>(st_rsrc[2], (uint64_t)(q.qa[2] + lane * g.e[2]) * 5u, r.d3);
        d5_fetch<6>(st_rsrc[3], (uint64_t)(q.qa[3] + lane * g.e[3]) * 6u, r.d4);
        d5_fetch<8>(last_rsrc, (uint64_t)(g.at_last + lane * g.e[4]) * 8u, r.d5);
        return r;
    };

    // flat spans dealt to the waves of the launch in turn, or (TILE) the workgroup's contiguous share of the steps,
    // every wave of it on its own row
    const uint32_t stride = TILE ? 1u : gridDim.x * kD5Waves;
    const uint32_t sp_end = TILE ? (uint32_t)(((uint64_t)blockIdx.x + 1u) * ta.total_steps / gridDim.x) : n_spans;
    uint32_t sp = TILE ? (uint32_t)((uint64_t)blockIdx.x * ta.total_steps / gridDim.x) : blockIdx.x * kD5Waves + wave;
    if (sp >= sp_end) return;
    DtMfmaSink<kD5Region> sink;
    if (TILE) {
        sink.x = ta.x; sink.ldx = ta.ldx; sink.m = ta.m; sink.ws = ta.ws;
        sink.out_f = P.out_f; sink.in_f = P.in_f; sink.spans_per_row = ta.spans_per_row; sink.n_pieces = ta.n_pieces;
        sink.total_steps = ta.total_steps; sink.step_end = sp_end;
        sink.wave = wave; sink.lane = lane; sink.wc = wc;
        sink.tile_addr = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t *)(d5_smem + kD5LutBytes);
        sink.red = reinterpret_cast<float *>(d5_smem + kD5TileLds - kDtSumsBytes);
        sink.acc = dt_f32x4{0.f, 0.f, 0.f, 0.f};
    }
    // past the end the last span is fetched once more: loads that nobody uses
    auto next_of = [&](uint32_t s) { return s + stride < sp_end ? s + stride : s; };
    Ranks q_now = table_of(sp);
    Shape g_now = shape_of(sp, q_now);
    Loads in_now = fetch(g_now, q_now);
    uint32_t sp_next = next_of(sp);
    Ranks q_next = table_of(sp_next);
    for (uint32_t turn = wave;; ++turn) {
        if (!TILE) {  // the waves that share a SIMD take turns at the issue priority, one span each (not where they
                      // meet at a barrier every span)
            const uint32_t pr = turn % 3u;  // s_setprio takes an immediate
            if (pr == 0) __builtin_amdgcn_s_setprio(0);
            else if (pr == 1) __builtin_amdgcn_s_setprio(1);
            else __builtin_amdgcn_s_setprio(2);
        }
        const Shape g_next = shape_of(sp_next, q_next);
        const Loads in_next = fetch(g_next, q_next);
        const uint32_t sp_after = next_of(sp_next);
        const Ranks q_after = table_of(sp_after);
        const DtStep step{sp / (TILE ? ta.spans_per_row : 1u), sp % (TILE ? ta.spans_per_row : 1u), sp};
        if (TILE) sink.begin(step);

        const uint32_t p0 = g_now.p0, n_el = g_now.n_el;
        const uint32_t(&qa)[4] = q_now.qa;
        const uint32_t(&e)[5] = g_now.e;
        const uint32_t(&base)[5] = g_now.base;
        const uint32_t g1 = g_now.g1, g2 = g_now.g2, g3 = g_now.g3, at_last = g_now.at_last;

        // positions of this lane inside the span, and its bitmap word
        const uint32_t n_here = 32 * lane < n_el ? min(32u, n_el - 32 * lane) : 0u;
        const uint32_t w1 = in_now.w1;
#pragma unroll
        for (int j = 0; j < 3; ++j) {
            bmw[j][lane] = in_now.bm[j];
            if (lane < 4) bmw[j][64 + lane] = in_now.bmx[j];
        }
        uint32_t c1w[3], c2w[4], c3w[5], c4w[6], c5w[8];
        d5_align<3>(in_now.d1, (uint64_t)(qa[0] + lane * e[0]) * 3u, c1w);
        d5_align<4>(in_now.d2, (uint64_t)(qa[1] + lane * e[1]) * 4u, c2w);
        d5_align<5>(in_now.d3, (uint64_t)(qa[2] + lane * e[2]) * 5u, c3w);
        d5_align<6>(in_now.d4, (uint64_t)(qa[3] + lane * e[3]) * 6u, c4w);
        d5_align<8>(in_now.d5, (uint64_t)(at_last + lane * e[4]) * 8u, c5w);

        // ---- dequantise every level where its codes lie ----
        {
            uint32_t *dst = wc32 + (lane * e[0]) / 2;
#pragma unroll
            for (int g = 0; g < 8; ++g) {
                if (e[0] > 4u * g) {
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
                        dst[t] = lut[((a & 0x1F80u) | lut_lane) >> 2];
                    }
                }
            }
        }
        d5_dequant<4>(c2w, wc32 + (base[1] + lane * e[1]) / 2, e[1], scale, m7);
        d5_dequant<5>(c3w, wc32 + (base[2] + lane * e[2]) / 2, e[2], scale, m15);
        d5_dequant<6>(c4w, wc32 + (base[3] + lane * e[3]) / 2, e[3], scale, m31);
        d5_dequant<8>(c5w, wc32 + (base[4] + lane * e[4]) / 2, e[4], scale, m127);

        // ---- ranks: first slot of this lane in each array ----
        auto window = [&](int j, uint32_t g, uint32_t first, uint32_t alive) {
            const uint32_t o = (g & 31u) + first;
            const uint32_t lo = bmw[j][o >> 5], hi = bmw[j][(o >> 5) + 1];
            return __builtin_amdgcn_alignbit(hi, lo, o & 31u) & d5_low_mask(alive);
        };
        const uint32_t cnt1 = (uint32_t)__popc(w1);
        const uint32_t alive1 = n_here - cnt1;
        const uint32_t sc1 = wave_scan_inclusive(cnt1 | (alive1 << 16));
        const uint32_t first1 = (sc1 & 0xffffu) - cnt1, first_a1 = (sc1 >> 16) - alive1;
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
        const uint32_t bits2 = window(0, g1, first_a1, alive1);
        const uint32_t cnt2 = (uint32_t)__popc(bits2), alive2 = alive1 - cnt2;
        const uint32_t sc2 = wave_scan_inclusive(cnt2 | (alive2 << 16));
        const uint32_t first2 = (sc2 & 0xffffu) - cnt2, first_a2 = (sc2 >> 16) - alive2;
        const uint32_t bits3 = window(1, g2, first_a2, alive2);
        const uint32_t cnt3 = (uint32_t)__popc(bits3), alive3 = alive2 - cnt3;
        const uint32_t sc3 = wave_scan_inclusive(cnt3 | (alive3 << 16));
        const uint32_t first3 = (sc3 & 0xffffu) - cnt3, first_a3 = (sc3 >> 16) - alive3;
        const uint32_t bits4 = window(2, g3, first_a3, alive3);
        const uint32_t cnt4 = (uint32_t)__popc(bits4);
        const uint32_t first4 = wave_scan_inclusive(cnt4) - cnt4;
        const uint32_t first5 = first_a3 - first4;

        // ---- gather the lane's 32 weights from their levels' arrays: the walk of the product kernel's scatter ----
        uint32_t o[16];
        {
            const uint32_t wc_half = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint16_t *)wc >> 1;
            const uint32_t low1 = (uint32_t)__popc(w1 & 0xffffu);
            const uint32_t low_a1 = min(n_here, 16u) - low1;
            const uint32_t low2 = (uint32_t)__popc(bits2 & d5_low_mask(low_a1)), low_a2 = low_a1 - low2;
            const uint32_t low3 = (uint32_t)__popc(bits3 & d5_low_mask(low_a2)), low_a3 = low_a2 - low3;
            const uint32_t low4 = (uint32_t)__popc(bits4 & d5_low_mask(low_a3)), low5 = low_a3 - low4;
            const uint32_t a1 = wc_half + base[0] + first1, a2 = wc_half + base[1] + first2, a3 = wc_half + base[2] + first3;
            const uint32_t a4 = wc_half + base[3] + first4, a5 = wc_half + base[4] + first5;
            e_u16x2 s1 = __builtin_bit_cast(e_u16x2, a1 | ((a1 + low1) << 16));
            e_u16x2 s2 = __builtin_bit_cast(e_u16x2, a2 | ((a2 + low2) << 16));
            e_u16x2 s3 = __builtin_bit_cast(e_u16x2, a3 | ((a3 + low3) << 16));
            e_u16x2 s4 = __builtin_bit_cast(e_u16x2, a4 | ((a4 + low4) << 16));
            e_u16x2 s5 = __builtin_bit_cast(e_u16x2, a5 | ((a5 + low5) << 16));
            const e_u16x2 f2 = __builtin_bit_cast(e_u16x2, (bits2 & 0xffffu) | ((uint32_t)((uint64_t)bits2 >> low_a1) << 16));
            const e_u16x2 f3 = __builtin_bit_cast(e_u16x2, (bits3 & 0xffffu) | ((uint32_t)((uint64_t)bits3 >> low_a2) << 16));
            const e_u16x2 f4 = __builtin_bit_cast(e_u16x2, (bits4 & 0xffffu) | ((uint32_t)((uint64_t)bits4 >> low_a3) << 16));
            e_u16x2 ja = {0, 0}, jb = {0, 0}, jc = {0, 0};
            const e_u16x2 one = {1, 1};
#pragma unroll
            for (int t = 0; t < 16; ++t) {
                const e_u16x2 in1 = __builtin_bit_cast(e_u16x2, (w1 >> t) & 0x00010001u);
                const e_u16x2 out1 = in1 ^ one;
                const e_u16x2 in2 = (f2 >> ja) & out1;
                const e_u16x2 out2 = out1 ^ in2;
                const e_u16x2 in3 = (f3 >> jb) & out2;
                const e_u16x2 out3 = out2 ^ in3;
                const e_u16x2 in4 = (f4 >> jc) & out3;
                const e_u16x2 in5 = out3 ^ in4;
                const e_u16x2 at = in1 * (s1 - s5) + (in2 * (s2 - s5) + (in3 * (s3 - s5) + (in4 * (s4 - s5) + s5)));
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
                s1 += in1; s2 += in2; s3 += in3; s4 += in4; s5 += in5;
                ja += out1; jb += out2; jc += out3;
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();

        // ---- the lane's 64 bytes to their place in the output (or to the tile, and the matrix pipe) ----
        uint16_t *dst = out + (size_t)p0 + 32 * lane;
        if (TILE) {
            sink.end(step, o);
        } else if (n_el == kD5Span) {
            e_u32x4 *const rows = reinterpret_cast<e_u32x4 *>(wc);
#pragma unroll
            for (int j = 0; j < 4; ++j) rows[lane * 5 + j] = e_u32x4{o[4 * j], o[4 * j + 1], o[4 * j + 2], o[4 * j + 3]};
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
            __builtin_amdgcn_wave_barrier();
            e_u32x4 *const line = reinterpret_cast<e_u32x4 *>(out + (size_t)p0);
#pragma unroll
            for (int j = 0; j < 4; ++j) line[64 * j + lane] = rows[(16 * j + (lane >> 2)) * 5 + (lane & 3u)];
        } else if (n_here == 32) {
#pragma unroll
            for (int j = 0; j < 4; ++j)
                reinterpret_cast<e_u32x4 *>(dst)[j] = e_u32x4{o[4 * j], o[4 * j + 1], o[4 * j + 2], o[4 * j + 3]};
        } else {
            for (uint32_t t = 0; t < n_here; ++t) {
                uint32_t v = 0;
#pragma unroll
                for (int j = 0; j < 16; ++j) v = (t >> 1) == (uint32_t)j ? o[j] : v;  // o[j]: positions 2j and 2j + 1
                dst[t] = (uint16_t)((t & 1u) ? v >> 16 : v);
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
        if (sp + stride >= sp_end) break;
        sp = sp_next;
        q_now = q_next;
        g_now = g_next;
        in_now = in_next;
        sp_next = sp_after;
        q_next = q_after;
    }
}

bool decode_dense34568_supports(const Dev &P, uint32_t chunk, const int8_t *o8, const uint16_t *o16) {
    return P.n_levels == 5 && P.bits[0] == 3 && P.bits[1] == 4 && P.bits[2] == 5 && P.bits[3] == 6 && P.bits[4] == 8 &&
           chunk == kFastChunk && !o8 && o16 && ((uintptr_t)o16 & 15u) == 0 && ((uintptr_t)P.last & 3u) == 0 && P.n != 0;
}

int launch_decode_dense34568(const Dev &P, const int32_t *prefix, uint16_t *o16, hipStream_t s) {
    const uint32_t n_units = (P.n + kFastChunk - 1) / kFastChunk;
    const uint32_t n_spans = (n_units + 3) / 4;
    static const uint32_t resident = [] {
        int dev = 0, n_cu = 256, per_cu = 0;
        if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev);
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, k_decode34568_dense<false>, kWave * kD5Waves, 0) != hipSuccess || per_cu < 1)
            per_cu = 3;
        return (uint32_t)n_cu * (uint32_t)per_cu;
    }();
    const uint32_t blocks = min(resident, (n_spans + kD5Waves - 1) / kD5Waves);
    hipLaunchKernelGGL(k_decode34568_dense<false>, dim3(blocks), dim3(kWave * kD5Waves), 0, s, P, prefix, n_units, n_spans, o16,
                       D5TileArgs{0, 0, 0, 0, nullptr, 0, 0, nullptr});
    return hipGetLastError() == hipSuccess ? IXH_OK : IXH_ELAUNCH;
}

// 2..16 activation rows on dense five-level mixes: the decoder above in its tile mode
bool gemv_dense34568_tiles_supports(const Dev &P, uint32_t chunk, int m, const uint16_t *x, int64_t ldx) {
    return P.n_levels == 5 && P.bits[0] == 3 && P.bits[1] == 4 && P.bits[2] == 5 && P.bits[3] == 6 && P.bits[4] == 8 &&
           chunk == kFastChunk && m >= 2 && m <= 16 && P.in_f % kFastChunk == 0 && P.in_f >= 2 * kFastChunk &&
           ((uintptr_t)x & 15u) == 0 && (ldx & 7) == 0 && ((uintptr_t)P.last & 3u) == 0 && P.out_f != 0 &&
           (uint64_t)P.out_f * P.in_f == P.n;
}

int launch_gemv_dense34568_tiles(const Dev &P, const int32_t *prefix, const uint16_t *x, int m, int64_t ldx, uint16_t *y,
                                 int64_t ldy, float *ws, hipStream_t s) {
    static const bool raised = hipFuncSetAttribute(reinterpret_cast<const void *>(k_decode34568_dense<true>),
                                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)kD5TileLds) == hipSuccess;
    if (!raised) return IXH_EUNSUPPORTED;
    static const uint32_t n_cu = [] {
        int dev = 0, v = 256;
        if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev);
        return (uint32_t)v;
    }();
    const DtPlan plan = dt_plan(P.out_f, P.in_f, n_cu);
    if (plan.groups == 0) return IXH_EUNSUPPORTED;
    const uint32_t n_units = P.out_f * plan.n_chunks;
    hipLaunchKernelGGL(k_decode34568_dense<true>, dim3(plan.groups), dim3(kWave * kDtWaves), kD5TileLds, s, P, prefix, n_units,
                       0u, (uint16_t *)nullptr,
                       D5TileArgs{plan.n_chunks, plan.spans_per_row, plan.total_steps, plan.n_pieces, x, m, ldx, ws});
    if (hipGetLastError() != hipSuccess) return IXH_ELAUNCH;
    return launch_reduce_chunks(ws, plan.n_pieces, m, P.out_f, y, ldy, s);
}

bool gemv_dense34568_supports(const Dev &P, uint32_t chunk, int m, const uint16_t *x) {
    return P.n_levels == 5 && P.bits[0] == 3 && P.bits[1] == 4 && P.bits[2] == 5 && P.bits[3] == 6 && P.bits[4] == 8 &&
           chunk == kFastChunk && m == 1 && P.in_f % kFastChunk == 0 && P.in_f != 0 && ((uintptr_t)x & 15u) == 0 &&
           ((uintptr_t)P.last & 3u) == 0;
}

int launch_gemv_dense34568(const Dev &P, const int32_t *prefix, const uint16_t *x, uint16_t *y, float *y32, float *ws,
                           bool atomic, hipStream_t s) {
    const uint32_t n_chunks = P.in_f / kFastChunk;
    const uint32_t spans_per_row = (n_chunks + 3) / 4;
    const uint32_t n_spans = P.out_f * spans_per_row;
    if (n_spans == 0) return IXH_OK;
    // one resident set of workgroups; each wave walks its items with the stride of the launch
    static const uint32_t resident = [] {
        int dev = 0, n_cu = 256, per_cu = 0;
        if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev);
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, k_gemv34568_dense, kWave * kD5Waves, 0) != hipSuccess || per_cu < 1)
            per_cu = 3;
        return (uint32_t)n_cu * (uint32_t)per_cu;
    }();
    // Whole rows per wave when they spread over the resident waves within 12 %: one launch, no workspace, each
    // output summed in one register.  Otherwise spans are dealt out and a second kernel adds a row's partial sums.
    const uint32_t waves_res = resident * kD5Waves;
    const uint32_t rounds = (P.out_f + waves_res - 1) / waves_res;
    const bool by_rows = spans_per_row == 1 || (uint64_t)rounds * waves_res * 100u <= (uint64_t)P.out_f * 112u;
    const uint32_t n_items = by_rows ? P.out_f : n_spans;
    const uint32_t blocks = min(resident, (n_items + kD5Waves - 1) / kD5Waves);
    const int out_mode = atomic ? kD5Atomic : (by_rows ? kD5Direct : kD5Workspace);
    hipLaunchKernelGGL(k_gemv34568_dense, dim3(blocks), dim3(kWave * kD5Waves), 0, s, P, prefix, n_chunks, spans_per_row,
                       n_spans, x, y, y32, ws, out_mode, by_rows);
    if (hipGetLastError() != hipSuccess) return IXH_ELAUNCH;
    if (out_mode == kD5Workspace) return launch_reduce_chunks(ws, spans_per_row, 1, P.out_f, y, P.out_f, s);
    return IXH_OK;
}

}  // namespace ixh
