/*
 * CPU oracle for the INT8-X hot path.  TEST INFRASTRUCTURE ONLY: nothing in the
 * shipped package links, loads or calls this file; it exists so that tests,
 * the smoke check and the CPU-baseline leg of the benchmark have something
 * independent to compare the gfx950 kernels with.
 *
 * Every function restates, as plain sequential C, what one piece of the
 * reference (dfytensor/ixrun, Python + Triton) computes.  The restatement is
 * written from the reference's definitions, element by element, and shares no
 * code or tables with the HIP kernels or with the package's torch encoder.
 *
 *   ixo_pack_bits / ixo_unpack_bits   ixrun/bitpack.py:13-61, :64-84
 *   ixo_quantize_bf16                 ixrun/quantize.py:64-73
 *   ixo_encode                        ixrun/quantize.py:25-37, :76-108
 *   ixo_decode_i8                     ixrun/quantize.py:126-183,
 *                                     ixrun/triton_kernels.py:36-59 (per-level
 *                                     positions + scatter), written here as the
 *                                     equivalent single forward walk
 *   ixo_dequant_bf16                  ixrun/triton_kernels.py:59, :168-177
 *   ixo_prefix                        ixrun/fused.py:35-78 (row / chunk
 *                                     prefixes), ixrun/triton_kernels.py:180-220
 *                                     (block offsets)
 *   ixo_gemm_f64, ixo_gemm_f32        ixrun/fused.py:84-179 (what the fused
 *                                     kernel sums), ixrun/engine.py:171-173
 *                                     (decode then F.linear for M > 1)
 *
 *   ixo_gs_quantize                   ixgs/quantize.py:49-63 (per-group fp16
 *                                     scale = group max / 15, values clamped to
 *                                     [-127, 128])
 *   ixo_gs_encode                     ixgs/quantize.py:65-91 (tiers by value
 *                                     range: [-3,4], [-15,16], rest)
 *   ixo_gs_decode_i16                 ixgs/quantize.py:113-147, ixgs/kernels.py:46-99
 *   ixo_gs_dequant_bf16               ixgs/quantize.py:149-150, ixgs/kernels.py:102-104
 *
 * Pinning (what each function is checked against, see tests/test_oracle.py):
 *   bit packing   closed form word[j] = sum code_i << (i*b - 32j); the known
 *                 answer pack([0..7], 3) = 0x00FAC688; round trips on the sizes
 *                 of the reference's tests/test_core.py:15-35
 *   quantize      the reference tests' own ground truth "plain int8 dequant"
 *                 (tests/test_core.py:38-64, tests/test_int8_equivalence.py:29-33)
 *   encode/decode hand-derived known answer (2x5 tensor, all three levels),
 *                 counts partition N, byte accounting formula, brute-force
 *                 rank by linear scan on tiny inputs, round trip to the int8
 *   prefix        brute-force running counts; known answer q1=[0,3], q2=[0,2]
 *   gemm          one-hot x gives a decoded column exactly; ones give row sums
 *   group scale   fp16 conversion against numpy's float16 (every bit pattern, and
 *                 fp32 values on and next to every rounding boundary); the reference
 *                 test's own property (ixgs/test_gs.py:38-52): decode equals
 *                 bf16(round(w / s) * s) with s the fp16-rounded scale, on its
 *                 heavy-tailed recipe; a hand-derived known answer; round trip
 * Parity unpinned: the M > 1 path of the reference ends in an external BLAS
 * whose summation order is not fixed by any reference test; ixo_gemm_f64 is the
 * build's own yardstick there.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ---- bf16 <-> f32 (round to nearest even, as torch's .bfloat16()) ---- */
static inline float bf16_to_f32(uint16_t h) {
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

static inline uint16_t f32_to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40u); /* NaN */
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

uint16_t ixo_f32_to_bf16(float f) { return f32_to_bf16(f); }
float ixo_bf16_to_f32(uint16_t h) { return bf16_to_f32(h); }

static inline int threshold_of(int bits) { return (1 << (bits - 1)) - 1; } /* config.py:27-36 */

/* ---- bit streams: code i occupies string bits [i*b, i*b+b), LSB first ---- */
void ixo_pack_bits(const uint32_t *codes, int64_t n, int bits, uint32_t *words) {
    int64_t nw = (n * bits + 31) / 32;
    memset(words, 0, (size_t)nw * 4);
    for (int64_t i = 0; i < n; ++i) {
        uint64_t c = codes[i] & (bits >= 32 ? 0xFFFFFFFFull : ((1ull << bits) - 1));
        int64_t pos = i * bits;
        int64_t j = pos >> 5;
        int s = (int)(pos & 31);
        uint64_t placed = c << s;
        words[j] |= (uint32_t)placed;
        if (s + bits > 32) words[j + 1] |= (uint32_t)(placed >> 32);
    }
}

static inline uint32_t read_code(const uint32_t *words, int64_t idx, int bits) {
    int64_t pos = idx * bits;
    int64_t j = pos >> 5;
    int s = (int)(pos & 31);
    uint64_t lo = words[j];
    uint64_t hi = (s + bits > 32) ? words[j + 1] : 0;
    return (uint32_t)(((lo | (hi << 32)) >> s) & ((1ull << bits) - 1));
}

void ixo_unpack_bits(const uint32_t *words, int64_t n, int bits, uint32_t *codes) {
    for (int64_t i = 0; i < n; ++i) codes[i] = read_code(words, i, bits);
}

/* ---- per-tensor int8 of a bf16 weight -------------------------------- */
/* scale = bf16( max|w| clamped below at bf16(1e-8), divided by 127 in fp32 );
 * q = clamp(rint(f32(w) / f32(scale)), -127, 127).  The division by the
 * already-rounded bf16 scale and the half-to-even rounding are the reference's
 * (quantize.py:64-67 with a bf16 weight). */
void ixo_quantize_bf16(const uint16_t *w, int64_t n, uint16_t *scale_out, int8_t *q) {
    float amax = 0.0f;
    for (int64_t i = 0; i < n; ++i) {
        float a = fabsf(bf16_to_f32(w[i]));
        if (a > amax) amax = a;
    }
    float floor_ = bf16_to_f32(f32_to_bf16(1e-8f));
    if (amax < floor_) amax = floor_;
    uint16_t sb = f32_to_bf16(amax / 127.0f);
    float s = bf16_to_f32(sb);
    for (int64_t i = 0; i < n; ++i) {
        float r = rintf(bf16_to_f32(w[i]) / s); /* default rounding mode: half to even */
        if (r > 127.0f) r = 127.0f;
        if (r < -127.0f) r = -127.0f;
        q[i] = (int8_t)r;
    }
    *scale_out = sb;
}

/* level of a value: first i with |v| <= T(level_bits[i]); last level takes the rest */
static inline int level_of(int v, const int *level_bits, int n_levels) {
    int a = v < 0 ? -v : v;
    for (int i = 0; i < n_levels - 1; ++i)
        if (a <= threshold_of(level_bits[i])) return i;
    return n_levels - 1;
}

void ixo_count_levels(const int8_t *q, int64_t n, const int *level_bits, int n_levels, int64_t *counts) {
    for (int i = 0; i < n_levels; ++i) counts[i] = 0;
    for (int64_t p = 0; p < n; ++p) counts[level_of(q[p], level_bits, n_levels)]++;
}

/* Encode.  bitmaps[i] needs ceil(remaining_i/32) words where remaining_0 = n and
 * remaining_{i+1} = remaining_i - counts[i]; streams[i] needs
 * ceil(counts[i]*b_i/32) words; last needs counts[L-1] bytes.  Buffers must be
 * zero-filled by the caller.  Returns total_bytes (quantize.py:99-108). */
int64_t ixo_encode(const int8_t *q, int64_t n, const int *level_bits, int n_levels,
                   uint32_t **bitmaps, uint32_t **streams, uint8_t *last, const int64_t *counts) {
    int64_t bm_cur[8] = {0}, st_cur[8] = {0};
    for (int64_t p = 0; p < n; ++p) {
        int v = q[p];
        int lv = level_of(v, level_bits, n_levels);
        for (int i = 0; i < lv && i < n_levels - 1; ++i) bm_cur[i]++; /* a 0 bit in every lower bitmap */
        if (lv < n_levels - 1) {
            int64_t b = bm_cur[lv]++;
            bitmaps[lv][b >> 5] |= 1u << (b & 31);
            uint64_t code = (uint64_t)(v + threshold_of(level_bits[lv]));
            int bits = level_bits[lv];
            int64_t pos = st_cur[lv]++ * bits;
            int s = (int)(pos & 31);
            uint64_t placed = code << s;
            streams[lv][pos >> 5] |= (uint32_t)placed;
            if (s + bits > 32) streams[lv][(pos >> 5) + 1] |= (uint32_t)(placed >> 32);
        } else {
            last[st_cur[lv]++] = (uint8_t)(v + 127);
        }
    }
    int64_t total = 2 + counts[n_levels - 1];
    int64_t remaining = n;
    for (int i = 0; i < n_levels - 1; ++i) {
        total += 4 * ((counts[i] * level_bits[i] + 31) / 32);
        total += 4 * ((remaining + 31) / 32);
        remaining -= counts[i];
    }
    return total;
}

/* Decode by one forward walk: element p asks bitmap 0, then (if not taken)
 * bitmap 1 at the next unread bit, and so on; the taking level hands out its
 * next unread code.  This is the nested-bitmap definition itself and equals the
 * reference's "positions per level, then scatter" decoder. */
void ixo_decode_i8(int64_t n, const int *level_bits, int n_levels, uint32_t *const *bitmaps,
                   uint32_t *const *streams, const uint8_t *last, int8_t *q) {
    int64_t bm_cur[8] = {0}, st_cur[8] = {0};
    for (int64_t p = 0; p < n; ++p) {
        int lv = n_levels - 1;
        for (int i = 0; i < n_levels - 1; ++i) {
            int64_t b = bm_cur[i]++;
            if ((bitmaps[i][b >> 5] >> (b & 31)) & 1u) { lv = i; break; }
        }
        int v;
        if (lv < n_levels - 1)
            v = (int)read_code(streams[lv], st_cur[lv]++, level_bits[lv]) - threshold_of(level_bits[lv]);
        else
            v = (int)last[st_cur[lv]++] - 127;
        q[p] = (int8_t)v;
    }
}

/* w = bf16( f32(v) * f32(scale) ) */
void ixo_dequant_bf16(const int8_t *q, int64_t n, uint16_t scale, uint16_t *w) {
    float s = bf16_to_f32(scale);
    for (int64_t i = 0; i < n; ++i) w[i] = f32_to_bf16((float)q[i] * s);
}

/* Exclusive level counts at every flat position u*chunk, u = 0..ceil(n/chunk):
 * prefix[i*(n_units+1) + u] = number of level-i elements with flat index <
 * min(u*chunk, n), for i < n_levels-1.  chunk = in_f gives the per-row table of
 * compute_row_prefixes, a divisor of in_f its per-(row,chunk) table, 1024 the
 * block offsets of precompute_block_offsets. */
void ixo_prefix(int64_t n, int n_levels, uint32_t *const *bitmaps, int64_t chunk, int32_t *prefix) {
    int64_t n_units = (n + chunk - 1) / chunk;
    int64_t bm_cur[8] = {0}, cnt[8] = {0};
    for (int64_t p = 0; p <= n; ++p) {
        if (p % chunk == 0 || p == n) {
            int64_t u = (p == n) ? n_units : p / chunk;
            for (int i = 0; i < n_levels - 1; ++i) prefix[i * (n_units + 1) + u] = (int32_t)cnt[i];
            if (p == n) break;
        }
        for (int i = 0; i < n_levels - 1; ++i) {
            int64_t b = bm_cur[i]++;
            if ((bitmaps[i][b >> 5] >> (b & 31)) & 1u) { cnt[i]++; break; }
        }
    }
}

/* y[m][r] = sum_k f64(x[m][k]) * f64(w[r][k]) on bf16 inputs, exact products, f64 sum */
void ixo_gemm_f64(const uint16_t *w, int64_t out_f, int64_t in_f, const uint16_t *x, int64_t m_rows, double *y) {
    for (int64_t m = 0; m < m_rows; ++m)
        for (int64_t r = 0; r < out_f; ++r) {
            const uint16_t *wr = w + r * in_f, *xm = x + m * in_f;
            double acc = 0.0;
            for (int64_t k = 0; k < in_f; ++k) acc += (double)bf16_to_f32(xm[k]) * (double)bf16_to_f32(wr[k]);
            y[m * out_f + r] = acc;
        }
}

/* the same contraction with a sequential fp32 accumulator, rounded to bf16 */
void ixo_gemm_f32(const uint16_t *w, int64_t out_f, int64_t in_f, const uint16_t *x, int64_t m_rows, uint16_t *y) {
    for (int64_t m = 0; m < m_rows; ++m)
        for (int64_t r = 0; r < out_f; ++r) {
            const uint16_t *wr = w + r * in_f, *xm = x + m * in_f;
            float acc = 0.0f;
            for (int64_t k = 0; k < in_f; ++k) acc += bf16_to_f32(xm[k]) * bf16_to_f32(wr[k]);
            y[m * out_f + r] = f32_to_bf16(acc);
        }
}

/* Fused walk used as the timed CPU baseline: decode row by row into a small
 * bf16 row buffer and contract it with x, fp32 accumulate, bf16 out.  Same
 * arithmetic as ixo_decode_i8 + ixo_dequant_bf16 + ixo_gemm_f32. */
void ixo_fused_gemv_f32(int64_t out_f, int64_t in_f, const int *level_bits, int n_levels,
                        uint32_t *const *bitmaps, uint32_t *const *streams, const uint8_t *last,
                        uint16_t scale, const uint16_t *x, uint16_t *y) {
    int64_t bm_cur[8] = {0}, st_cur[8] = {0};
    float s = bf16_to_f32(scale);
    for (int64_t r = 0; r < out_f; ++r) {
        float acc = 0.0f;
        for (int64_t k = 0; k < in_f; ++k) {
            int lv = n_levels - 1;
            for (int i = 0; i < n_levels - 1; ++i) {
                int64_t b = bm_cur[i]++;
                if ((bitmaps[i][b >> 5] >> (b & 31)) & 1u) { lv = i; break; }
            }
            int v;
            if (lv < n_levels - 1)
                v = (int)read_code(streams[lv], st_cur[lv]++, level_bits[lv]) - threshold_of(level_bits[lv]);
            else
                v = (int)last[st_cur[lv]++] - 127;
            float wv = bf16_to_f32(f32_to_bf16((float)v * s));
            acc += bf16_to_f32(x[k]) * wv;
        }
        y[r] = f32_to_bf16(acc);
    }
}

/* ======================================================================
 * Group-scale sibling format (reference: ixgs/).  Same streams as (3,5,8)
 * with code offsets 3 / 15 / 127; membership is by value range, and every
 * group of `group` consecutive elements has its own fp16 scale.
 * ====================================================================== */

/* fp32 -> fp16 bit pattern, round to nearest even (torch .to(float16)) */
static uint16_t f32_to_f16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    uint32_t sign = (u >> 16) & 0x8000u, a = u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return (uint16_t)(sign | 0x7E00u);            /* NaN */
    if (a >= 0x47800000u) return (uint16_t)(sign | 0x7C00u);           /* >= 65536 (or inf): inf; 65520..65536 below */
    if (a < 0x33000000u) return (uint16_t)sign;                         /* < 2^-25: zero */
    int e = (int)(a >> 23) - 127;
    uint32_t m = (a & 0x7FFFFFu) | 0x800000u;                          /* 24-bit significand */
    int shift = e >= -14 ? 13 : 13 + (-14 - e);                        /* bits dropped */
    uint32_t kept = m >> shift, rem = m & ((1u << shift) - 1u), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (kept & 1u))) kept++;
    uint32_t h;
    if (e >= -14) h = ((uint32_t)(e + 15) << 10) + (kept - 0x400u);   /* carry into the exponent is the right answer */
    else h = kept;                                                      /* subnormal; kept == 0x400 becomes the first normal */
    if (h >= 0x7C00u) h = 0x7C00u;
    return (uint16_t)(sign | h);
}

static float f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16, e = (h >> 10) & 31u, m = h & 0x3FFu, u;
    if (e == 31) u = sign | 0x7F800000u | (m << 13);
    else if (e != 0) u = sign | ((e + 112u) << 23) | (m << 13);
    else if (m == 0) u = sign;
    else {
        int k = 0;
        while (!(m & 0x400u)) { m <<= 1; ++k; }
        u = sign | ((uint32_t)(113 - k) << 23) | ((m & 0x3FFu) << 13);
    }
    float f;
    memcpy(&f, &u, 4);
    return f;
}

uint16_t ixo_f32_to_f16(float f) { return f32_to_f16(f); }
float ixo_f16_to_f32(uint16_t h) { return f16_to_f32(h); }

/* scales[g] = fp16( max(group max / 15, 1e-10) ); q = clamp(round_half_even(w / f32(scale)), -127, 128).
 * A group whose fp16 scale is zero (all-zero group, or max below 4.5e-7) divides by zero in the
 * reference and its integers are undefined there; here they are 0, which decodes to 0. */
void ixo_gs_quantize(const uint16_t *w, int64_t n, int64_t group, uint16_t *scales, int16_t *q) {
    int64_t n_groups = (n + group - 1) / group;
    for (int64_t g = 0; g < n_groups; ++g) {
        int64_t a = g * group, b = a + group < n ? a + group : n;
        float gmax = 0.0f;
        for (int64_t i = a; i < b; ++i) {
            float v = fabsf(bf16_to_f32(w[i]));
            if (v > gmax) gmax = v;
        }
        float s32 = gmax / 15.0f;
        if (s32 < 1e-10f) s32 = 1e-10f;
        uint16_t h = f32_to_f16(s32);
        float s = f16_to_f32(h);
        scales[g] = h;
        for (int64_t i = a; i < b; ++i) {
            float r = s == 0.0f ? 0.0f : rintf(bf16_to_f32(w[i]) / s);
            if (r > 128.0f) r = 128.0f;
            if (r < -127.0f) r = -127.0f;
            q[i] = (int16_t)r;
        }
    }
}

/* b1: one bit per element (1 = tier 1); b2: one bit per element outside tier 1 (1 = tier 2);
 * l1: 3-bit codes v+3; l2: 5-bit codes v+15; l3: bytes v+127.  Buffers zero-filled by the caller,
 * counts[3] written.  (The reference pads an empty b2 / l3 to one element; padding is the caller's.) */
void ixo_gs_encode(const int16_t *q, int64_t n, uint32_t *b1, uint32_t *b2, uint32_t *l1, uint32_t *l2, uint8_t *l3,
                   int64_t *counts) {
    int64_t n1 = 0, n2 = 0, n3 = 0, rest = 0;
    for (int64_t p = 0; p < n; ++p) {
        int v = q[p];
        if (v >= -3 && v <= 4) {
            b1[p >> 5] |= 1u << (p & 31);
            int64_t bit = n1 * 3;
            uint64_t c = (uint64_t)(uint32_t)(v + 3) << (bit & 31);
            l1[bit >> 5] |= (uint32_t)c;
            if (c >> 32) l1[(bit >> 5) + 1] |= (uint32_t)(c >> 32);
            ++n1;
        } else {
            if (v >= -15 && v <= 16) {
                b2[rest >> 5] |= 1u << (rest & 31);
                int64_t bit = n2 * 5;
                uint64_t c = (uint64_t)(uint32_t)(v + 15) << (bit & 31);
                l2[bit >> 5] |= (uint32_t)c;
                if (c >> 32) l2[(bit >> 5) + 1] |= (uint32_t)(c >> 32);
                ++n2;
            } else {
                l3[n3++] = (uint8_t)(v + 127);
            }
            ++rest;
        }
    }
    counts[0] = n1; counts[1] = n2; counts[2] = n3;
}

void ixo_gs_decode_i16(int64_t n, const uint32_t *b1, const uint32_t *b2, const uint32_t *l1, const uint32_t *l2,
                       const uint8_t *l3, int16_t *q) {
    int64_t n1 = 0, n2 = 0, n3 = 0, rest = 0;
    for (int64_t p = 0; p < n; ++p) {
        if ((b1[p >> 5] >> (p & 31)) & 1u) {
            q[p] = (int16_t)((int)read_code(l1, n1++, 3) - 3);
        } else {
            if ((b2[rest >> 5] >> (rest & 31)) & 1u) q[p] = (int16_t)((int)read_code(l2, n2++, 5) - 15);
            else q[p] = (int16_t)((int)l3[n3++] - 127);
            ++rest;
        }
    }
}

/* w = bf16( f32(v) * f32(fp16 scale of the element's group) ) */
void ixo_gs_dequant_bf16(const int16_t *q, int64_t n, int64_t group, const uint16_t *scales, uint16_t *w) {
    for (int64_t i = 0; i < n; ++i) w[i] = f32_to_bf16((float)q[i] * f16_to_f32(scales[i / group]));
}
