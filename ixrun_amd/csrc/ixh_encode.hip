// The INT8-X encoder on the device: bf16 weights -> scale, rank table, nested bitmaps and code streams,
// byte for byte what the reference's CPU writer produces (ixrun/quantize.py:41-122 with the bit packing of
// ixrun/bitpack.py:13-61, :87-89).  Three passes over the weights, all bound by HBM reads:
//   1. k_enc_absmax      largest magnitude, one partial result per workgroup (no atomics, nothing to clear);
//                        k_enc_scale (one wave) turns the partial results into the bf16 scale
//   2. k_enc_count<L>    quantise, count every level per 512-element unit; the counts are then summed into
//                        the rank table (k_enc_tile_sums, k_enc_scan), which is the table the decoders take
//   3. k_enc_pack<L>     quantise again, one wave per unit: the table says at which bit of every stream the
//                        unit starts.  The first level is packed eight elements per lane (a wave prefix sum
//                        places each lane's codes); what the first level leaves is queued in LDS in flat
//                        order and taken through the other levels 64 elements at a time, ranked by ballots.
//                        Each stream's piece is assembled in LDS and written as whole words; the two words a
//                        piece may share with its neighbours are OR-ed in (the streams are cleared first)
// Between passes 2 and 3 the caller reads the level totals (last table entries) and sizes the streams.
#include "ixh_dev.h"

namespace ixh {

constexpr uint32_t kEncUnit = 512;          // elements per wave and step: eight per lane
constexpr int kEncWaves = 4;                // waves per workgroup
constexpr uint32_t kEncParts = 256;         // partial maxima of pass 1 (one per workgroup of 1024 lanes)
constexpr uint32_t kEncWindow = kEncUnit * 7 / 32 + 4;  // LDS words for one unit's piece of the widest stream
constexpr uint32_t kScanTile = 8192;        // table entries per workgroup of the scan

// Eight consecutive bf16 starting at element p, widened to fp32 (zero past n).  Vector load when the address
// allows it.
__device__ __forceinline__ void load8(const uint16_t *__restrict__ w, uint32_t p, uint32_t n, bool aligned,
                                      float (&f)[8]) {
    if (aligned && p + 8 <= n) {
        const uint4 v = *reinterpret_cast<const uint4 *>(w + p);
        const uint32_t d[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            f[2 * k] = __uint_as_float(d[k] << 16);
            f[2 * k + 1] = __uint_as_float(d[k] & 0xffff0000u);
        }
    } else {
#pragma unroll
        for (int t = 0; t < 8; ++t) f[t] = p + t < n ? bf16_bits_to_f32(w[p + t]) : 0.0f;
    }
}

__device__ __forceinline__ uint32_t wave_max(uint32_t v) {
    for (int off = 32; off > 0; off >>= 1) v = max(v, (uint32_t)__shfl_xor((int)v, off));
    return v;
}

// scale = bf16( max(|w|max, bf16(1e-8)) / 127 ), the bf16 arithmetic of quantize.py:64 (the quotient is formed
// in fp32 and rounded once)
__device__ __forceinline__ uint32_t scale_bits_from_parts(const uint32_t *__restrict__ parts, uint32_t lane) {
    uint32_t m = 0;
    for (uint32_t i = lane; i < kEncParts; i += kWave) m = max(m, parts[i]);
    m = wave_max(m);
    const float floor_ = bf16_bits_to_f32(f32_to_bf16_bits(1e-8f));
    const float amax = fmaxf(bf16_bits_to_f32(m), floor_);
    return f32_to_bf16_bits(__fdiv_rn(amax, 127.0f));
}

// int8 of one weight: round-half-even of the fp32 quotient, clamped (quantize.py:65-70), without the division.
// Weight and scale are bf16 values (8-bit significands), so the exact quotient is either a tie k + 1/2 itself or at
// least 2^-9 away from every tie, and the fp32 rounding of the quotient cannot move it across one: the reference's
// round(fl(w / s)) equals round-half-even of the exact quotient.  w * (1/s) is within 2.5e-5 of that quotient (|q| <=
// 127.25); adding and subtracting 3072 snaps it to a multiple of 2^-12, which puts exact ties back on k + 1/2 and
// leaves everything else on its side.  Checked against the division for every bf16 weight and scale significand.
__device__ __forceinline__ float quantise(float w, float inv_scale) {
    const float snapped = __fmaf_rn(w, inv_scale, 3072.0f) - 3072.0f;
    return __builtin_amdgcn_fmed3f(rintf(snapped), -127.0f, 127.0f);
}

struct EncLevels {
    int n_levels;
    int bits[IXH_MAX_LEVELS];
};

__global__ void __launch_bounds__(1024) k_enc_absmax(const uint16_t *__restrict__ w, uint32_t n, uint32_t *parts) {
    const bool aligned = (reinterpret_cast<uintptr_t>(w) & 15u) == 0;
    uint32_t m = 0;
    const uint32_t stride = gridDim.x * 1024u * 8u;
    for (uint64_t p = ((uint64_t)blockIdx.x * 1024u + threadIdx.x) * 8u; p < n; p += stride) {
        float f[8];
        load8(w, (uint32_t)p, n, aligned, f);
#pragma unroll
        for (int t = 0; t < 8; ++t) m = max(m, (__float_as_uint(f[t]) >> 16) & 0x7fffu);
    }
    __shared__ uint32_t wave_m[16];
    m = wave_max(m);
    if ((threadIdx.x & 63) == 0) wave_m[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x < 16) {
        m = wave_m[threadIdx.x];
        for (int off = 8; off > 0; off >>= 1) m = max(m, (uint32_t)__shfl_xor((int)m, off));
        if (threadIdx.x == 0) parts[blockIdx.x] = m;
    }
}

__global__ void __launch_bounds__(kWave) k_enc_scale(const uint32_t *__restrict__ parts, uint16_t *scale_out) {
    const uint32_t sbits = scale_bits_from_parts(parts, threadIdx.x);
    if (threadIdx.x == 0) *scale_out = (uint16_t)sbits;
}

// table[i * entries + u + 1] = number of level-i elements of unit u (raw counts; the scan turns them into ranks).
// A wave takes kCountUnits units in a row; a level is "the thresholds below |v|" (quantize.py:25-37), so the
// kernel counts, per threshold, the values above it and takes differences.
constexpr int kCountUnits = 4;

template <int L>
__global__ void __launch_bounds__(kWave *kEncWaves)
k_enc_count(const uint16_t *__restrict__ w, uint32_t n, uint32_t n_units, const uint16_t *__restrict__ scale_in,
            EncLevels lv, int32_t *table) {
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t u0 = (blockIdx.x * kEncWaves + (threadIdx.x >> 6)) * kCountUnits;
    if (u0 >= n_units) return;
    const bool aligned = (reinterpret_cast<uintptr_t>(w) & 15u) == 0;
    float thr[L - 1];
#pragma unroll
    for (int i = 0; i < L - 1; ++i) thr[i] = (float)threshold_of(lv.bits[i]);
    float f[kCountUnits][8];
#pragma unroll
    for (int k = 0; k < kCountUnits; ++k) load8(w, min((u0 + k) * kEncUnit + lane * 8u, n), n, aligned, f[k]);
    const float inv_scale = __fdiv_rn(1.0f, bf16_bits_to_f32(*scale_in));
    const uint32_t entries = n_units + 1;
#pragma unroll
    for (int k = 0; k < kCountUnits; ++k) {
        const uint32_t u = u0 + k;
        if (u >= n_units) break;
        // values above each threshold, 10-bit fields, three to a word: a wave holds at most 512 of anything
        uint32_t above[L - 1] = {};
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            const float a = fabsf(quantise(f[k][t], inv_scale));
#pragma unroll
            for (int i = 0; i < L - 1; ++i) above[i] += a > thr[i] ? 1u : 0u;
        }
        uint32_t acc[(L + 1) / 3] = {};
#pragma unroll
        for (int i = 0; i < L - 1; ++i) acc[i / 3] |= above[i] << (10 * (i % 3));
#pragma unroll
        for (int j = 0; j < (L + 1) / 3; ++j) acc[j] = wave_scan_inclusive(acc[j]);
        // elements of the unit (those past n were loaded as zero and are above nothing)
        uint32_t prev = min(kEncUnit, n - u * kEncUnit);
#pragma unroll
        for (int i = 0; i < L - 1; ++i) {
            const uint32_t ab = (acc[i / 3] >> (10 * (i % 3))) & 1023u;
            if (lane == 63) table[(size_t)i * entries + u + 1] = (int32_t)(prev - ab);
            prev = ab;
        }
    }
}

// sums[row * tiles + tile] = sum of the raw counts of one tile of one table row
__global__ void __launch_bounds__(1024) k_enc_tile_sums(const int32_t *__restrict__ table, uint32_t n_units,
                                                         uint32_t *sums) {
    const int32_t *row = table + (size_t)blockIdx.y * (n_units + 1) + 1;
    const uint32_t base = blockIdx.x * kScanTile;
    uint32_t s = 0;
    for (uint32_t k = threadIdx.x; k < kScanTile && base + k < n_units; k += 1024) s += (uint32_t)row[base + k];
    __shared__ uint32_t wave_s[16];
    s = wave_scan_inclusive(s);
    if ((threadIdx.x & 63) == 63) wave_s[threadIdx.x >> 6] = s;
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t t = 0;
        for (int i = 0; i < 16; ++i) t += wave_s[i];
        sums[blockIdx.y * gridDim.x + blockIdx.x] = t;
    }
}

// In place, per row: row[0] = 0, row[u + 1] = counts of units 0 .. u.  Each thread takes eight consecutive entries.
__global__ void __launch_bounds__(1024) k_enc_scan(int32_t *table, uint32_t n_units, const uint32_t *__restrict__ sums) {
    int32_t *row = table + (size_t)blockIdx.y * (n_units + 1);
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    __shared__ uint32_t wave_s[16], wave_c[16];
    // ranks before this tile: the partial sums of the tiles in front of it
    {
        uint32_t c = 0;
        const uint32_t *mine_sums = sums + (size_t)blockIdx.y * gridDim.x;
        for (uint32_t t = tid; t < blockIdx.x; t += 1024) c += mine_sums[t];
        c = wave_scan_inclusive(c);
        if (lane == 63) wave_c[wave] = c;
    }
    const uint32_t first = blockIdx.x * kScanTile + tid * 8u;
    uint32_t v[8];
    uint32_t mine = 0;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
        v[t] = first + t < n_units ? (uint32_t)row[first + t + 1] : 0u;
        mine += v[t];
    }
    const uint32_t incl = wave_scan_inclusive(mine);
    if (lane == 63) wave_s[wave] = incl;
    __syncthreads();
    uint32_t run = incl - mine;
    for (uint32_t k = 0; k < 16; ++k) run += wave_c[k] + (k < wave ? wave_s[k] : 0u);
#pragma unroll
    for (int t = 0; t < 8; ++t) {
        run += v[t];
        if (first + t < n_units) row[first + t + 1] = (int32_t)run;
    }
    if (blockIdx.x == 0 && tid == 0) row[0] = 0;
}

// every stream that is assembled with OR, in one launch
struct EncClear {
    uint32_t *dst[2 * (IXH_MAX_LEVELS - 1)];
    uint32_t words[2 * (IXH_MAX_LEVELS - 1)];
    int n;
};

__global__ void __launch_bounds__(256) k_enc_clear(EncClear c) {
    for (int k = 0; k < c.n; ++k)
        for (uint32_t i = blockIdx.x * 256u + threadIdx.x; i < c.words[k]; i += gridDim.x * 256u) c.dst[k][i] = 0u;
}

// Destination of the encoder: the same fields as Dev, writable.
struct EncOut {
    uint32_t *bm[IXH_MAX_LEVELS - 1];
    uint32_t bm_words[IXH_MAX_LEVELS - 1];
    uint32_t *st[IXH_MAX_LEVELS - 1];
    uint32_t st_words[IXH_MAX_LEVELS - 1];
    uint8_t *last;
    uint32_t last_bytes;
};

// OR `nbits` <= 64 bits of `value` into the window at bit `off`
__device__ __forceinline__ void window_or(uint32_t *win, uint32_t off, uint64_t value, uint32_t nbits) {
    if (nbits == 0) return;
    const uint32_t wi = off >> 5, sh = off & 31u;
    const uint64_t low = value << sh;
    const uint32_t w0 = (uint32_t)low, w1 = (uint32_t)(low >> 32);
    const uint32_t w2 = sh ? (uint32_t)(value >> (64u - sh)) : 0u;
    if (w0) atomicOr(&win[wi], w0);
    if (w1) atomicOr(&win[wi + 1], w1);
    if (w2) atomicOr(&win[wi + 2], w2);
}

// the same for a value of at most 8 bits
__device__ __forceinline__ void window_or_small(uint32_t *win, uint32_t off, uint32_t value) {
    const uint32_t wi = off >> 5, sh = off & 31u;
    const uint32_t w0 = value << sh, w1 = sh ? value >> (32u - sh) : 0u;
    if (w0) atomicOr(&win[wi], w0);
    if (w1) atomicOr(&win[wi + 1], w1);
}

// LDS traffic of this wave so far is visible to all its lanes after this
__device__ __forceinline__ void wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

// Write the window's words for the stream bits [bit0, bit1) and clear the window again.  The first and the last
// word may also hold bits of the neighbouring units and are OR-ed into the cleared stream; the words between
// belong to this unit alone.
__device__ __forceinline__ void window_flush(uint32_t *win, uint32_t *dst, uint32_t dst_words, uint64_t bit0,
                                             uint64_t bit1, uint32_t lane) {
    wave_lds_sync();
    if (bit1 > bit0) {
        const uint32_t w_first = (uint32_t)(bit0 >> 5);
        const uint32_t n_words = (uint32_t)((bit1 - 1) >> 5) - w_first + 1;
        for (uint32_t j = lane; j < n_words; j += kWave) {
            const uint32_t val = win[j];
            win[j] = 0u;
            if (w_first + j < dst_words) {
                if (j == 0 || j == n_words - 1) {
                    if (val) atomicOr(&dst[w_first + j], val);
                } else {
                    dst[w_first + j] = val;
                }
            }
        }
    }
    wave_lds_sync();
}

constexpr uint32_t kEncBmWindow = kEncUnit / 32 + 4;  // LDS words for one unit's piece of a bitmap

template <int L>
__global__ void __launch_bounds__(kWave *kEncWaves)
k_enc_pack(const uint16_t *__restrict__ w, uint32_t n, uint32_t n_units, const uint16_t *__restrict__ scale_in,
           EncLevels lv, const int32_t *__restrict__ table, EncOut out) {
    __shared__ uint32_t windows[kEncWaves][kEncWindow];
    __shared__ uint32_t bm_windows[kEncWaves][kEncBmWindow];
    __shared__ uint8_t queues[kEncWaves][kEncUnit];
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    uint32_t *win = windows[wave], *bm_win = bm_windows[wave];
    uint8_t *queue = queues[wave];
    for (uint32_t j = lane; j < kEncWindow; j += kWave) win[j] = 0u;
    if (lane < kEncBmWindow) bm_win[lane] = 0u;
    const uint32_t u = blockIdx.x * kEncWaves + wave;
    if (u >= n_units) return;
    const float inv_scale = __fdiv_rn(1.0f, bf16_bits_to_f32(*scale_in));
    const bool aligned = (reinterpret_cast<uintptr_t>(w) & 15u) == 0;
    const uint32_t entries = n_units + 1;
    // the unit's first rank in every level and the next unit's: requested now, needed after the first level
    uint32_t ranks0[L - 1], ranks1[L - 1];
#pragma unroll
    for (int i = 0; i < L - 1; ++i) {
        ranks0[i] = (uint32_t)table[(size_t)i * entries + u];
        ranks1[i] = (uint32_t)table[(size_t)i * entries + u + 1];
    }
    const uint32_t e0 = u * kEncUnit, e1 = min(e0 + kEncUnit, n);  // the unit's elements
    const uint32_t p = e0 + lane * 8u;
    float f[8];
    load8(w, min(p, n), n, aligned, f);
    const uint32_t n_valid = p < e1 ? min(8u, e1 - p) : 0u;
    const uint32_t valid = (1u << n_valid) - 1u;

    // ---- first level, eight elements per lane ----
    const uint32_t b0 = (uint32_t)lv.bits[0];
    const int thr0 = threshold_of((int)b0);
    int q[8];
    uint32_t above = 0;  // bit t: element t is not in the first level
#pragma unroll
    for (int t = 7; t >= 0; --t) {
        const float r = quantise(f[t], inv_scale);
        q[t] = (int)r;
        above = (above << 1) | (fabsf(r) > (float)thr0 ? 1u : 0u);
    }
    const uint32_t member = ~above & valid;  // elements past n were loaded as zero and are not above
    // bitmap 0 is indexed by the flat element: the lane's byte, four lanes to a word, whole words to memory
    reinterpret_cast<uint8_t *>(bm_win)[lane] = (uint8_t)member;
    wave_lds_sync();
    if (lane < kEncUnit / 32) {
        const uint32_t word = bm_win[lane], at = e0 / 32 + lane;
        bm_win[lane] = 0u;
        if (at < (n + 31u) / 32u && at < out.bm_words[0]) out.bm[0][at] = word;
    }
    uint32_t n_codes = 0;
    uint64_t codes = 0;
    if (b0 <= 4) {  // eight codes fit one register
        uint32_t c32 = 0, sh = 0;
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            const bool m = (member >> t) & 1u;
            c32 |= (m ? (uint32_t)(q[t] + thr0) : 0u) << sh;
            sh += m ? b0 : 0u;
        }
        codes = c32;
        n_codes = sh;
    } else {  // four and four, joined once
        uint32_t half[2] = {0, 0}, sh[2] = {0, 0};
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            const bool m = (member >> t) & 1u;
            half[t >> 2] |= (m ? (uint32_t)(q[t] + thr0) : 0u) << sh[t >> 2];
            sh[t >> 2] += m ? b0 : 0u;
        }
        codes = (uint64_t)half[0] | ((uint64_t)half[1] << sh[0]);
        n_codes = sh[0] + sh[1];
    }  // n_codes: bits of this lane's codes
    const uint32_t n_above = (uint32_t)__popc(above);
    const uint32_t incl = wave_scan_inclusive(n_codes | (n_above << 16));
    const uint32_t bits_before = (incl & 0xffffu) - n_codes, above_before = (incl >> 16) - n_above;
    const uint32_t total_above = (uint32_t)__builtin_amdgcn_readlane((int)(incl >> 16), 63);
    uint32_t rank0 = ranks0[0], rank1 = ranks1[0];
    {
        const uint64_t bit0 = (uint64_t)rank0 * b0, bit1 = (uint64_t)rank1 * b0;
        window_or(win, ((uint32_t)bit0 & 31u) + bits_before, codes, n_codes);
        window_flush(win, out.st[0], out.st_words[0], bit0, bit1, lane);
    }
    if (total_above == 0) return;  // the whole wave

    // ---- what the first level left, queued in flat order as v + 128 ----
    {
        uint32_t at = above_before;
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            if ((above >> t) & 1u) queue[at++] = (uint8_t)(q[t] + 128);
        }
    }
    wave_lds_sync();
    // first index of this unit and of the next one in the index space of the current level's bitmap
    uint32_t space0 = e0 - rank0, space1 = e1 - rank1;
    int thr_below = thr0;
#pragma unroll
    for (int i = 1; i < L - 1; ++i) {
        const uint32_t b = (uint32_t)lv.bits[i];
        const int thr_i = threshold_of((int)b);
        rank0 = ranks0[i];
        rank1 = ranks1[i];
        const uint64_t bit0 = (uint64_t)rank0 * b, bit1 = (uint64_t)rank1 * b;
        uint32_t seen_alive = space0 & 31u, seen_codes = (uint32_t)bit0 & 31u;  // window positions, in bits
        if (space1 > space0) {
            for (uint32_t s = 0; s < total_above; s += kWave) {
                const bool have = s + lane < total_above;
                const int v = have ? (int)queue[s + lane] - 128 : 0;
                const int a = v < 0 ? -v : v;
                const bool alive = have && a > thr_below;
                const bool mine = alive && a <= thr_i;
                const uint64_t alive_mask = __ballot(alive), mine_mask = __ballot(mine);
                if (mine) {
                    window_or_small(bm_win, seen_alive + lanes_below(alive_mask), 1u);
                    window_or_small(win, seen_codes + lanes_below(mine_mask) * b, (uint32_t)(v + thr_i));
                }
                seen_alive += (uint32_t)__popcll(alive_mask);
                seen_codes += (uint32_t)__popcll(mine_mask) * b;
            }
        }
        window_flush(bm_win, out.bm[i], out.bm_words[i], space0, space1, lane);
        window_flush(win, out.st[i], out.st_words[i], bit0, bit1, lane);
        space0 -= rank0;
        space1 -= rank1;
        thr_below = thr_i;
    }
    // last level: one byte per element left over (quantize.py:84-86)
    if (space1 > space0) {
        uint32_t at = space0;
        for (uint32_t s = 0; s < total_above; s += kWave) {
            const bool have = s + lane < total_above;
            const int v = have ? (int)queue[s + lane] - 128 : 0;
            const bool mine = have && (v < 0 ? -v : v) > thr_below;
            const uint64_t mine_mask = __ballot(mine);
            const uint32_t dst = at + lanes_below(mine_mask);
            if (mine && dst < out.last_bytes) out.last[dst] = (uint8_t)(v + 127);
            at += (uint32_t)__popcll(mine_mask);
        }
    }
}

size_t encode_workspace_bytes(uint64_t n, int n_levels) {
    const uint64_t n_units = (n + kEncUnit - 1) / kEncUnit;
    const uint64_t tiles = (n_units + kScanTile - 1) / kScanTile;
    return (size_t)(kEncParts * 4u + (uint64_t)(n_levels - 1) * (tiles ? tiles : 1) * 4u);
}

template <int L>
static void scan_launch(const uint16_t *w, uint32_t n, uint32_t n_units, const EncLevels &lv, const uint16_t *scale,
                        int32_t *table, hipStream_t s) {
    const uint32_t per_block = kEncWaves * kCountUnits;
    hipLaunchKernelGGL(k_enc_count<L>, dim3((n_units + per_block - 1) / per_block), dim3(kWave * kEncWaves), 0, s, w, n,
                       n_units, scale, lv, table);
}

int launch_encode_scan(const uint16_t *w, uint32_t n, int n_levels, const int *bits, uint16_t *scale, int32_t *table,
                       void *workspace, hipStream_t s) {
    const uint32_t n_units = (n + kEncUnit - 1) / kEncUnit;
    const uint32_t tiles = max(1u, (n_units + kScanTile - 1) / kScanTile);
    uint32_t *parts = static_cast<uint32_t *>(workspace);
    uint32_t *sums = parts + kEncParts;
    EncLevels lv;
    lv.n_levels = n_levels;
    for (int i = 0; i < IXH_MAX_LEVELS; ++i) lv.bits[i] = i < n_levels ? bits[i] : 0;
    hipLaunchKernelGGL(k_enc_absmax, dim3(kEncParts), dim3(1024), 0, s, w, n, parts);
    hipLaunchKernelGGL(k_enc_scale, dim3(1), dim3(kWave), 0, s, parts, scale);
    switch (n_levels) {
        case 2: scan_launch<2>(w, n, n_units, lv, scale, table, s); break;
        case 3: scan_launch<3>(w, n, n_units, lv, scale, table, s); break;
        case 4: scan_launch<4>(w, n, n_units, lv, scale, table, s); break;
        case 5: scan_launch<5>(w, n, n_units, lv, scale, table, s); break;
        case 6: scan_launch<6>(w, n, n_units, lv, scale, table, s); break;
        case 7: scan_launch<7>(w, n, n_units, lv, scale, table, s); break;
        default: scan_launch<8>(w, n, n_units, lv, scale, table, s); break;
    }
    hipLaunchKernelGGL(k_enc_tile_sums, dim3(tiles, n_levels - 1), dim3(1024), 0, s, table, n_units, sums);
    hipLaunchKernelGGL(k_enc_scan, dim3(tiles, n_levels - 1), dim3(1024), 0, s, table, n_units, sums);
    return hipGetLastError() == hipSuccess ? IXH_OK : IXH_ELAUNCH;
}

template <int L>
static void pack_launch(const uint16_t *w, uint32_t n, uint32_t n_units, const uint16_t *scale, const EncLevels &lv,
                        const int32_t *table, const EncOut &out, hipStream_t s) {
    hipLaunchKernelGGL(k_enc_pack<L>, dim3((n_units + kEncWaves - 1) / kEncWaves), dim3(kWave * kEncWaves), 0, s, w, n,
                       n_units, scale, lv, table, out);
}

int launch_encode_pack(const uint16_t *w, const Dev &P, const int32_t *table, hipStream_t s) {
    const uint32_t n = P.n;
    const uint32_t n_units = (n + kEncUnit - 1) / kEncUnit;
    EncLevels lv;
    lv.n_levels = P.n_levels;
    EncOut out;
    for (int i = 0; i < IXH_MAX_LEVELS; ++i) lv.bits[i] = i < P.n_levels ? P.bits[i] : 0;
    for (int i = 0; i < IXH_MAX_LEVELS - 1; ++i) {
        out.bm[i] = const_cast<uint32_t *>(P.bm[i]);
        out.bm_words[i] = P.bm_words[i];
        out.st[i] = const_cast<uint32_t *>(P.st[i]);
        out.st_words[i] = P.st_words[i];
    }
    out.last = const_cast<uint8_t *>(P.last);
    out.last_bytes = P.last_bytes;
    EncClear clr;
    clr.n = 0;
    uint32_t most = 0;
    for (int i = 0; i < P.n_levels - 1; ++i) {
        if (out.bm_words[i] && i > 0) {  // bitmap 0 is written in whole words
            clr.dst[clr.n] = out.bm[i];
            clr.words[clr.n++] = out.bm_words[i];
            most = max(most, out.bm_words[i]);
        }
        if (out.st_words[i]) {
            clr.dst[clr.n] = out.st[i];
            clr.words[clr.n++] = out.st_words[i];
            most = max(most, out.st_words[i]);
        }
    }
    if (clr.n) hipLaunchKernelGGL(k_enc_clear, dim3(min(2048u, (most + 255u) / 256u)), dim3(256), 0, s, clr);
    if (n_units != 0) {
        switch (P.n_levels) {
            case 2: pack_launch<2>(w, n, n_units, P.scale, lv, table, out, s); break;
            case 3: pack_launch<3>(w, n, n_units, P.scale, lv, table, out, s); break;
            case 4: pack_launch<4>(w, n, n_units, P.scale, lv, table, out, s); break;
            case 5: pack_launch<5>(w, n, n_units, P.scale, lv, table, out, s); break;
            case 6: pack_launch<6>(w, n, n_units, P.scale, lv, table, out, s); break;
            case 7: pack_launch<7>(w, n, n_units, P.scale, lv, table, out, s); break;
            default: pack_launch<8>(w, n, n_units, P.scale, lv, table, out, s); break;
        }
    }
    return hipGetLastError() == hipSuccess ? IXH_OK : IXH_ELAUNCH;
}

}  // namespace ixh
