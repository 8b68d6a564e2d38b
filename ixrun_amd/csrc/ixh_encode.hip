// The INT8-X encoder on the device: bf16 weights -> scale, rank table, nested bitmaps and code streams,
// byte for byte what the reference's CPU writer produces (ixrun/quantize.py:41-122 with the bit packing of
// ixrun/bitpack.py:13-61, :87-89).  Three passes over the weights, all bound by HBM reads:
//   1. k_enc_absmax      largest magnitude, one partial result per workgroup (no atomics, nothing to clear)
//   2. k_enc_count<L>    quantise, count every level per 512-element unit; the counts are then summed into
//                        the rank table (k_enc_tile_sums, k_enc_scan), which is the table the decoders take
//   3. k_enc_pack<L>     quantise again, one wave per unit: the table says at which bit of every stream the
//                        unit starts, a wave prefix sum says where each lane's eight elements go; the wave
//                        assembles each stream's piece in LDS and writes whole words, the two words it may
//                        share with its neighbours with an atomic OR (the streams are cleared first)
// Between passes 2 and 3 the caller reads the level totals (last table entries) and sizes the streams.
#include "ixh_dev.h"

namespace ixh {

constexpr uint32_t kEncUnit = 512;          // elements per wave and step: eight per lane
constexpr int kEncWaves = 4;                // waves per workgroup
constexpr uint32_t kEncParts = 1024;        // partial maxima of pass 1
constexpr uint32_t kEncWindow = kEncUnit * 7 / 32 + 4;  // LDS words for one unit's piece of the widest stream
constexpr uint32_t kScanTile = 8192;        // table entries per workgroup of the scan

// Eight consecutive bf16 starting at element p (zero past n).  Vector load when the address allows it.
__device__ __forceinline__ void load8(const uint16_t *__restrict__ w, uint32_t p, uint32_t n, bool aligned,
                                      uint32_t (&h)[8]) {
    if (aligned && p + 8 <= n) {
        const uint4 v = *reinterpret_cast<const uint4 *>(w + p);
        h[0] = v.x & 0xffffu; h[1] = v.x >> 16; h[2] = v.y & 0xffffu; h[3] = v.y >> 16;
        h[4] = v.z & 0xffffu; h[5] = v.z >> 16; h[6] = v.w & 0xffffu; h[7] = v.w >> 16;
    } else {
#pragma unroll
        for (int t = 0; t < 8; ++t) h[t] = p + t < n ? w[p + t] : 0u;
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

// int8 of one weight: round-half-even of the fp32 quotient, clamped (quantize.py:65-70)
__device__ __forceinline__ int quantise(uint32_t h, float scale) {
    float r = rintf(__fdiv_rn(bf16_bits_to_f32(h), scale));
    r = fminf(fmaxf(r, -127.0f), 127.0f);
    return (int)r;
}

struct EncLevels {
    int n_levels;
    int bits[IXH_MAX_LEVELS];
};

// level of a value: number of thresholds below |v| (the thresholds ascend; quantize.py:25-37)
template <int L>
__device__ __forceinline__ int level_of(int v, const int (&thr)[L - 1]) {
    const int a = v < 0 ? -v : v;
    int lvl = 0;
#pragma unroll
    for (int i = 0; i < L - 1; ++i) lvl += a > thr[i] ? 1 : 0;
    return lvl;
}

__global__ void __launch_bounds__(256) k_enc_absmax(const uint16_t *__restrict__ w, uint32_t n, uint32_t *parts) {
    const bool aligned = (reinterpret_cast<uintptr_t>(w) & 15u) == 0;
    uint32_t m = 0;
    const uint32_t stride = gridDim.x * 256u * 8u;
    for (uint64_t p = ((uint64_t)blockIdx.x * 256u + threadIdx.x) * 8u; p < n; p += stride) {
        uint32_t h[8];
        load8(w, (uint32_t)p, n, aligned, h);
#pragma unroll
        for (int t = 0; t < 8; ++t) m = max(m, h[t] & 0x7fffu);
    }
    __shared__ uint32_t wave_m[4];
    m = wave_max(m);
    if ((threadIdx.x & 63) == 0) wave_m[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0) parts[blockIdx.x] = max(max(wave_m[0], wave_m[1]), max(wave_m[2], wave_m[3]));
}

// table[i * entries + u + 1] = number of level-i elements of unit u (raw counts; the scan turns them into ranks)
template <int L>
__global__ void __launch_bounds__(kWave *kEncWaves)
k_enc_count(const uint16_t *__restrict__ w, uint32_t n, uint32_t n_units, const uint32_t *__restrict__ parts,
            EncLevels lv, uint16_t *scale_out, int32_t *table) {
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t sbits = scale_bits_from_parts(parts, lane);
    if (blockIdx.x == 0 && threadIdx.x == 0) *scale_out = (uint16_t)sbits;
    const uint32_t u = blockIdx.x * kEncWaves + (threadIdx.x >> 6);
    if (u >= n_units) return;
    const float scale = bf16_bits_to_f32(sbits);
    const bool aligned = (reinterpret_cast<uintptr_t>(w) & 15u) == 0;
    int thr[L - 1];
#pragma unroll
    for (int i = 0; i < L - 1; ++i) thr[i] = threshold_of(lv.bits[i]);
    const uint32_t p = u * kEncUnit + lane * 8u;
    uint32_t h[8];
    load8(w, min(p, n), n, aligned, h);
    // per-level counts of this lane in 10-bit fields, three to a word: a wave holds at most 512 of a level
    uint32_t acc[(L + 1) / 3] = {};
#pragma unroll
    for (int t = 0; t < 8; ++t) {
        if (p + t < n) {
            const int lvl = level_of<L>(quantise(h[t], scale), thr);
#pragma unroll
            for (int i = 0; i < L - 1; ++i) acc[i / 3] += (lvl == i ? 1u : 0u) << (10 * (i % 3));
        }
    }
#pragma unroll
    for (int k = 0; k < (L + 1) / 3; ++k)
        for (int off = 32; off > 0; off >>= 1) acc[k] += (uint32_t)__shfl_xor((int)acc[k], off);
    if (lane == 0) {
        const uint32_t entries = n_units + 1;
#pragma unroll
        for (int i = 0; i < L - 1; ++i)
            table[(size_t)i * entries + u + 1] = (int32_t)((acc[i / 3] >> (10 * (i % 3))) & 1023u);
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
    for (int off = 32; off > 0; off >>= 1) s += (uint32_t)__shfl_xor((int)s, off);
    if ((threadIdx.x & 63) == 0) wave_s[threadIdx.x >> 6] = s;
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t t = 0;
        for (int i = 0; i < 16; ++i) t += wave_s[i];
        sums[blockIdx.y * gridDim.x + blockIdx.x] = t;
    }
}

// In place, per row: row[0] = 0, row[u + 1] = counts of units 0 .. u.  Each thread takes eight consecutive entries.
__global__ void __launch_bounds__(1024) k_enc_scan(int32_t *table, uint32_t n_units, const uint32_t *__restrict__ sums,
                                                    int64_t *totals, uint32_t n) {
    int32_t *row = table + (size_t)blockIdx.y * (n_units + 1);
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    __shared__ uint32_t wave_s[16];
    __shared__ uint32_t carry_in;
    // ranks before this tile: the sums of the tiles in front of it
    if (wave == 0) {
        uint32_t c = 0;
        for (uint32_t t = lane; t < blockIdx.x; t += kWave) c += sums[blockIdx.y * gridDim.x + t];
        for (int off = 32; off > 0; off >>= 1) c += (uint32_t)__shfl_xor((int)c, off);
        if (lane == 0) carry_in = c;
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
    uint32_t run = carry_in + incl - mine;
    for (uint32_t k = 0; k < wave; ++k) run += wave_s[k];
#pragma unroll
    for (int t = 0; t < 8; ++t) {
        run += v[t];
        if (first + t < n_units) row[first + t + 1] = (int32_t)run;
    }
    if (blockIdx.x == 0 && tid == 0) row[0] = 0;
    // level totals for the caller: the last entry of each row; the last level takes what is left.  Written by
    // the workgroup that owns the row's last entry; the last level's total by a later, tiny kernel.
    if (totals && n_units != 0 && first <= n_units - 1 && n_units - 1 < first + 8) totals[blockIdx.y] = (int64_t)run;
    (void)n;
}

__global__ void k_enc_last_total(int64_t *totals, int n_levels, uint32_t n, uint32_t n_units) {
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    int64_t rest = n;
    for (int i = 0; i < n_levels - 1; ++i) {
        if (n_units == 0) totals[i] = 0;
        rest -= totals[i];
    }
    totals[n_levels - 1] = rest;
}

__global__ void __launch_bounds__(256) k_enc_clear(uint32_t *dst, uint32_t words) {
    for (uint32_t i = blockIdx.x * 256u + threadIdx.x; i < words; i += gridDim.x * 256u) dst[i] = 0u;
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

// Write the window's words for the stream bits [bit0, bit1) and clear the window again.  The first and the last
// word may also hold bits of the neighbouring units and are OR-ed into the cleared stream; the words between
// belong to this unit alone.
__device__ __forceinline__ void window_flush(uint32_t *win, uint32_t *dst, uint32_t dst_words, uint64_t bit0,
                                             uint64_t bit1, uint32_t lane) {
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
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
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

template <int L>
__global__ void __launch_bounds__(kWave *kEncWaves)
k_enc_pack(const uint16_t *__restrict__ w, uint32_t n, uint32_t n_units, const uint16_t *__restrict__ scale_in,
           EncLevels lv, const int32_t *__restrict__ table, EncOut out) {
    __shared__ uint32_t windows[kEncWaves][kEncWindow];
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    uint32_t *win = windows[wave];
    for (uint32_t j = lane; j < kEncWindow; j += kWave) win[j] = 0u;
    const uint32_t u = blockIdx.x * kEncWaves + wave;
    if (u >= n_units) return;
    const float scale = bf16_bits_to_f32(*scale_in);
    const bool aligned = (reinterpret_cast<uintptr_t>(w) & 15u) == 0;
    const uint32_t entries = n_units + 1;
    const uint32_t p = u * kEncUnit + lane * 8u;
    uint32_t h[8];
    load8(w, min(p, n), n, aligned, h);
    int q[8], lvl[8];
    {
        int thr[L - 1];
#pragma unroll
        for (int i = 0; i < L - 1; ++i) thr[i] = threshold_of(lv.bits[i]);
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            q[t] = quantise(h[t], scale);
            lvl[t] = p + t < n ? level_of<L>(q[t], thr) : -1;  // -1: past the end, in no level and not alive
        }
    }
    // first rank of this unit and of the next one in the index space of the current level's bitmap
    uint64_t space0 = min((uint64_t)u * kEncUnit, (uint64_t)n), space1 = min((uint64_t)(u + 1) * kEncUnit, (uint64_t)n);
#pragma unroll
    for (int i = 0; i < L - 1; ++i) {
        const uint32_t b = (uint32_t)lv.bits[i];
        const int thr_i = threshold_of((int)b);
        const uint32_t rank0 = (uint32_t)table[(size_t)i * entries + u];
        const uint32_t rank1 = (uint32_t)table[(size_t)i * entries + u + 1];
        // this lane's bitmap bits (one per element still alive) and codes (one per member), lowest first
        uint32_t bm_bits = 0, n_alive = 0, n_codes = 0;
        uint64_t codes = 0;
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            const bool alive = lvl[t] >= i;
            const bool member = lvl[t] == i;
            bm_bits |= (member ? 1u : 0u) << n_alive;
            codes |= (uint64_t)(member ? (uint32_t)(q[t] + thr_i) : 0u) << (n_codes * b);
            n_alive += alive ? 1u : 0u;
            n_codes += member ? 1u : 0u;
        }
        const uint32_t incl = wave_scan_inclusive(n_alive | (n_codes << 16));
        const uint32_t alive_before = (incl & 0xffffu) - n_alive, codes_before = (incl >> 16) - n_codes;
        // bitmap i
        window_or(win, ((uint32_t)space0 & 31u) + alive_before, bm_bits, n_alive);
        window_flush(win, out.bm[i], out.bm_words[i], space0, space1, lane);
        // stream i
        const uint64_t bit0 = (uint64_t)rank0 * b, bit1 = (uint64_t)rank1 * b;
        window_or(win, ((uint32_t)bit0 & 31u) + codes_before * b, codes, n_codes * b);
        window_flush(win, out.st[i], out.st_words[i], bit0, bit1, lane);
        space0 -= rank0;
        space1 -= rank1;
    }
    // last level: one byte per element left over (quantize.py:84-86)
    {
        uint32_t n_mine = 0;
#pragma unroll
        for (int t = 0; t < 8; ++t) n_mine += lvl[t] == L - 1 ? 1u : 0u;
        uint32_t at = (uint32_t)space0 + wave_scan_inclusive(n_mine) - n_mine;
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            if (lvl[t] == L - 1) {
                if (at < out.last_bytes) out.last[at] = (uint8_t)(q[t] + 127);
                ++at;
            }
        }
    }
}

size_t encode_workspace_bytes(uint64_t n, int n_levels) {
    const uint64_t n_units = (n + kEncUnit - 1) / kEncUnit;
    const uint64_t tiles = (n_units + kScanTile - 1) / kScanTile;
    return (size_t)(kEncParts * 4u + (uint64_t)(n_levels - 1) * (tiles ? tiles : 1) * 4u);
}

template <int L>
static void scan_launch(const uint16_t *w, uint32_t n, uint32_t n_units, const uint32_t *parts, const EncLevels &lv,
                        uint16_t *scale, int32_t *table, hipStream_t s) {
    hipLaunchKernelGGL(k_enc_count<L>, dim3(max(1u, (n_units + kEncWaves - 1) / kEncWaves)), dim3(kWave * kEncWaves), 0,
                       s, w, n, n_units, parts, lv, scale, table);
}

int launch_encode_scan(const uint16_t *w, uint32_t n, int n_levels, const int *bits, uint16_t *scale, int32_t *table,
                       int64_t *totals, void *workspace, hipStream_t s) {
    const uint32_t n_units = (n + kEncUnit - 1) / kEncUnit;
    uint32_t *parts = static_cast<uint32_t *>(workspace);
    uint32_t *sums = parts + kEncParts;
    EncLevels lv;
    lv.n_levels = n_levels;
    for (int i = 0; i < IXH_MAX_LEVELS; ++i) lv.bits[i] = i < n_levels ? bits[i] : 0;
    hipLaunchKernelGGL(k_enc_absmax, dim3(kEncParts), dim3(256), 0, s, w, n, parts);
    switch (n_levels) {
        case 2: scan_launch<2>(w, n, n_units, parts, lv, scale, table, s); break;
        case 3: scan_launch<3>(w, n, n_units, parts, lv, scale, table, s); break;
        case 4: scan_launch<4>(w, n, n_units, parts, lv, scale, table, s); break;
        case 5: scan_launch<5>(w, n, n_units, parts, lv, scale, table, s); break;
        case 6: scan_launch<6>(w, n, n_units, parts, lv, scale, table, s); break;
        case 7: scan_launch<7>(w, n, n_units, parts, lv, scale, table, s); break;
        default: scan_launch<8>(w, n, n_units, parts, lv, scale, table, s); break;
    }
    const uint32_t tiles = max(1u, (n_units + kScanTile - 1) / kScanTile);
    if (n_units != 0)
        hipLaunchKernelGGL(k_enc_tile_sums, dim3(tiles, n_levels - 1), dim3(1024), 0, s, table, n_units, sums);
    hipLaunchKernelGGL(k_enc_scan, dim3(tiles, n_levels - 1), dim3(1024), 0, s, table, n_units, sums, totals, n);
    if (totals) hipLaunchKernelGGL(k_enc_last_total, dim3(1), dim3(64), 0, s, totals, n_levels, n, n_units);
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
    for (int i = 0; i < P.n_levels - 1; ++i) {
        if (out.bm_words[i])
            hipLaunchKernelGGL(k_enc_clear, dim3(min(2048u, (out.bm_words[i] + 255u) / 256u)), dim3(256), 0, s, out.bm[i],
                               out.bm_words[i]);
        if (out.st_words[i])
            hipLaunchKernelGGL(k_enc_clear, dim3(min(2048u, (out.st_words[i] + 255u) / 256u)), dim3(256), 0, s, out.st[i],
                               out.st_words[i]);
    }
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
