// Level-scheme-agnostic gfx950 kernels: rank-prefix tables, full decode and the
// general fused decode+GEMV.  One wave64 owns a run of consecutive flat
// elements and ranks them with ballots (decode64 in ixh_dev.h), so any number
// of levels, any chunk size and ragged tails are handled by the same code.
#include "ixh_dev.h"

namespace ixh {

constexpr int kWavesPerBlock = 4;

// ---------------------------------------------------------------------------
// Prefix tables.  Level i is counted after levels < i have been scanned, since
// unit u covers, in level i's index space, the bits
//   [min(u*chunk, n) - sum_{j<i} prefix[j][u],  the same at u+1).
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(kWave *kWavesPerBlock)
k_count_level(Dev P, int level, uint32_t chunk, uint32_t n_units, int32_t *prefix) {
    const uint32_t u = blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
    if (u >= n_units) return;
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t entries = n_units + 1;
    const uint64_t e0 = (uint64_t)u * chunk, e1 = e0 + chunk;
    uint32_t lo = (uint32_t)min(e0, (uint64_t)P.n), hi = (uint32_t)min(e1, (uint64_t)P.n);
    for (int j = 0; j < level; ++j) {
        lo -= (uint32_t)prefix[(size_t)j * entries + u];
        hi -= (uint32_t)prefix[(size_t)j * entries + u + 1];
    }
    const uint32_t words = P.bm_words[level];
    const uint32_t *bm = P.bm[level];
    uint32_t count = 0;
    if (hi > lo && words != 0) {
        const uint32_t w_first = lo >> 5, w_last = (hi - 1) >> 5;
        for (uint32_t w = w_first + lane; w <= w_last && w < words; w += kWave) {
            uint32_t bits = bm[w];
            if (w == w_first) bits &= ~0u << (lo & 31);
            if (w == w_last && ((hi & 31) != 0)) bits &= ~0u >> (32 - (hi & 31));
            count += __popc(bits);
        }
    }
    for (int off = 32; off > 0; off >>= 1) count += __shfl_xor(count, off);
    if (lane == 0) prefix[(size_t)level * entries + u + 1] = (int32_t)count;
}

// In place: row[0] = 0, row[u+1] = row[1] + ... + row[u+1], without a workspace, in three launches over tiles of
// kScanTile entries.  k_scan_tiles scans every tile by itself; the last entry of a tile then holds the tile's sum.
// k_scan_tile_ends (one workgroup) turns those last entries into their final values.  k_scan_tile_add adds the
// final value of the tile in front to every other entry of a tile: it reads only entries it never writes.
constexpr uint32_t kScanTile = 8192;

__global__ void __launch_bounds__(1024) k_scan_tiles(int32_t *row, uint32_t n_units) {
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    __shared__ uint32_t wave_s[16];
    const uint32_t first = blockIdx.x * kScanTile + tid * 8u;
    uint32_t v[8], mine = 0;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
        v[t] = first + t < n_units ? (uint32_t)row[first + t + 1] : 0u;
        mine += v[t];
    }
    const uint32_t incl = wave_scan_inclusive(mine);
    if (lane == 63) wave_s[wave] = incl;
    __syncthreads();
    uint32_t run = incl - mine;
    for (uint32_t k = 0; k < wave; ++k) run += wave_s[k];
#pragma unroll
    for (int t = 0; t < 8; ++t) {
        run += v[t];
        if (first + t < n_units) row[first + t + 1] = (int32_t)run;
    }
    if (blockIdx.x == 0 && tid == 0) row[0] = 0;
}

__global__ void __launch_bounds__(1024) k_scan_tile_ends(int32_t *row, uint32_t n_units, uint32_t tiles) {
    __shared__ uint32_t carry;
    __shared__ uint32_t wave_s[16];
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (tid == 0) carry = 0;
    __syncthreads();
    for (uint32_t base = 0; base < tiles; base += 1024) {
        const uint32_t t = base + tid;
        const uint32_t at = min((t + 1) * kScanTile, n_units);  // entry index of the tile's last unit, plus one
        const uint32_t mine = t < tiles ? (uint32_t)row[at] : 0u;
        const uint32_t incl = wave_scan_inclusive(mine);
        if (lane == 63) wave_s[wave] = incl;
        __syncthreads();
        uint32_t run = carry + incl;
        for (uint32_t k = 0; k < wave; ++k) run += wave_s[k];
        if (t < tiles) row[at] = (int32_t)run;
        __syncthreads();
        if (tid == 1023) carry = run;
        __syncthreads();
    }
}

__global__ void __launch_bounds__(1024) k_scan_tile_add(int32_t *row, uint32_t n_units) {
    const uint32_t tile = blockIdx.x + 1;  // the first tile is final already
    const uint32_t add = (uint32_t)row[tile * kScanTile];  // final value of the last entry of the tile in front
    const uint32_t last = min((tile + 1) * kScanTile, n_units);
    for (uint32_t e = tile * kScanTile + 1 + threadIdx.x; e < last; e += 1024) row[e] = (int32_t)((uint32_t)row[e] + add);
}

static void launch_scan_row(int32_t *row, uint32_t n_units, hipStream_t s) {
    const uint32_t tiles = max(1u, (n_units + kScanTile - 1) / kScanTile);
    hipLaunchKernelGGL(k_scan_tiles, dim3(tiles), dim3(1024), 0, s, row, n_units);
    if (tiles > 1) {
        hipLaunchKernelGGL(k_scan_tile_ends, dim3(1), dim3(1024), 0, s, row, n_units, tiles);
        hipLaunchKernelGGL(k_scan_tile_add, dim3(tiles - 1), dim3(1024), 0, s, row, n_units);
    }
}

int launch_prefix_build(const Dev &P, uint32_t chunk, int32_t *prefix, hipStream_t s) {
    const uint32_t n_units = (uint32_t)(((uint64_t)P.n + chunk - 1) / chunk);
    const uint32_t entries = n_units + 1;
    for (int i = 0; i < P.n_levels - 1; ++i) {
        if (n_units != 0) {
            const uint32_t blocks = (n_units + kWavesPerBlock - 1) / kWavesPerBlock;
            hipLaunchKernelGGL(k_count_level, dim3(blocks), dim3(kWave * kWavesPerBlock), 0, s, P, i, chunk,
                               n_units, prefix);
        }
        launch_scan_row(prefix + (size_t)i * entries, n_units, s);
    }
    return hipGetLastError() == hipSuccess ? IXH_OK : IXH_ELAUNCH;
}

// A plain fill, used instead of a memset so that every call stays capturable.
__global__ void __launch_bounds__(256) k_fill_u16(uint16_t *dst, uint32_t n, uint16_t value) {
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) dst[i] = value;
}

int launch_fill_u16(uint16_t *dst, uint32_t n, uint16_t value, hipStream_t s) {
    if (n == 0) return IXH_OK;
    hipLaunchKernelGGL(k_fill_u16, dim3((n + 255) / 256), dim3(256), 0, s, dst, n, value);
    return hipGetLastError() == hipSuccess ? IXH_OK : IXH_ELAUNCH;
}

// ---------------------------------------------------------------------------
// Full decode.  One wave per table unit.
// ---------------------------------------------------------------------------
template <int L>
__global__ void __launch_bounds__(kWave *kWavesPerBlock)
k_decode(Dev P, const int32_t *__restrict__ prefix, uint32_t chunk, uint32_t n_units,
         int8_t *__restrict__ o8, uint16_t *__restrict__ o16, GroupScales gs) {
    const uint32_t u = blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
    if (u >= n_units) return;
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t entries = n_units + 1;
    uint32_t cnt[L - 1];
#pragma unroll
    for (int i = 0; i < L - 1; ++i) cnt[i] = (uint32_t)prefix[(size_t)i * entries + u];
    const float scale = gs.fp16 ? 0.0f : bf16_bits_to_f32(*P.scale);
    const uint64_t e0 = (uint64_t)u * chunk;
    const uint32_t p_begin = (uint32_t)e0;
    const uint32_t p_end = (uint32_t)min(e0 + chunk, (uint64_t)P.n);
    for (uint32_t p0 = p_begin; p0 < p_end; p0 += kWave) {
        const bool alive = p0 + lane < p_end;
        const int v = decode64<L>(P, p0, alive, cnt);
        if (alive) {
            if (o8) o8[p0 + lane] = (int8_t)v;
            if (o16) o16[p0 + lane] = (uint16_t)f32_to_bf16_bits((float)v * scale_of(gs, scale, p0 + lane));
        }
    }
}

template <int L>
static void decode_launch(const Dev &P, const int32_t *prefix, uint32_t chunk, uint32_t n_units, int8_t *o8,
                          uint16_t *o16, GroupScales gs, hipStream_t s) {
    const uint32_t blocks = (n_units + kWavesPerBlock - 1) / kWavesPerBlock;
    hipLaunchKernelGGL(k_decode<L>, dim3(blocks), dim3(kWave * kWavesPerBlock), 0, s, P, prefix, chunk, n_units,
                       o8, o16, gs);
}

int launch_decode(const Dev &P, const int32_t *prefix, uint32_t chunk, int8_t *o8, uint16_t *o16, GroupScales gs,
                  hipStream_t s) {
    const uint32_t n_units = (uint32_t)(((uint64_t)P.n + chunk - 1) / chunk);
    if (n_units == 0) return IXH_OK;
    switch (P.n_levels) {
        case 2: decode_launch<2>(P, prefix, chunk, n_units, o8, o16, gs, s); break;
        case 3: decode_launch<3>(P, prefix, chunk, n_units, o8, o16, gs, s); break;
        case 4: decode_launch<4>(P, prefix, chunk, n_units, o8, o16, gs, s); break;
        case 5: decode_launch<5>(P, prefix, chunk, n_units, o8, o16, gs, s); break;
        case 6: decode_launch<6>(P, prefix, chunk, n_units, o8, o16, gs, s); break;
        case 7: decode_launch<7>(P, prefix, chunk, n_units, o8, o16, gs, s); break;
        case 8: decode_launch<8>(P, prefix, chunk, n_units, o8, o16, gs, s); break;
        default: set_error("n_levels %d not in 2..8", P.n_levels); return IXH_EINVAL;
    }
    return hipGetLastError() == hipSuccess ? IXH_OK : IXH_ELAUNCH;
}

// ---------------------------------------------------------------------------
// General fused decode + GEMV.  One wave per (row, chunk) unit; MT is the
// compiled row capacity of x (m <= MT rows are live).
// ---------------------------------------------------------------------------
enum : int { kOutDirect = 0, kOutAtomic = 1, kOutWorkspace = 2 };

template <int L, int MT>
__global__ void __launch_bounds__(kWave *kWavesPerBlock)
k_gemv_generic(Dev P, const int32_t *__restrict__ prefix, uint32_t chunk, uint32_t n_chunks,
               const uint16_t *__restrict__ x, int m, int64_t ldx, uint16_t *__restrict__ y, int64_t ldy,
               float *__restrict__ y32, float *__restrict__ ws, int out_mode) {
    const uint32_t n_units = P.out_f * n_chunks;
    const uint32_t u = blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
    if (u >= n_units) return;
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t entries = n_units + 1;
    const uint32_t row = u / n_chunks, c = u - row * n_chunks;
    uint32_t cnt[L - 1];
#pragma unroll
    for (int i = 0; i < L - 1; ++i) cnt[i] = (uint32_t)prefix[(size_t)i * entries + u];
    const float scale = bf16_bits_to_f32(*P.scale);
    const uint32_t p_begin = u * chunk;  // = row * in_f + c * chunk
    const uint32_t k_begin = c * chunk;
    float acc[MT];
#pragma unroll
    for (int j = 0; j < MT; ++j) acc[j] = 0.0f;

    for (uint32_t off = 0; off < chunk; off += kWave) {
        const bool alive = off + lane < chunk;
        const int v = decode64<L>(P, p_begin + off, alive, cnt);
        if (alive) {
            const float w = dequant(v, scale);
            const uint32_t k = k_begin + off + lane;
#pragma unroll
            for (int j = 0; j < MT; ++j)
                if (j < m) acc[j] = fmaf(bf16_bits_to_f32(x[(int64_t)j * ldx + k]), w, acc[j]);
        }
    }
#pragma unroll
    for (int j = 0; j < MT; ++j)
        for (int o = 32; o > 0; o >>= 1) acc[j] += __shfl_xor(acc[j], o);
    if (lane == 0) {
#pragma unroll
        for (int j = 0; j < MT; ++j) {
            if (j >= m) break;
            if (out_mode == kOutDirect)
                y[(int64_t)j * ldy + row] = (uint16_t)f32_to_bf16_bits(acc[j]);
            else if (out_mode == kOutAtomic)
                atomicAdd(&y32[(size_t)j * P.out_f + row], acc[j]);
            else
                ws[((size_t)c * m + j) * P.out_f + row] = acc[j];
        }
    }
}

// y[j][row] = bf16(sum over chunks, in chunk order)
__global__ void __launch_bounds__(256)
k_reduce_chunks(const float *__restrict__ ws, uint32_t n_chunks, int m, uint32_t out_f,
                uint16_t *__restrict__ y, int64_t ldy) {
    const uint32_t row = blockIdx.x * 256 + threadIdx.x;
    const int j = blockIdx.y;
    if (row >= out_f) return;
    // sixteen loads in flight at a time (the pieces come from memory, written by other workgroups: one after the other
    // they cost a trip each), the last ones past the end clamped to the last piece and left out of the sum; the additions
    // stay in chunk order
    const size_t stride = (size_t)m * out_f;
    const float *p = ws + (size_t)j * out_f + row;
    float sum = 0.0f;
    for (uint32_t c = 0; c < n_chunks; c += 16) {
        float v[16];
#pragma unroll
        for (uint32_t k = 0; k < 16; ++k) v[k] = p[(size_t)min(c + k, n_chunks - 1u) * stride];
#pragma unroll
        for (uint32_t k = 0; k < 16; ++k)
            if (c + k < n_chunks) sum += v[k];
    }
    y[(int64_t)j * ldy + row] = (uint16_t)f32_to_bf16_bits(sum);
}

int launch_reduce_chunks(const float *ws, uint32_t n_chunks, int m, uint32_t out_f, uint16_t *y, int64_t ldy,
                         hipStream_t s) {
    hipLaunchKernelGGL(k_reduce_chunks, dim3((out_f + 255) / 256, m), dim3(256), 0, s, ws, n_chunks, m, out_f, y,
                       ldy);
    return hipGetLastError() == hipSuccess ? IXH_OK : IXH_ELAUNCH;
}

template <int L, int MT>
static void gemv_launch(const Dev &P, const int32_t *prefix, uint32_t chunk, uint32_t n_chunks,
                        const uint16_t *x, int m, int64_t ldx, uint16_t *y, int64_t ldy, float *y32, float *ws,
                        int out_mode, hipStream_t s) {
    const uint32_t n_units = P.out_f * n_chunks;
    const uint32_t blocks = (n_units + kWavesPerBlock - 1) / kWavesPerBlock;
    hipLaunchKernelGGL((k_gemv_generic<L, MT>), dim3(blocks), dim3(kWave * kWavesPerBlock), 0, s, P, prefix, chunk,
                       n_chunks, x, m, ldx, y, ldy, y32, ws, out_mode);
}

template <int L>
static void gemv_pick_m(const Dev &P, const int32_t *prefix, uint32_t chunk, uint32_t n_chunks,
                        const uint16_t *x, int m, int64_t ldx, uint16_t *y, int64_t ldy, float *y32, float *ws,
                        int out_mode, hipStream_t s) {
    if (m == 1) gemv_launch<L, 1>(P, prefix, chunk, n_chunks, x, m, ldx, y, ldy, y32, ws, out_mode, s);
    else if (m == 2) gemv_launch<L, 2>(P, prefix, chunk, n_chunks, x, m, ldx, y, ldy, y32, ws, out_mode, s);
    else if (m <= 4) gemv_launch<L, 4>(P, prefix, chunk, n_chunks, x, m, ldx, y, ldy, y32, ws, out_mode, s);
    else if (m <= 8) gemv_launch<L, 8>(P, prefix, chunk, n_chunks, x, m, ldx, y, ldy, y32, ws, out_mode, s);
    else gemv_launch<L, 16>(P, prefix, chunk, n_chunks, x, m, ldx, y, ldy, y32, ws, out_mode, s);
}

int launch_gemv_generic(const Dev &P, const int32_t *prefix, uint32_t chunk, const uint16_t *x, int m,
                        int64_t ldx, uint16_t *y, int64_t ldy, float *y32, float *ws, bool atomic,
                        hipStream_t s) {
    const uint32_t n_chunks = P.in_f / chunk;
    if (P.out_f == 0 || P.in_f == 0) return IXH_OK;
    const int out_mode = atomic ? kOutAtomic : (n_chunks == 1 ? kOutDirect : kOutWorkspace);
#define IXH_CASE(LV) \
    case LV: gemv_pick_m<LV>(P, prefix, chunk, n_chunks, x, m, ldx, y, ldy, y32, ws, out_mode, s); break;
    switch (P.n_levels) {
        IXH_CASE(2) IXH_CASE(3) IXH_CASE(4) IXH_CASE(5) IXH_CASE(6) IXH_CASE(7) IXH_CASE(8)
        default: set_error("n_levels %d not in 2..8", P.n_levels); return IXH_EINVAL;
    }
#undef IXH_CASE
    if (hipGetLastError() != hipSuccess) return IXH_ELAUNCH;
    if (out_mode == kOutWorkspace) return launch_reduce_chunks(ws, n_chunks, m, P.out_f, y, ldy, s);
    return IXH_OK;
}

}  // namespace ixh
