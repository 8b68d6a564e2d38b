// Fused decode + GEMM for many activation rows (prefill): Y[m, n] = sum_k X[m, k] * W[n, k]
// with W decoded from the packed streams into LDS and multiplied on the matrix cores
// (v_mfma_f32_32x32x16_bf16, fp32 accumulate); the bf16 weight never reaches HBM.
// Any level scheme (2..8 levels).
//
// A workgroup of 8 waves owns 32 weight rows x up to 512 activation rows x one K slice (a
// run of 512-element table units); two workgroups share a CU (four waves per SIMD), so
// that one decodes (VALU) while the other multiplies (MFMA, memory).  Per 512-wide unit
// column: every wave decodes 4 of the 32 rows into a 32 x 512 bf16 tile in LDS.  The
// streams of a row unit reach LDS by DMA a few row units ahead of their decode (a ring of
// slots per wave, ixh_staged.h), and the rank-table entries that say where the streams
// start are held in registers a column ahead, so that no decode waits on memory.  Then the
// waves multiply: a wave owns 64 m x 32 n of the output, takes the weight operand from
// the LDS tile and the activation operand straight from global memory (each lane's 16
// bytes are contiguous in a row of X, which is the MFMA operand layout), one block of
// 64 k ahead of the MFMAs.  Partial sums of the K slices go to an fp32 workspace
// [slice][m][n]; a second kernel adds them in slice order and rounds to bf16.  The number
// of K slices is chosen per shape so that the workgroups fill the CUs in whole rounds.
#include "ixh_prefill358.h"
#include "ixh_staged.h"

namespace ixh {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4p __attribute__((ext_vector_type(4)));

constexpr int kPWaves = 8;
constexpr uint32_t kPRows = 32;      // weight rows per workgroup
constexpr uint32_t kPMaxM = 512;     // activation rows per launch
constexpr uint32_t kPWStride = 520;  // bf16 per row of the weight tile (512 + pad: 260 words, = 4 mod 32 banks)
constexpr uint32_t kPMaxSlices = 16;
constexpr uint32_t kPRowsPerWave = kPRows / kPWaves;        // rows of the weight tile a wave decodes
constexpr uint32_t kPMTiles = kPMaxM / (32 * kPWaves);      // 32 x 32 output tiles of a wave
constexpr uint32_t kPWaveM = 32 * kPMTiles;                 // activation rows of a wave
// slots per wave: row units in flight ahead of the decode, plus one (fewer for the schemes with large slots, so
// that two workgroups fit a CU's LDS)
__host__ __device__ constexpr uint32_t prefill_ring(int n_levels) { return n_levels <= 5 ? 4u : 3u; }

__host__ __device__ constexpr uint32_t prefill_slot_bytes(int n_levels) {
    return ((staged_slot_words(n_levels) + 5u * (uint32_t)(n_levels - 1) + 1u) * 4u + 15u) & ~15u;  // spans + record
}
__host__ __device__ constexpr uint32_t prefill_wave_bytes(int n_levels) {
    return prefill_ring(n_levels) * prefill_slot_bytes(n_levels) + kStagedQueue * 2u;  // ring + queue of non-level-1 positions
}
__host__ __device__ constexpr uint32_t prefill_lds_bytes(int n_levels) {
    return kPRows * kPWStride * 2u + kPWaves * prefill_wave_bytes(n_levels);
}

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits for every vector-memory operation
// of the wave, which here would be the copies staged ahead for the next rows: they are private to the wave and
// need not have landed.
__device__ __forceinline__ void barrier_lds() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    static_assert(N >= 0 && N < 64, "s_waitcnt vmcnt holds 6 bits");
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// One unit column (512 k) of a wave's output tile: NT tiles of 32 m x 32 n.  Inside a block of 64 k the
// MFMA k index is permuted so that a lane's four operands of a block are 64 contiguous bytes of a row of X
// (lanes 0-31 take k 0..31 of the block, lanes 32-63 take k 32..63; step s uses the s-th 16 bytes): the four
// loads of a lane hit the same cache line back to back.  The weight operand follows the same permutation.
// An activation operand register is reloaded for the next block as soon as its MFMA has been issued.
template <int NT>
__device__ __forceinline__ void mfma_column(__amdgpu_buffer_rsrc_t x_rs, uint32_t x_off, uint32_t x_tile,
                                            const uint16_t *b_lane, f32x16 (&acc)[kPMTiles]) {
    u32x4p a[NT][4];
#pragma unroll
    for (int s = 0; s < 4; ++s)
#pragma unroll
        for (int t = 0; t < NT; ++t)
            a[t][s] = __builtin_amdgcn_raw_buffer_load_b128(x_rs, (int)(x_off + t * x_tile + s * 16), 0, 0);
#pragma unroll
    for (int blk = 0; blk < 8; ++blk) {
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const bf16x8 b = *reinterpret_cast<const bf16x8 *>(b_lane + blk * 64 + s * 8);
#pragma unroll
            for (int t = 0; t < NT; ++t)
                acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a[t][s]), b, acc[t], 0, 0, 0);
            if (blk + 1 < 8) {
#pragma unroll
                for (int t = 0; t < NT; ++t)
                    a[t][s] = __builtin_amdgcn_raw_buffer_load_b128(
                        x_rs, (int)(x_off + t * x_tile + (blk + 1) * 128 + s * 16), 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);  // keep the reloads here: the scheduler would sink them to their use
        }
    }
}

template <int L>
__global__ void __launch_bounds__(kWave *kPWaves, L <= 5 ? 4 : 2)  // four waves per SIMD (two workgroups per CU) where the registers allow
k_prefill(Dev P, const int32_t *__restrict__ prefix, uint32_t n_chunks, const uint16_t *__restrict__ x, uint32_t m_rows,
          int64_t ldx, float *__restrict__ ws, uint32_t n_slices) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    uint16_t *const wt = reinterpret_cast<uint16_t *>(smem);  // [64][520]
    constexpr int kDma = staged_dma_count(L);
    constexpr uint32_t kPRing = prefill_ring(L);
    static_assert((kPRing - 1) * kDma < 64, "ring too deep for the wait counter");

    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const uint32_t slice = blockIdx.x % n_slices, tile = blockIdx.x / n_slices;
    const uint32_t n0 = tile * kPRows;
    const uint32_t c_begin = slice * n_chunks / n_slices, c_end = (slice + 1) * n_chunks / n_slices;
    const uint32_t total = (c_end - c_begin) * kPRowsPerWave;  // row units this wave decodes
    const uint32_t entries = P.out_f * n_chunks + 1;
    const float scale = bf16_bits_to_f32(*P.scale);

    uint8_t *const my_area = smem + kPRows * kPWStride * 2 + wave * prefill_wave_bytes(L);
    const uint32_t my_slots = (uint32_t)(uintptr_t)(lds_ptr_t)my_area;
    uint16_t *const queue = reinterpret_cast<uint16_t *>(my_area + kPRing * prefill_slot_bytes(L));
    const uint32_t row_first = n0 + wave * kPRowsPerWave;

    // Rank-table entries in registers: lane 8 j + i holds, for row j of this wave and level i, the count before
    // unit column c (q0), c + 1 (q1), c + 2 (q2); the entry for c + 3 is fetched while column c is decoded.
    // Rows past the end of the tensor repeat the last row: their copies are made and thrown away, so that
    // every row unit issues the same number of loads.
    const uint32_t t_lev = lane & 7;
    const bool t_has = t_lev < (uint32_t)(L - 1);
    const int32_t *const t_base =
        prefix + (size_t)(t_has ? t_lev : 0) * entries + (size_t)min(row_first + (lane >> 3), P.out_f - 1) * n_chunks;
    auto table_at = [&](uint32_t cb) -> uint32_t { return t_has ? (uint32_t)t_base[min(cb, c_end)] : 0u; };
    uint32_t q0 = table_at(c_begin), q1 = table_at(c_begin + 1), q2 = table_at(c_begin + 2);

    // row unit t of this wave: column c_begin + t / 8, row t % 8; `ahead` says whether that column is the one
    // being decoded (q0, q1) or the next (q1, q2)
    auto stage_row = [&](uint32_t t, uint32_t c_now) {
        const uint32_t c = c_begin + t / kPRowsPerWave, j = t % kPRowsPerWave;
        const bool ahead = c != c_now;
        const uint32_t lo = ahead ? q1 : q0, hi = ahead ? q2 : q1;
        uint32_t q_lo[L - 1], q_hi[L - 1];
#pragma unroll
        for (int i = 0; i < L - 1; ++i) {
            q_lo[i] = (uint32_t)__builtin_amdgcn_readlane((int)lo, (int)(j * 8 + i));
            q_hi[i] = (uint32_t)__builtin_amdgcn_readlane((int)hi, (int)(j * 8 + i));
        }
        StagedUnit<L> S;
        const uint32_t slot = my_slots + (t % kPRing) * prefill_slot_bytes(L);
        stage_unit<L>(P, min(row_first + j, P.out_f - 1) * n_chunks + c, kStagedChunk, q_lo, q_hi, slot, lane, S);
        put_unit<L>(slot + staged_slot_words(L) * 4, lane, S);
    };
    for (uint32_t t = 0; t < kPRing - 1 && t < total; ++t) stage_row(t, c_begin);

    // output tile of this wave: m in [64 w, +64), the 32 n of the workgroup
    const uint32_t m_tiles = kPWaveM * wave < m_rows ? min(kPMTiles, (m_rows - kPWaveM * wave + 31) / 32) : 0u;
    f32x16 acc[kPMTiles];
#pragma unroll
    for (int t = 0; t < (int)kPMTiles; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[t][r] = 0.0f;
    // X through a buffer descriptor that ends with row m_rows - 1: rows past it read as zero
    const __amdgpu_buffer_rsrc_t x_rs = __builtin_amdgcn_make_buffer_rsrc(
        (void *)x, 0, (int)((((int64_t)m_rows - 1) * ldx + P.in_f) * 2), 0x00020000);
    const uint32_t x_lane = (uint32_t)(((int64_t)(kPWaveM * wave + (lane & 31)) * ldx + 32 * (lane >> 5)) * 2);
    const uint32_t x_tile = (uint32_t)(32 * ldx * 2);

    for (uint32_t c = c_begin; c < c_end; ++c) {
        const uint32_t q3 = table_at(c + 3);
        barrier_lds();  // the previous column's MFMAs are done with the weight tile
        // ---- decode the 64 x 512 weight tile of unit column c: wave w takes rows 8w .. 8w+7 ----
#pragma unroll 1
        for (uint32_t j = 0; j < kPRowsPerWave; ++j) {
            const uint32_t t = (c - c_begin) * kPRowsPerWave + j;
            if (t + kPRing - 1 < total) stage_row(t + kPRing - 1, c);
            // row unit t has landed once at most the loads of the units staged after it are outstanding
            const uint32_t after = min(kPRing - 1, total - 1 - t);
            if (after >= 3) wait_vmcnt<3 * kDma>();
            else if (after == 2) wait_vmcnt<2 * kDma>();
            else if (after == 1) wait_vmcnt<kDma>();
            else wait_vmcnt<0>();
            uint16_t *wrow = wt + (wave * kPRowsPerWave + j) * kPWStride;
            if (row_first + j < P.out_f) {
                const uint32_t slot = my_slots + (t % kPRing) * prefill_slot_bytes(L);
                StagedUnit<L> S;
                get_unit<L>(slot + staged_slot_words(L) * 4, S);
                decode_unit_lds<L>(P, S, ((row_first + j) * n_chunks + c) * kStagedChunk, kStagedChunk,
                                   [scale](uint32_t) { return scale; }, wrow,
                                   queue, lane);
            } else {
#pragma unroll 1
                for (uint32_t g = 0; g < kStagedChunk / kWave; ++g) wrow[g * kWave + lane] = 0;
            }
        }
        q0 = q1, q1 = q2, q2 = q3;
        barrier_lds();  // weight tile complete

        // ---- eight blocks of 64 k over the decoded tile ----
        const uint16_t *b_lane = wt + (lane & 31) * kPWStride + 32 * (lane >> 5);
        const uint32_t x_col = x_lane + c * (kStagedChunk * 2);
        switch (m_tiles) {
            case 2: mfma_column<2>(x_rs, x_col, x_tile, b_lane, acc); break;
            case 1: mfma_column<1>(x_rs, x_col, x_tile, b_lane, acc); break;
            default: break;
        }
    }

    // ---- partial sums of this K slice: ws[slice][m][n] ----
    const uint32_t n = n0 + (lane & 31);
    if (n < P.out_f) {
#pragma unroll
        for (int t = 0; t < (int)kPMTiles; ++t)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const uint32_t m = kPWaveM * wave + 32 * t + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                if (m < m_rows) ws[((size_t)slice * m_rows + m) * P.out_f + n] = acc[t][r];
            }
    }
}

// y[m][n] = bf16(sum over the K slices, in slice order)
__global__ void __launch_bounds__(256)
k_prefill_reduce(const float *__restrict__ ws, uint32_t m_rows, uint32_t out_f, uint32_t n_slices,
                 uint16_t *__restrict__ y, int64_t ldy) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    const size_t total = (size_t)m_rows * out_f;
    if (i >= total) return;
    float sum = 0.0f;
    uint32_t s = 0;
    for (; s + 4 <= n_slices; s += 4) {
        const float v0 = ws[s * total + i], v1 = ws[(s + 1) * total + i], v2 = ws[(s + 2) * total + i],
                    v3 = ws[(s + 3) * total + i];
        sum = (((sum + v0) + v1) + v2) + v3;
    }
    for (; s < n_slices; ++s) sum += ws[s * total + i];
    const uint32_t m = (uint32_t)(i / out_f), n = (uint32_t)(i - (size_t)m * out_f);
    y[(int64_t)m * ldy + n] = (uint16_t)f32_to_bf16_bits(sum);
}

int launch_prefill_reduce(const float *ws, uint32_t m_rows, uint32_t out_f, uint32_t n_slices, uint16_t *y, int64_t ldy,
                          hipStream_t s) {
    const size_t total = (size_t)m_rows * out_f;
    hipLaunchKernelGGL(k_prefill_reduce, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, ws, m_rows, out_f, n_slices,
                       y, ldy);
    return hipGetLastError() == hipSuccess ? IXH_OK : IXH_ELAUNCH;
}

// K slices for a shape: the count that makes rounds x (columns per workgroup + a start-up share) smallest,
// with two workgroups per CU.
static uint32_t pick_slices(uint32_t tiles, uint32_t n_chunks) {
    static int n_cu = 0;
    if (!n_cu) {
        int dev = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess) n_cu = prop.multiProcessorCount;
        if (n_cu <= 0) n_cu = 256;
    }
    const uint32_t slots = 2u * (uint32_t)n_cu;
    uint32_t best = 1;
    double best_cost = 1e30;
    for (uint32_t s = 1; s <= kPMaxSlices && s <= n_chunks; ++s) {
        const uint32_t cols = (n_chunks + s - 1) / s, rounds = (tiles * s + slots - 1) / slots;
        const double cost = rounds * (cols + 0.35) + 0.02 * s;  // the reduction reads one more slice
        if (cost < best_cost) best_cost = cost, best = s;
    }
    return best;
}

size_t prefill_workspace_bytes(const Dev &P, uint32_t m_rows) {
    return (size_t)kPMaxSlices * min(m_rows, kPMaxM) * P.out_f * sizeof(float);
}

bool prefill_supports(const Dev &P, const uint16_t *x, int64_t ldx) {
    return P.in_f % kStagedChunk == 0 && ((uintptr_t)x & 15u) == 0 &&
           (ldx & 7) == 0 && ldx < (1 << 20) && ((uintptr_t)P.last & 3u) == 0 && P.n_levels >= 2 && P.n_levels <= IXH_MAX_LEVELS;
}


template <int L>
static int prefill_launch(const Dev &P, const int32_t *prefix, const uint16_t *x, uint32_t m_rows, int64_t ldx,
                          uint16_t *y, int64_t ldy, float *ws, hipStream_t s) {
    static bool raised = false;
    const size_t lds = prefill_lds_bytes(L);
    if (!raised) {
        if (hipFuncSetAttribute(reinterpret_cast<const void *>(k_prefill<L>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)lds) != hipSuccess)
            return IXH_EUNSUPPORTED;
        raised = true;
    }
    const uint32_t n_chunks = P.in_f / kStagedChunk;
    const uint32_t tiles = (P.out_f + kPRows - 1) / kPRows;
    const uint32_t n_slices = pick_slices(tiles, n_chunks);
    for (uint32_t m0 = 0; m0 < m_rows; m0 += kPMaxM) {
        const uint32_t mb = min(kPMaxM, m_rows - m0);
        hipLaunchKernelGGL(k_prefill<L>, dim3(tiles * n_slices), dim3(kWave * kPWaves), lds, s, P, prefix, n_chunks,
                           x + (int64_t)m0 * ldx, mb, ldx, ws, n_slices);
        const size_t total = (size_t)mb * P.out_f;
        hipLaunchKernelGGL(k_prefill_reduce, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, ws, mb, P.out_f,
                           n_slices, y + (int64_t)m0 * ldy, ldy);
    }
    return hipGetLastError() == hipSuccess ? IXH_OK : IXH_ELAUNCH;
}

int launch_prefill(const Dev &P, const int32_t *prefix, const uint16_t *x, uint32_t m_rows, int64_t ldx, uint16_t *y,
                   int64_t ldy, float *ws, hipStream_t s) {
    switch (P.n_levels) {
        case 2: return prefill_launch<2>(P, prefix, x, m_rows, ldx, y, ldy, ws, s);
        case 3: return prefill_launch<3>(P, prefix, x, m_rows, ldx, y, ldy, ws, s);
        case 4: return prefill_launch<4>(P, prefix, x, m_rows, ldx, y, ldy, ws, s);
        case 5: return prefill_launch<5>(P, prefix, x, m_rows, ldx, y, ldy, ws, s);
        case 6: return prefill_launch<6>(P, prefix, x, m_rows, ldx, y, ldy, ws, s);
        case 7: return prefill_launch<7>(P, prefix, x, m_rows, ldx, y, ldy, ws, s);
        case 8: return prefill_launch<8>(P, prefix, x, m_rows, ldx, y, ldy, ws, s);
        default: return IXH_EUNSUPPORTED;
    }
}

}  // namespace ixh
