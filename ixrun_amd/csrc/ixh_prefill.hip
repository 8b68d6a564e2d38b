// Fused decode + GEMM for many activation rows (prefill): Y[m, n] = sum_k X[m, k] * W[n, k]
// with W decoded from the packed streams into LDS and multiplied on the matrix cores
// (v_mfma_f32_32x32x16_bf16, fp32 accumulate); the bf16 weight never reaches HBM.
// Any level scheme (2..8 levels).
//
// A workgroup of 8 waves owns 64 weight rows x up to 512 activation rows x one K slice
// (a run of 512-element table units; the 8 slices of a launch map to the 8 XCDs through
// blockIdx % 8, so that the X columns of a slice stay in one L2).  Per 512-wide unit
// column: every wave decodes 8 of the 64 rows (streams staged in LDS by DMA, two slots
// per wave so that the next row loads while this one is ranked: ixh_staged.h) into a
// 64 x 512 bf16 tile; then eight K steps of 64 follow, each copying a 512 x 64 X tile to
// LDS (prefetched into registers one step ahead) and issuing 16 MFMAs per wave
// (a wave owns 128 m x 32 n of the output).  Partial sums of the K slices go to an fp32
// workspace [slice][m][n] and a second kernel adds them in slice order and rounds to bf16.
#include "ixh_staged.h"

namespace ixh {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4p __attribute__((ext_vector_type(4)));

constexpr int kPWaves = 8;
constexpr uint32_t kPRows = 64;    // weight rows per workgroup
constexpr uint32_t kPMaxM = 512;   // activation rows per launch
constexpr uint32_t kPWStride = 520;  // bf16 per row of the weight tile (512 + pad: 260 words, = 4 mod 32 banks)
constexpr uint32_t kPXStride = 72;   // bf16 per row of the X tile (64 + pad: 36 words, = 4 mod 32 banks)
constexpr uint32_t kPSlices = 8;

__host__ __device__ constexpr uint32_t prefill_slot_bytes(int n_levels) {
    return ((staged_slot_words(n_levels) + 5u * (uint32_t)(n_levels - 1) + 1u) * 4u + 15u) & ~15u;  // spans + record
}
__host__ __device__ constexpr uint32_t prefill_lds_bytes(int n_levels) {
    return kPRows * kPWStride * 2u + kPMaxM * kPXStride * 2u + kPWaves * 2u * prefill_slot_bytes(n_levels);
}

template <int L>
__global__ void __launch_bounds__(kWave *kPWaves)
k_prefill(Dev P, const int32_t *__restrict__ prefix, uint32_t n_chunks, const uint16_t *__restrict__ x, uint32_t m_rows,
          int64_t ldx, float *__restrict__ ws) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    uint16_t *const wt = reinterpret_cast<uint16_t *>(smem);                                  // [64][520]
    uint16_t *const xt = reinterpret_cast<uint16_t *>(smem + kPRows * kPWStride * 2);         // [512][72]
    const uint32_t slots0 = (uint32_t)(uintptr_t)(lds_ptr_t)(smem + kPRows * kPWStride * 2 + kPMaxM * kPXStride * 2);

    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const uint32_t slice = blockIdx.x % kPSlices, tile = blockIdx.x / kPSlices;
    const uint32_t n0 = tile * kPRows;
    const uint32_t c_begin = slice * n_chunks / kPSlices, c_end = (slice + 1) * n_chunks / kPSlices;
    const uint32_t entries = P.out_f * n_chunks + 1;
    const float scale = bf16_bits_to_f32(*P.scale);

    const uint32_t my_slots = slots0 + wave * 2 * prefill_slot_bytes(L);

    // output tile of this wave: m in [128*wm, +128), n in [32*wn, +32)
    const uint32_t wn = wave & 1, wm = wave >> 1;
    f32x16 acc[4];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[t][r] = 0.0f;

    // rows of X beyond m_rows stay zero in the tile
    for (uint32_t i = tid; i < kPMaxM * kPXStride / 2; i += blockDim.x) reinterpret_cast<uint32_t *>(xt)[i] = 0u;

    // activation tile of one K step: thread t brings the 64 columns of row t
    const bool x_row = tid < m_rows;
    const uint16_t *x_base = x + (int64_t)(x_row ? tid : 0) * ldx;
    u32x4p xreg[8];
#define IXH_FETCH_X(k0)                                                                     \
    {                                                                                       \
        const u32x4p *p_ = reinterpret_cast<const u32x4p *>(x_base + (k0));                 \
        _Pragma("unroll") for (int t_ = 0; t_ < 8; ++t_) xreg[t_] = p_[t_]; \
    }

    // The streams of a row are copied one row ahead of its decode: two slots per wave, alternating; the
    // record of where the spans landed waits at the end of the slot.
    const uint32_t row_first = n0 + wave * 8;
    auto stage_row = [&](uint32_t row, uint32_t c, uint32_t which) {
        uint32_t q_lo[L - 1], q_hi[L - 1];
        const uint32_t u = row * n_chunks + c;
#pragma unroll
        for (int i = 0; i < L - 1; ++i) {
            q_lo[i] = (uint32_t)prefix[(size_t)i * entries + u];
            q_hi[i] = (uint32_t)prefix[(size_t)i * entries + u + 1];
        }
        StagedUnit<L> S;
        const uint32_t slot = my_slots + which * prefill_slot_bytes(L);
        stage_unit<L>(P, u, kStagedChunk, q_lo, q_hi, slot, lane, S);
        put_unit<L>(slot + staged_slot_words(L) * 4, lane, S);
    };
    if (c_begin < c_end && row_first < P.out_f) stage_row(row_first, c_begin, 0);

    for (uint32_t c = c_begin; c < c_end; ++c) {
        // ---- decode the 64 x 512 weight tile of unit column c: wave w takes rows 8w .. 8w+7 ----
        __syncthreads();  // the previous column's MFMAs are done with the weight tile
        IXH_FETCH_X(c * kStagedChunk);
#pragma unroll 1
        for (uint32_t j = 0; j < 8; ++j) {
            const uint32_t row = row_first + j;
            // row j's copies (issued one row ago) have landed once nothing is outstanding
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            if (j + 1 < 8 && row + 1 < P.out_f) stage_row(row + 1, c, (j + 1) & 1);
            uint16_t *wrow = wt + (wave * 8 + j) * kPWStride;
            if (row < P.out_f) {
                StagedUnit<L> S;
                get_unit<L>(my_slots + (j & 1) * prefill_slot_bytes(L) + staged_slot_words(L) * 4, S);
                uint32_t cnt[L - 1];
#pragma unroll
                for (int i = 0; i < L - 1; ++i) cnt[i] = S.cnt0[i];
                const uint32_t p_begin = (row * n_chunks + c) * kStagedChunk;
#pragma unroll 1
                for (uint32_t g = 0; g < kStagedChunk / kWave; ++g) {
                    const int v = decode64_lds<L>(P, S, p_begin + g * kWave, true, cnt);
                    wrow[g * kWave + lane] = (uint16_t)f32_to_bf16_bits((float)v * scale);
                }
            } else {
#pragma unroll 1
                for (uint32_t g = 0; g < kStagedChunk / kWave; ++g) wrow[g * kWave + lane] = 0;
            }
        }
        // first row of the next column, while the MFMAs run
        if (c + 1 < c_end && row_first < P.out_f) stage_row(row_first, c + 1, 0);

        // ---- eight K steps of 64 over the decoded tile ----
        for (uint32_t ks = 0; ks < 8; ++ks) {
            __syncthreads();  // weight tile written (ks == 0) / previous X tile consumed
            if (x_row) {
                u32x4p *dst = reinterpret_cast<u32x4p *>(xt + tid * kPXStride);
#pragma unroll
                for (int t = 0; t < 8; ++t) dst[t] = xreg[t];
            }
            if (ks + 1 < 8) IXH_FETCH_X(c * kStagedChunk + (ks + 1) * 64);
            __syncthreads();
#pragma unroll
            for (int kk = 0; kk < 4; ++kk) {
                const uint32_t kcol = 16 * kk + 8 * (lane >> 5);
                const bf16x8 b = *reinterpret_cast<const bf16x8 *>(wt + (32 * wn + (lane & 31)) * kPWStride + ks * 64 + kcol);
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const bf16x8 a = *reinterpret_cast<const bf16x8 *>(xt + (128 * wm + 32 * t + (lane & 31)) * kPXStride + kcol);
                    acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[t], 0, 0, 0);
                }
            }
        }
    }

    // ---- partial sums of this K slice: ws[slice][m][n] ----
    const uint32_t n = n0 + 32 * wn + (lane & 31);
    if (n < P.out_f) {
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const uint32_t m = 128 * wm + 32 * t + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                if (m < m_rows) ws[((size_t)slice * m_rows + m) * P.out_f + n] = acc[t][r];
            }
    }
}

// y[m][n] = bf16(sum over the K slices, in slice order)
__global__ void __launch_bounds__(256)
k_prefill_reduce(const float *__restrict__ ws, uint32_t m_rows, uint32_t out_f, uint16_t *__restrict__ y, int64_t ldy) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    const size_t total = (size_t)m_rows * out_f;
    if (i >= total) return;
    float v[kPSlices];
#pragma unroll
    for (uint32_t s = 0; s < kPSlices; ++s) v[s] = ws[s * total + i];
    float sum = 0.0f;
#pragma unroll
    for (uint32_t s = 0; s < kPSlices; ++s) sum += v[s];
    const uint32_t m = (uint32_t)(i / out_f), n = (uint32_t)(i - (size_t)m * out_f);
    y[(int64_t)m * ldy + n] = (uint16_t)f32_to_bf16_bits(sum);
}

size_t prefill_workspace_bytes(const Dev &P, uint32_t m_rows) {
    return (size_t)kPSlices * min(m_rows, kPMaxM) * P.out_f * sizeof(float);
}

bool prefill_supports(const Dev &P, const uint16_t *x, int64_t ldx) {
    return P.in_f % kStagedChunk == 0 && P.in_f / kStagedChunk >= kPSlices && ((uintptr_t)x & 15u) == 0 &&
           (ldx & 7) == 0 && ((uintptr_t)P.last & 3u) == 0 && P.n_levels >= 2 && P.n_levels <= IXH_MAX_LEVELS;
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
    for (uint32_t m0 = 0; m0 < m_rows; m0 += kPMaxM) {
        const uint32_t mb = min(kPMaxM, m_rows - m0);
        hipLaunchKernelGGL(k_prefill<L>, dim3(tiles * kPSlices), dim3(kWave * kPWaves), lds, s, P, prefix, n_chunks,
                           x + (int64_t)m0 * ldx, mb, ldx, ws);
        const size_t total = (size_t)mb * P.out_f;
        hipLaunchKernelGGL(k_prefill_reduce, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, ws, mb, P.out_f,
                           y + (int64_t)m0 * ldy, ldy);
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
