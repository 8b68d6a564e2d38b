// The matrix-pipe end of the level-by-level kernels for 2..16 activation rows on dense mixes, shared by the (3,5,8)
// and the (3,4,5,6,8) kernel: a workgroup of 16 waves takes 16 neighbouring weight rows, one per wave, span by span
// (2048 columns); every wave leaves its row's span in position order in its own LDS array (64 lane rows of 80 bytes,
// the layout the full decoders store from; the arrays REGION bytes apart, REGION = 16 mod 128, so that the 16 rows of
// a column start four banks apart).  After a barrier the 16 arrays are a 16 x 2048 tile, and wave w multiplies columns
// 128 w .. 128 w + 127 of it with four v_mfma_f32_16x16x32_bf16 (weights of row n, eight at a time, from wave n's
// array; eight activations of row a at the same columns, loaded from global memory while the span was decoded); a
// second barrier lets the arrays be overwritten.  The accumulators stay in registers from span to span; when the row
// block ends (or the workgroup's share of the work does) the 16 waves' accumulators are added in wave order through
// LDS and written as one piece of the block's partial sums, [piece][activation row][weight row] fp32, which
// k_reduce_chunks adds in piece order: the steps (row block, span) are dealt to the workgroups in equal contiguous
// shares, so a row block's spans may lie in two or more workgroups.
#pragma once
#include "ixh_fast358.h"

namespace ixh {

typedef uint32_t dt_u32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 dt_bf16x8 __attribute__((ext_vector_type(8)));
typedef float dt_f32x4 __attribute__((ext_vector_type(4)));

constexpr int kDtWaves = 16;
constexpr uint32_t kDtSpan = 2048;                          // columns per span
constexpr uint32_t kDtSumsBytes = kDtWaves * 256 * 4;       // [16 waves][16 activation rows][16 weight rows] fp32
extern std::atomic<int> g_opt_gemv_tile_cus;                // ixh_set_option("gemv_tile_cus")

// step `step` of the sequence (row block, span of the row): block rb, span k of the row
struct DtStep {
    uint32_t rb, k, step;
};

template <uint32_t REGION>
struct DtMfmaSink {
    static_assert(REGION % 128u == 16u, "the tile's rows must start four banks apart");
    const uint16_t *__restrict__ x;
    int64_t ldx;
    int m;
    float *__restrict__ ws;
    uint32_t out_f, in_f, spans_per_row, n_pieces, total_steps, step_end;
    uint32_t wave, lane;
    uint16_t *wc;        // this wave's array
    uint32_t tile_addr;  // LDS address of wave 0's array
    float *red;          // kDtSumsBytes of LDS
    dt_u32x4 xa[4];
    dt_f32x4 acc;

    // the workgroup that holds step t when `total_steps` steps are dealt to gridDim.x workgroups in contiguous shares
    __device__ __forceinline__ uint32_t group_of(uint32_t t) const {
        return (uint32_t)((((uint64_t)t + 1u) * gridDim.x + total_steps - 1u) / total_steps) - 1u;
    }
    // before the span's arithmetic: the activations this wave will multiply with (rows lane % 16, eight columns per k
    // group of each of its four 32-column steps) are asked for
    __device__ __forceinline__ void begin(const DtStep &st) {
        const uint32_t a = lane & 15u, kg = lane >> 4;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t col = st.k * kDtSpan + (wave * 4u + (uint32_t)j) * 32u + kg * 8u;
            xa[j] = dt_u32x4{0u, 0u, 0u, 0u};
            if (a < (uint32_t)m && col < in_f) {
                const uint4 v = *reinterpret_cast<const uint4 *>(x + (int64_t)a * ldx + col);
                xa[j] = dt_u32x4{v.x, v.y, v.z, v.w};
            }
        }
    }
    // o: the lane's 32 weights of the span in position order, as 16 bf16 pairs (lanes past the row's end: anything
    // finite; their activations are zero)
    // A barrier for LDS traffic only: this wave's LDS accesses have completed, nothing is said about global memory.
    // __syncthreads() carries a fence that waits for every load in flight, and here the next span's table entries,
    // bitmap words and code windows are in flight across both barriers of a span.
    static __device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }
    __device__ __forceinline__ void end(const DtStep &st, const uint32_t (&o)[16]) {
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
        dt_u32x4 *const rows = reinterpret_cast<dt_u32x4 *>(wc);
#pragma unroll
        for (int j = 0; j < 4; ++j) rows[lane * 5 + j] = dt_u32x4{o[4 * j], o[4 * j + 1], o[4 * j + 2], o[4 * j + 3]};
        lds_barrier();  // the tile is whole
        const uint32_t n = lane & 15u, kg = lane >> 4;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            // weight row n, columns 32 (4 wave + j) + 8 kg ..: lane row 4 wave + j of wave n's array, 16 bytes in
            const dt_u32x4 b = *reinterpret_cast<const __attribute__((address_space(3))) dt_u32x4 *>(
                (uintptr_t)(tile_addr + n * REGION + (wave * 4u + (uint32_t)j) * 80u + kg * 16u));
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(dt_bf16x8, xa[j]),
                                                         __builtin_bit_cast(dt_bf16x8, b), acc, 0, 0, 0);
        }
        lds_barrier();  // before any wave's next span overwrites its array
        const bool block_ends = st.k + 1 == spans_per_row;
        if (!block_ends && st.step + 1 != step_end) return;
        // ---- the block's sums so far leave: added over the waves in order, one piece per workgroup ----
#pragma unroll
        for (int i = 0; i < 4; ++i) red[wave * 256u + (4u * kg + (uint32_t)i) * 16u + n] = acc[i];
        acc = dt_f32x4{0.f, 0.f, 0.f, 0.f};
        __syncthreads();
        const uint32_t tid = wave * kWave + lane;
        if (tid < 256) {
            const uint32_t a = tid >> 4, row = st.rb * (uint32_t)kDtWaves + (tid & 15u);
            if (a < (uint32_t)m && row < out_f) {
                float sum = 0.0f;
#pragma unroll
                for (int w = 0; w < kDtWaves; ++w) sum += red[(uint32_t)w * 256u + tid];
                const uint32_t piece = blockIdx.x - group_of(st.rb * spans_per_row);
                ws[((size_t)piece * m + a) * out_f + row] = sum;
                if (block_ends)  // the pieces nobody writes
                    for (uint32_t q = piece + 1; q < n_pieces; ++q) ws[((size_t)q * m + a) * out_f + row] = 0.0f;
            }
        }
        __syncthreads();  // the sums are read before the next block's arrive
    }
};

// How the steps of a tensor are dealt: one workgroup per CU, fewer where the pieces of a row block would not fit the
// workspace of in_f / 512 pieces that ixh_gemv_workspace_bytes asks for (a block's spans lie in at most
// ceil(groups / blocks) + 1 workgroups).  groups == 0: the shape is not taken.
struct DtPlan {
    uint32_t n_chunks, spans_per_row, total_steps, groups, n_pieces;
};
inline DtPlan dt_plan(uint32_t out_f, uint32_t in_f, uint32_t n_cu) {
    DtPlan p{in_f / kFastChunk, 0, 0, 0, 0};
    p.spans_per_row = (p.n_chunks + 3) / 4;
    const uint32_t n_blocks = (out_f + kDtWaves - 1) / kDtWaves;
    const uint64_t total = (uint64_t)n_blocks * p.spans_per_row;
    if (total == 0 || total >= (1ull << 31) || p.n_chunks < 2) return p;
    const int cus_opt = g_opt_gemv_tile_cus.load(std::memory_order_relaxed);
    uint64_t groups = cus_opt > 0 ? (uint64_t)cus_opt : (uint64_t)n_cu;
    if (groups > total) groups = total;
    if (groups > (uint64_t)(p.n_chunks - 1u) * n_blocks) groups = (uint64_t)(p.n_chunks - 1u) * n_blocks;
    const uint32_t n_pieces = (uint32_t)((groups + n_blocks - 1) / n_blocks) + 1;
    if (n_pieces > p.n_chunks) return p;
    p.total_steps = (uint32_t)total;
    p.groups = (uint32_t)groups;
    p.n_pieces = n_pieces;
    return p;
}

}  // namespace ixh
