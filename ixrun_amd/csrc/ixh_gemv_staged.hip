// Fused decode + GEMV / skinny GEMM for any level scheme and any level mix, through
// LDS-staged streams.  A wave owns one piece of one weight row (a run of 512-element table
// units: the whole row, or 1/splits of it), copies each unit's spans of every stream into
// LDS by DMA a few units ahead (ring of slots, ixh_staged.h), decodes the unit into an LDS
// row (eight elements per lane) and multiplies it with the activations of its columns
// (16 bytes of x per lane and activation row, v_dot2_f32_bf16, fp32 accumulate).  Pieces of
// a row are combined in piece order through a workspace [piece][m][row], or added into the
// caller's fp32 vector with atomics.
#include "ixh_fast358.h"
#include "ixh_staged.h"

namespace ixh {

typedef __bf16 gs_bf16x2 __attribute__((ext_vector_type(2)));

constexpr int kGWaves = 4;
constexpr uint32_t kGRing = 4;

__host__ __device__ constexpr uint32_t gstaged_slot_bytes(int n_levels) {
    return ((staged_slot_words(n_levels) + 5u * (uint32_t)(n_levels - 1) + 1u) * 4u + 15u) & ~15u;  // spans + record
}
__host__ __device__ constexpr uint32_t gstaged_wave_bytes(int n_levels) {
    return kGRing * gstaged_slot_bytes(n_levels) + kStagedQueue * 2u + kStagedChunk * 2u;  // ring, queue, row
}

template <int N>
__device__ __forceinline__ void gwait_vmcnt() {
    static_assert(N >= 0 && N < 64, "s_waitcnt vmcnt holds 6 bits");
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

__device__ __forceinline__ float wave_sum(float v) {
    v += __uint_as_float((uint32_t)__builtin_amdgcn_update_dpp(0, (int)__float_as_uint(v), 0x111, 0xf, 0xf, true));
    v += __uint_as_float((uint32_t)__builtin_amdgcn_update_dpp(0, (int)__float_as_uint(v), 0x112, 0xf, 0xf, true));
    v += __uint_as_float((uint32_t)__builtin_amdgcn_update_dpp(0, (int)__float_as_uint(v), 0x114, 0xf, 0xf, true));
    v += __uint_as_float((uint32_t)__builtin_amdgcn_update_dpp(0, (int)__float_as_uint(v), 0x118, 0xf, 0xf, true));
    // lane 15 of every 16-lane row holds the row's sum; rows are added in row order
    return __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(v), 15)) +
           __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(v), 31)) +
           __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(v), 47)) +
           __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(v), 63));
}

enum : int { kGDirect = 0, kGAtomic = 1, kGWorkspace = 2 };

template <int L, int MT>
__global__ void __launch_bounds__(kWave *kGWaves)
k_gemv_staged(Dev P, const int32_t *__restrict__ prefix, uint32_t n_chunks, uint32_t splits,
              const uint16_t *__restrict__ x, int m, int64_t ldx, uint16_t *__restrict__ y, int64_t ldy,
              float *__restrict__ y32, float *__restrict__ ws, int out_mode) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    constexpr int kDma = staged_dma_count(L);
    static_assert((kGRing - 1) * kDma < 64, "ring too deep for the wait counter");
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const uint32_t piece = blockIdx.x * kGWaves + wave;
    const uint32_t row = piece / splits, split = piece - row * splits;
    if (row >= P.out_f) return;  // no barriers in this kernel
    const uint32_t c_begin = split * n_chunks / splits, c_end = (split + 1) * n_chunks / splits;
    const uint32_t total = c_end - c_begin;
    const uint32_t u_begin = row * n_chunks + c_begin, n_units = P.out_f * n_chunks;
    const uint32_t entries = n_units + 1;
    const float scale = bf16_bits_to_f32(*P.scale);

    uint8_t *const my_area = smem + wave * gstaged_wave_bytes(L);
    const uint32_t my_slots = (uint32_t)(uintptr_t)(lds_ptr_t)my_area;
    uint16_t *const queue = reinterpret_cast<uint16_t *>(my_area + kGRing * gstaged_slot_bytes(L));
    uint16_t *const wrow = queue + kStagedQueue;

    // units are staged in order; their table entries arrive one unit ahead (scalar loads)
    TableWalk<L> table;
    table.start(prefix, entries, u_begin);
    auto stage = [&](uint32_t t) {
        uint32_t q_lo[L - 1], q_hi[L - 1];
        table.next(q_lo, q_hi);
        StagedUnit<L> S;
        const uint32_t slot = my_slots + (t % kGRing) * gstaged_slot_bytes(L);
        stage_unit<L>(P, u_begin + t, kStagedChunk, q_lo, q_hi, slot, lane, S);
        put_unit<L>(slot + staged_slot_words(L) * 4, lane, S);
    };
    for (uint32_t t = 0; t < kGRing - 1 && t < total; ++t) stage(t);

    float acc[MT];
#pragma unroll
    for (int j = 0; j < MT; ++j) acc[j] = 0.0f;

    // The lane's eight activations per row of x travel one unit ahead of their use, in loads the compiler does
    // not see (it would wait for everything outstanding, copies included, before the first use): the wait below
    // counts them by hand.  Rows of x past m repeat row 0 so that every unit issues MT loads.
    staged_u32x4 x_a[MT], x_b[MT];
    auto load_x = [&](uint32_t t, staged_u32x4 (&xv)[MT]) {
        const uint16_t *xp = x + (size_t)(c_begin + min(t, total - 1)) * kStagedChunk + 8 * lane;
#pragma unroll
        for (int j = 0; j < MT; ++j) {
            const uint16_t *pj = xp + (int64_t)(j < m ? j : 0) * ldx;
            asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(xv[j]) : "v"(pj) : "memory");
        }
    };
    // one unit: x_cur was requested an iteration ago, x_nxt is requested now; the two buffers swap roles every
    // unit (no register is read while a load into it is in flight)
    auto unit = [&](uint32_t t, staged_u32x4 (&x_cur)[MT], staged_u32x4 (&x_nxt)[MT]) {
        load_x(t + 1, x_nxt);
        if (t + kGRing - 1 < total) stage(t + kGRing - 1);
        // Issued after x(t), in order: the copies of unit t+2 (one iteration ago), x(t+1), the copies of unit t+3.
        // Unit t's own copies are older than x(t).  Loads return in order, so once at most those remain
        // outstanding both have landed.
        const uint32_t after = min(kGRing - 1, total - 1 - t);
        if (after >= 3) gwait_vmcnt<2 * kDma + MT>();
        else if (after == 2) gwait_vmcnt<kDma + MT>();
        else gwait_vmcnt<MT>();
#pragma unroll
        for (int j = 0; j < MT; ++j) asm volatile("" : "+v"(x_cur[j]));  // uses of x(t) stay behind the wait
        const uint32_t u = u_begin + t;
        const uint32_t slot = my_slots + (t % kGRing) * gstaged_slot_bytes(L);
        StagedUnit<L> S;
        get_unit<L>(slot + staged_slot_words(L) * 4, S);
        decode_unit_lds<L>(P, S, u * kStagedChunk, kStagedChunk, [scale](uint32_t) { return scale; }, wrow, queue, lane);
        const staged_u32x4 w = *reinterpret_cast<const staged_u32x4 *>(wrow + 8 * lane);
        const uint32_t wk[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int j = 0; j < MT; ++j)
            if (j < m) {
                const uint32_t xk[4] = {x_cur[j].x, x_cur[j].y, x_cur[j].z, x_cur[j].w};
#pragma unroll
                for (int k = 0; k < 4; ++k)
                    acc[j] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(gs_bf16x2, wk[k]),
                                                             __builtin_bit_cast(gs_bf16x2, xk[k]), acc[j], false);
            }
    };
    load_x(0, x_a);
#pragma unroll 1
    for (uint32_t t = 0; t < total; t += 2) {
        unit(t, x_a, x_b);
        if (t + 1 < total) unit(t + 1, x_b, x_a);
    }
    gwait_vmcnt<0>();  // the last request for x writes registers: let it land before they are reused

#pragma unroll
    for (int j = 0; j < MT; ++j) {
        if (j >= m) break;
        const float sum = wave_sum(acc[j]);
        if (lane == 0) {
            if (out_mode == kGDirect) y[(int64_t)j * ldy + row] = (uint16_t)f32_to_bf16_bits(sum);
            else if (out_mode == kGAtomic) atomicAdd(y32 + (size_t)j * P.out_f + row, sum);
            else ws[((size_t)split * m + j) * P.out_f + row] = sum;
        }
    }
}

bool gemv_staged_supports(const Dev &P, uint32_t chunk, const uint16_t *x, int64_t ldx) {
    return chunk == kStagedChunk && P.in_f % kStagedChunk == 0 && ((uintptr_t)x & 15u) == 0 && (ldx & 7) == 0 &&
           ((uintptr_t)P.last & 3u) == 0 && P.n_levels >= 2 && P.n_levels <= IXH_MAX_LEVELS;
}

// pieces per row: enough waves to fill the chip several times over, at least four units per piece
static uint32_t gemv_staged_splits(const Dev &P, uint32_t n_chunks) {
    uint32_t splits = 1;
    while ((uint64_t)P.out_f * splits < 16384 && n_chunks / (splits * 2) >= 4) splits *= 2;
    return splits;
}

template <int L, int MT>
static void gemv_staged_launch(const Dev &P, const int32_t *prefix, uint32_t n_chunks, uint32_t splits,
                               const uint16_t *x, int m, int64_t ldx, uint16_t *y, int64_t ldy, float *y32, float *ws,
                               int out_mode, hipStream_t s) {
    const uint32_t pieces = P.out_f * splits;
    hipLaunchKernelGGL((k_gemv_staged<L, MT>), dim3((pieces + kGWaves - 1) / kGWaves), dim3(kWave * kGWaves),
                       kGWaves * gstaged_wave_bytes(L), s, P, prefix, n_chunks, splits, x, m, ldx, y, ldy, y32, ws,
                       out_mode);
}

template <int L>
static void gemv_staged_pick_m(const Dev &P, const int32_t *prefix, uint32_t n_chunks, uint32_t splits,
                               const uint16_t *x, int m, int64_t ldx, uint16_t *y, int64_t ldy, float *y32, float *ws,
                               int out_mode, hipStream_t s) {
    if (m == 1) gemv_staged_launch<L, 1>(P, prefix, n_chunks, splits, x, m, ldx, y, ldy, y32, ws, out_mode, s);
    else if (m == 2) gemv_staged_launch<L, 2>(P, prefix, n_chunks, splits, x, m, ldx, y, ldy, y32, ws, out_mode, s);
    else if (m <= 4) gemv_staged_launch<L, 4>(P, prefix, n_chunks, splits, x, m, ldx, y, ldy, y32, ws, out_mode, s);
    else if (m <= 8) gemv_staged_launch<L, 8>(P, prefix, n_chunks, splits, x, m, ldx, y, ldy, y32, ws, out_mode, s);
    else gemv_staged_launch<L, 16>(P, prefix, n_chunks, splits, x, m, ldx, y, ldy, y32, ws, out_mode, s);
}

// ws: at least splits * m * out_f floats (the n_chunks * m * out_f of ixh_gemv_workspace_bytes cover it)
int launch_gemv_staged(const Dev &P, const int32_t *prefix, const uint16_t *x, int m, int64_t ldx, uint16_t *y,
                       int64_t ldy, float *y32, float *ws, bool atomic, hipStream_t s) {
    const uint32_t n_chunks = P.in_f / kStagedChunk;
    if (P.out_f == 0 || n_chunks == 0) return IXH_OK;
    const uint32_t splits = gemv_staged_splits(P, n_chunks);
    const int out_mode = atomic ? kGAtomic : (splits == 1 ? kGDirect : kGWorkspace);
    switch (P.n_levels) {
#define IXH_CASE(LV) \
    case LV: gemv_staged_pick_m<LV>(P, prefix, n_chunks, splits, x, m, ldx, y, ldy, y32, ws, out_mode, s); break;
        IXH_CASE(2) IXH_CASE(3) IXH_CASE(4) IXH_CASE(5) IXH_CASE(6) IXH_CASE(7) IXH_CASE(8)
#undef IXH_CASE
        default: return IXH_EUNSUPPORTED;
    }
    if (hipGetLastError() != hipSuccess) return IXH_ELAUNCH;
    if (out_mode == kGWorkspace) return launch_reduce_chunks(ws, splits, m, P.out_f, y, ldy, s);
    return IXH_OK;
}

}  // namespace ixh
