// Full decode to bf16 through LDS-staged streams: every wave walks a contiguous run of
// 512-element table units, copies each unit's spans of every stream into LDS by DMA a few
// units ahead (ring of slots, ixh_staged.h), decodes the unit into an LDS row and stores it
// with one 16-byte write per lane.  The table entries of a unit arrive one unit ahead of its
// staging through scalar loads.  Needs the table at unit 512 and 16-byte aligned output.
#include "ixh_staged.h"

namespace ixh {

constexpr int kDWaves = 4;
constexpr uint32_t kDRing = 4;

__host__ __device__ constexpr uint32_t dstaged_slot_bytes(int n_levels) {
    return ((staged_slot_words(n_levels) + 5u * (uint32_t)(n_levels - 1) + 1u) * 4u + 15u) & ~15u;  // spans + record
}
__host__ __device__ constexpr uint32_t dstaged_wave_bytes(int n_levels) {
    return kDRing * dstaged_slot_bytes(n_levels) + kStagedQueue * 2u + kStagedChunk * 2u;  // ring, queue, row
}

template <int N>
__device__ __forceinline__ void dwait_vmcnt() {
    static_assert(N >= 0 && N < 64, "s_waitcnt vmcnt holds 6 bits");
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

template <int L>
__global__ void __launch_bounds__(kWave *kDWaves)
k_decode_staged(Dev P, const int32_t *__restrict__ prefix, uint32_t n_units, uint32_t units_per_wave,
                uint16_t *__restrict__ out, GroupScales gs) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    constexpr int kDma = staged_dma_count(L);
    static_assert((kDRing - 1) * kDma < 64, "ring too deep for the wait counter");
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const uint32_t u_begin = (blockIdx.x * kDWaves + wave) * units_per_wave;
    if (u_begin >= n_units) return;  // no barriers in this kernel
    const uint32_t total = min(units_per_wave, n_units - u_begin);
    const uint32_t entries = n_units + 1;
    const float scale = gs.fp16 ? 0.0f : bf16_bits_to_f32(*P.scale);

    uint8_t *const my_area = smem + wave * dstaged_wave_bytes(L);
    const uint32_t my_slots = (uint32_t)(uintptr_t)(lds_ptr_t)my_area;
    uint16_t *const queue = reinterpret_cast<uint16_t *>(my_area + kDRing * dstaged_slot_bytes(L));
    uint16_t *const row = queue + kStagedQueue;

    // units are staged in order; their table entries arrive one unit ahead (scalar loads)
    TableWalk<L> table;
    table.start(prefix, entries, u_begin);
    auto stage = [&](uint32_t t) {
        uint32_t q_lo[L - 1], q_hi[L - 1];
        table.next(q_lo, q_hi);
        StagedUnit<L> S;
        const uint32_t slot = my_slots + (t % kDRing) * dstaged_slot_bytes(L);
        stage_unit<L>(P, u_begin + t, kStagedChunk, q_lo, q_hi, slot, lane, S);
        put_unit<L>(slot + staged_slot_words(L) * 4, lane, S);
    };
    for (uint32_t t = 0; t < kDRing - 1 && t < total; ++t) stage(t);

#pragma unroll 1
    for (uint32_t t = 0; t < total; ++t) {
        if (t + kDRing - 1 < total) stage(t + kDRing - 1);
        // unit t has landed once at most the loads of the units staged after it are outstanding
        const uint32_t after = min(kDRing - 1, total - 1 - t);
        if (after >= 3) dwait_vmcnt<3 * kDma>();
        else if (after == 2) dwait_vmcnt<2 * kDma>();
        else if (after == 1) dwait_vmcnt<kDma>();
        else dwait_vmcnt<0>();
        const uint32_t u = u_begin + t;
        const uint32_t p_begin = u * kStagedChunk;
        const uint32_t n_el = min(kStagedChunk, P.n - p_begin);
        const uint32_t slot = my_slots + (t % kDRing) * dstaged_slot_bytes(L);
        StagedUnit<L> S;
        get_unit<L>(slot + staged_slot_words(L) * 4, S);
        decode_unit_lds<L>(P, S, p_begin, n_el,
                           [&](uint32_t e) { return scale_of(gs, scale, min(p_begin + e, P.n - 1)); }, row, queue, lane);
        const staged_u32x4 v = *reinterpret_cast<const staged_u32x4 *>(row + 8 * lane);
        if (8 * lane + 8 <= n_el) {
            *reinterpret_cast<staged_u32x4 *>(out + (size_t)p_begin + 8 * lane) = v;
        } else {
            for (uint32_t e = 8 * lane; e < n_el; ++e) out[(size_t)p_begin + e] = row[e];
        }
    }
}

bool decode_staged_supports(const Dev &P, uint32_t chunk, const int8_t *o8, const uint16_t *o16, GroupScales gs) {
    if (gs.fp16 && gs.group % 8u != 0) return false;  // a lane's eight elements share one scale
    return chunk == kStagedChunk && !o8 && o16 && ((uintptr_t)o16 & 15u) == 0 && ((uintptr_t)P.last & 3u) == 0 &&
           P.n_levels >= 2 && P.n_levels <= IXH_MAX_LEVELS && P.n >= kStagedChunk;
}

template <int L>
static int decode_staged_launch(const Dev &P, const int32_t *prefix, uint16_t *o16, GroupScales gs, hipStream_t s) {
    const uint32_t n_units = (uint32_t)(((uint64_t)P.n + kStagedChunk - 1) / kStagedChunk);
    // enough waves to fill the chip a few times over, each with a run long enough to keep its ring busy
    const uint32_t units_per_wave = max(8u, (n_units + 16383u) / 16384u);
    const uint32_t n_waves = (n_units + units_per_wave - 1) / units_per_wave;
    const uint32_t blocks = (n_waves + kDWaves - 1) / kDWaves;
    hipLaunchKernelGGL(k_decode_staged<L>, dim3(blocks), dim3(kWave * kDWaves), kDWaves * dstaged_wave_bytes(L), s, P,
                       prefix, n_units, units_per_wave, o16, gs);
    return hipGetLastError() == hipSuccess ? IXH_OK : IXH_ELAUNCH;
}

int launch_decode_staged(const Dev &P, const int32_t *prefix, uint16_t *o16, GroupScales gs, hipStream_t s) {
    switch (P.n_levels) {
        case 2: return decode_staged_launch<2>(P, prefix, o16, gs, s);
        case 3: return decode_staged_launch<3>(P, prefix, o16, gs, s);
        case 4: return decode_staged_launch<4>(P, prefix, o16, gs, s);
        case 5: return decode_staged_launch<5>(P, prefix, o16, gs, s);
        case 6: return decode_staged_launch<6>(P, prefix, o16, gs, s);
        case 7: return decode_staged_launch<7>(P, prefix, o16, gs, s);
        case 8: return decode_staged_launch<8>(P, prefix, o16, gs, s);
        default: return IXH_EUNSUPPORTED;
    }
}

}  // namespace ixh
