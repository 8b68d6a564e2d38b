// Device-side view of a packed tensor and the wave64 helpers shared by the
// gfx950 kernels.  Internal to the library; the public interface is
// include/ixhip.h.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "../../include/ixhip.h"

namespace ixh {

constexpr int kWave = 64;

// Kernel-argument form of IxhPacked: 32-bit lengths (N < 2^31 is checked at
// the C boundary) and the derived sizes the kernels need.
struct Dev {
    int n_levels;
    int bits[IXH_MAX_LEVELS];
    const uint32_t *bm[IXH_MAX_LEVELS - 1];
    uint32_t bm_words[IXH_MAX_LEVELS - 1];
    const uint32_t *st[IXH_MAX_LEVELS - 1];
    uint32_t st_words[IXH_MAX_LEVELS - 1];
    const uint8_t *last;
    uint32_t last_bytes;
    const uint16_t *scale;
    uint32_t out_f, in_f, n;
};

__device__ __forceinline__ uint32_t lanes_below(uint64_t mask) {
    return __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u));
}

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return __uint_as_float(h << 16); }

// round-to-nearest-even bf16 bit pattern of a finite fp32
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    return (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
}

// the reference's dequantisation: bf16(f32(v) * f32(scale)), returned as fp32
__device__ __forceinline__ float dequant(int v, float scale) {
    return bf16_bits_to_f32(f32_to_bf16_bits((float)v * scale));
}

// Where the dequantisation scale of an element comes from: the tensor's bf16 scale, or, for the group-scale
// sibling format (ixgs/quantize.py:56-61), the fp16 scale of the element's group of `group` consecutive elements.
struct GroupScales {
    const uint16_t *fp16;  // nullptr: per-tensor scale
    uint32_t group;
};

__device__ __forceinline__ float fp16_bits_to_f32(uint16_t h) { return (float)__builtin_bit_cast(_Float16, h); }

__device__ __forceinline__ float scale_of(const GroupScales &g, float tensor_scale, uint32_t p) {
    return g.fp16 ? fp16_bits_to_f32(g.fp16[p / g.group]) : tensor_scale;
}

__device__ __forceinline__ int threshold_of(int bits) { return (1 << (bits - 1)) - 1; }

// inclusive sum over the lanes at or below this one (DPP: shifts inside the 16-lane rows, then the two
// row broadcasts that carry the totals across rows)
__device__ __forceinline__ uint32_t wave_scan_inclusive(uint32_t v) {
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x111, 0xf, 0xf, true);   // row_shr:1
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x112, 0xf, 0xf, true);   // row_shr:2
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x114, 0xf, 0xf, true);   // row_shr:4
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x118, 0xf, 0xf, true);   // row_shr:8
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x142, 0xa, 0xf, false);  // row_bcast:15 into rows 1, 3
    v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x143, 0xc, 0xf, false);  // row_bcast:31 into rows 2, 3
    return v;
}


// Decode the 64 consecutive flat elements p0 .. p0+63 (one per lane; lanes with
// alive == false take no part).  cnt[i] is the number of level-i elements
// before p0 and is advanced past the group.  Works for any level scheme: lane
// ranks come from ballots, so there is no scan and no shared memory.
template <int L>
__device__ __forceinline__ int decode64(const Dev &P, uint32_t p0, bool alive, uint32_t (&cnt)[L - 1]) {
    int v = 0;
    uint32_t space = p0;  // rank, in the current level's index space, of the group's first element
#pragma unroll
    for (int i = 0; i < L - 1; ++i) {
        const uint64_t alive_mask = __ballot(alive);
        const uint32_t r = space + lanes_below(alive_mask);
        uint32_t bit = 0;
        if (alive && P.bm_words[i] != 0) {
            const uint32_t wi = min(r >> 5, P.bm_words[i] - 1);
            bit = (P.bm[i][wi] >> (r & 31)) & 1u;
        }
        const bool taken = alive && bit;
        const uint64_t taken_mask = __ballot(taken);
        if (taken && P.st_words[i] != 0) {
            const int b = P.bits[i];
            const uint64_t bitpos = (uint64_t)(cnt[i] + lanes_below(taken_mask)) * (uint32_t)b;
            const uint32_t wi = min((uint32_t)(bitpos >> 5), P.st_words[i] - 1);
            const uint32_t s = (uint32_t)bitpos & 31u;
            const uint32_t lo = P.st[i][wi];
            const uint32_t hi = (s + b > 32 && wi + 1 < P.st_words[i]) ? P.st[i][wi + 1] : 0u;
            const uint64_t both = ((uint64_t)hi << 32) | lo;
            v = (int)((uint32_t)(both >> s) & ((1u << b) - 1u)) - threshold_of(b);
        }
        alive = alive && !bit;
        space -= cnt[i];
        cnt[i] += (uint32_t)__popcll(taken_mask);
    }
    const uint64_t alive_mask = __ballot(alive);
    if (alive && P.last_bytes != 0) {
        const uint32_t r = min(space + lanes_below(alive_mask), P.last_bytes - 1);
        v = (int)P.last[r] - 127;
    }
    return v;
}

// ---- host-side launchers (one per translation unit of kernels) ----
int launch_prefix_build(const Dev &P, uint32_t chunk, int32_t *prefix, hipStream_t s);
int launch_decode(const Dev &P, const int32_t *prefix, uint32_t chunk, int8_t *o8, uint16_t *o16, GroupScales gs,
                  hipStream_t s);
int launch_gemv_generic(const Dev &P, const int32_t *prefix, uint32_t chunk, const uint16_t *x, int m,
                        int64_t ldx, uint16_t *y, int64_t ldy, float *y32, float *ws, bool atomic,
                        hipStream_t s);
bool gemv_staged_supports(const Dev &P, uint32_t chunk, const uint16_t *x, int64_t ldx);
int launch_gemv_staged(const Dev &P, const int32_t *prefix, const uint16_t *x, int m, int64_t ldx, uint16_t *y,
                       int64_t ldy, float *y32, float *ws, bool atomic, hipStream_t s);
bool decode_staged_supports(const Dev &P, uint32_t chunk, const int8_t *o8, const uint16_t *o16, GroupScales gs);
int launch_decode_staged(const Dev &P, const int32_t *prefix, uint16_t *o16, GroupScales gs, hipStream_t s);
size_t prefill_workspace_bytes(const Dev &P, uint32_t m_rows);
bool prefill_supports(const Dev &P, const uint16_t *x, int64_t ldx);
int launch_prefill(const Dev &P, const int32_t *prefix, const uint16_t *x, uint32_t m_rows, int64_t ldx, uint16_t *y,
                   int64_t ldy, float *ws, hipStream_t s);
size_t encode_workspace_bytes(uint64_t n, int n_levels);
int launch_encode_scan(const uint16_t *w, uint32_t n, int n_levels, const int *bits, uint16_t *scale, int32_t *table,
                       void *workspace, hipStream_t s);
int launch_encode_pack(const uint16_t *w, const Dev &P, const int32_t *table, hipStream_t s);
int launch_fill_u16(uint16_t *dst, uint32_t n, uint16_t value, hipStream_t s);
void set_error(const char *fmt, ...);

// Process-wide switches of ixh_set_option (testing and measurement; the defaults are what a caller gets).
enum DecodeKernel : int { kDecodeAuto = 0, kDecodeRows = 1, kDecodeDense = 2, kDecodeStaged = 3, kDecodeGeneric = 4 };
extern std::atomic<int> g_opt_decode_kernel;   // a DecodeKernel
extern std::atomic<int> g_opt_gemv_shared_x;   // most activation rows the shared-x row-block kernel serves (0..8)
extern std::atomic<int> g_opt_gemv_tiles;      // the tile kernel: -1 = never, 0 = where it pays, 1 = wherever it fits
extern std::atomic<int> g_opt_gemv_strips;     // the strip kernel: -1 = never, 0 = where it fits, 1..6 = with that many chains

}  // namespace ixh
