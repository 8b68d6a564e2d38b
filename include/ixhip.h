/*
 * ixhip -- C ABI of the gfx950 (MI355X) INT8-X decode / fused decode+GEMV library.
 *
 * The library replaces the three Triton kernels of dfytensor/ixrun and the
 * launch half of their Python wrappers.  Each entry point below names the
 * reference interface it stands in for (file:line in the reference tree).
 *
 * Conventions
 *   - every pointer inside IxhPacked and every buffer argument is a DEVICE
 *     pointer owned by the caller; the library never allocates, frees, copies
 *     to the host or synchronises, so every call may be stream-captured;
 *   - all work is enqueued on the given stream (0 = the null stream);
 *   - return value: IXH_OK (0) or a negative IXH_E* code; ixh_last_error()
 *     gives the calling thread's last message.  Nothing throws or aborts;
 *   - lengths of every stream are passed and respected: no kernel reads past
 *     them, whatever the level counts are (empty levels are legal);
 *   - int32 words of the reference's torch.int32 tensors are taken as raw
 *     32-bit patterns.
 */
#ifndef IXHIP_H
#define IXHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define IXH_MAX_LEVELS 8

#define IXH_OK 0
#define IXH_EINVAL (-1)       /* malformed argument (message says which) */
#define IXH_EUNSUPPORTED (-2) /* valid request this build has no kernel for */
#define IXH_ELAUNCH (-3)      /* the HIP runtime refused a launch */
#define IXH_EWORKSPACE (-4)   /* workspace missing or too small */

/* ixh_gemv flags */
#define IXH_GEMV_ATOMIC 1u /* add fp32 partials into y32 with atomics (caller zeroes y32) */
#define IXH_GEMV_FORCE_GENERIC 2u /* only the wave-per-unit kernel that gathers from global memory (testing / comparison) */
#define IXH_GEMV_COLUMN_KERNEL 4u /* of the (3,5,8) kernels, take the column-block one with the workspace */
#define IXH_GEMV_FORCE_358 8u /* use the (3,5,8) kernels even when less than 97 % of the elements are level 1 */
#define IXH_GEMV_STAGED 16u /* skip the (3,5,8) kernels: the any-scheme kernel that stages the streams in LDS */
#define IXH_GEMV_DENSE 32u /* (3,5,8) with M <= 8, (3,4,5,6,8) with M = 1: the level-by-level kernels even when almost all elements are level 1 */

typedef void *ixh_stream_t; /* a hipStream_t */

/*
 * One packed tensor: the device-resident fields of the dictionary written by
 * the reference's int8x_quantize (ixrun/quantize.py:110-122).
 *   level_bits  ascending code widths, last one 8 (quantize.py:55-58)
 *   bitmaps[i]  nested bitmap i, i < n_levels-1, 1 bit per element not in a
 *               lower level (quantize.py:91-96), LSB-first 32-bit words
 *   streams[i]  level-i codes, level_bits[i] bits each, LSB-first across
 *               32-bit words (bitpack.py:13-61), i < n_levels-1
 *   last        raw bytes of the 8-bit last level (quantize.py:84-86)
 *   scale       the bf16 per-tensor scale, read on the device
 */
typedef struct IxhPacked {
    int32_t n_levels;
    int32_t level_bits[IXH_MAX_LEVELS];
    int64_t out_f;
    int64_t in_f;
    const uint32_t *bitmaps[IXH_MAX_LEVELS - 1];
    uint64_t bitmap_words[IXH_MAX_LEVELS - 1];
    const uint32_t *streams[IXH_MAX_LEVELS - 1];
    uint64_t stream_words[IXH_MAX_LEVELS - 1];
    const uint8_t *last;
    uint64_t last_bytes;
    const uint16_t *scale;
} IxhPacked;

/* Library version (major*10000 + minor*100 + patch). */
int ixh_version(void);

/* Message of the last failing call on this thread ("" if none). */
const char *ixh_last_error(void);

/*
 * Number of int32 entries per level of a prefix table with the given chunk:
 * ceil(n / chunk) + 1.
 */
int64_t ixh_prefix_entries(int64_t n, int64_t chunk);

/*
 * Rank-prefix table, built on the device.
 *   prefix[i * entries + u] = number of level-i elements with flat index
 *   < min(u * chunk, N), for i < n_levels-1 and u = 0 .. entries-1.
 * chunk = in_f reproduces compute_row_prefixes(packed) (ixrun/fused.py:60-65),
 * a divisor of in_f reproduces compute_row_prefixes(packed, chunk)
 * (ixrun/fused.py:67-78), chunk = 1024 reproduces precompute_block_offsets
 * (ixrun/triton_kernels.py:180-220); the extra last entry holds the totals.
 */
int ixh_prefix_build(const IxhPacked *packed, int64_t chunk, int32_t *prefix, ixh_stream_t stream);

/*
 * Full decode: out_i8[p] = int8 value of flat element p (nullable),
 * out_bf16[p] = bf16(f32(v) * f32(scale)) (nullable).  Replaces
 * _ix_decode_kernel / decode_weight_triton (ixrun/triton_kernels.py:68-177,
 * :224-259) and StreamingLinear._decode (ixrun/engine.py:109-133), for any
 * level scheme.  prefix/chunk: a table from ixh_prefix_build; any chunk > 0.
 * Fastest with chunk = 512, bf16 output only and a 16-byte aligned out_bf16:
 * then one of three kernels that stage the streams through on-chip memory runs,
 * chosen from the tensor (a first level of 3 bits that holds 97 % or more of the
 * elements, with out_f * in_f a multiple of 2048: the row-block decoder; other
 * (3,5,8) tensors: the level-by-level decoder; any other scheme: the staged
 * decoder).  All kernels write the same bytes.
 */
int ixh_decode(const IxhPacked *packed, const int32_t *prefix, int64_t chunk, int8_t *out_i8,
               uint16_t *out_bf16, ixh_stream_t stream);

/*
 * Full decode of the group-scale sibling format ("ixgs"): the same (3,5,8) nested-bitmap
 * streams, but every run of group_size consecutive elements has its own fp16 scale:
 *   out_bf16[p] = bf16( f32(v[p]) * f32(group_scales[p / group_size]) ).
 * Replaces _ixgs_decode_kernel / decode_weight_triton (ixgs/kernels.py:30-105, :121-142)
 * and decode_weight_scatter (ixgs/quantize.py:113-151); the reference's per-element rank
 * tensors (ixgs/kernels.py:107-118, three int32 per weight) are replaced by the same
 * chunked rank table as ixh_decode.  packed->scale is not read and may be NULL; the codes
 * are offset by 3 / 15 / 127 exactly as in the per-tensor format, so values up to +128
 * (ixgs/quantize.py:63) decode correctly.  Fastest with chunk = 512, group_size a power of
 * two from 32 up (a multiple of 8 otherwise) and a 16-byte aligned out_bf16.
 */
int ixh_decode_gs(const IxhPacked *packed, const int32_t *prefix, int64_t chunk, const uint16_t *group_scales,
                  int64_t group_size, uint16_t *out_bf16, ixh_stream_t stream);

/*
 * Fused decode + GEMV / skinny GEMM:
 *   y[m, r] = bf16( sum_k f32(x[m, k]) * f32(bf16(f32(v[r, k]) * f32(scale))) ),
 * fp32 accumulation, m < M <= 16; x is bf16 [M, ldx], y is bf16 [M, ldy].
 * Replaces _ix_gemv_kernel / _ix_gemv_split_kernel / fused_gemv
 * (ixrun/fused.py:84-179, :209-294, :297-347) for M = 1 and the decode +
 * F.linear path of StreamingLinear.forward (ixrun/engine.py:171-173) for
 * 2 <= M <= 16.  chunk must divide in_f; the table must come from
 * ixh_prefix_build(packed, chunk); chunk = 512 with in_f a multiple of 512 and a
 * 16-byte aligned x is what the fast kernels take.  Partial sums of the pieces of
 * a row are combined in a fixed order through `workspace`
 * (ixh_gemv_workspace_bytes) and written to y, or, with IXH_GEMV_ATOMIC, added
 * into the caller-zeroed fp32 y32 [M, out_f] with atomics as the reference's
 * split kernel does (fused.py:294); y may then be NULL.  Kernels that own whole
 * rows add each output once, those whose workgroups share a block of rows once per
 * workgroup of the block (the same kernels as without the flag).
 */
int ixh_gemv(const IxhPacked *packed, const int32_t *prefix, int64_t chunk, const uint16_t *x,
             int32_t m, int64_t ldx, uint16_t *y, int64_t ldy, float *y32, void *workspace,
             size_t workspace_bytes, uint32_t flags, ixh_stream_t stream);

size_t ixh_gemv_workspace_bytes(const IxhPacked *packed, int64_t chunk, int32_t m, uint32_t flags);

/*
 * ixh_gemv for callers that cannot allocate device memory (code under stream capture, serving loops and
 * harnesses that forbid hipMalloc); it has no counterpart in the reference.  Same arguments, kernels and results
 * as ixh_gemv without IXH_GEMV_ATOMIC, but the partial sums of the kernels that need a workspace go to a buffer
 * of IXH_NOALLOC_WORKSPACE_BYTES that is part of the library's code object (every GPU the library runs on holds
 * it until the process ends).  The call allocates and frees nothing.  Where ixh_gemv_workspace_bytes asks for
 * more than the buffer holds, the kernels that need no workspace (a workgroup owns whole rows) still run, the tile
 * kernel divides a block of rows among as many workgroups as the buffer has room for (its sums are then added in
 * another order than ixh_gemv's with a full workspace), and a call that only a kernel with one piece per 512
 * columns can take fails with IXH_EWORKSPACE before anything is launched; IXH_GEMV_ATOMIC fails with IXH_EINVAL.  The device that
 * is current at the call must be the one the tensors live on; the first call on a device looks the buffer's
 * address up (make that call outside stream capture).  All calls on one GPU share the buffer: calls that may
 * overlap there (two streams, two threads) race on it and must be ordered by the caller.
 */
#define IXH_NOALLOC_WORKSPACE_BYTES (16u << 20)
int ixh_gemv_noalloc(const IxhPacked *packed, const int32_t *prefix, int64_t chunk, const uint16_t *x, int32_t m,
                     int64_t ldx, uint16_t *y, int64_t ldy, uint32_t flags, ixh_stream_t stream);

/*
 * Fused decode + GEMM for many activation rows (prefill, m > 16 in the reference's
 * dispatch): y[j, r] = bf16( sum_k f32(x[j, k]) * f32(w[r, k]) ) with
 * w = bf16(f32(v) * f32(scale)) decoded into on-chip memory tile by tile and multiplied
 * on the matrix cores (bf16 x bf16, fp32 accumulate).  Replaces the decode-to-bf16 +
 * F.linear pair of StreamingLinear.forward (ixrun/engine.py:171-173) and of
 * GraphLinear.forward (ixrun/engine.py:193-196), which materialise the whole bf16
 * weight in device memory first.  Any m >= 1; x is bf16 [m, ldx], y is bf16 [m, ldy].
 * The table must come from ixh_prefix_build(packed, 512).  Needs in_f a multiple of
 * 512, x 16-byte aligned with ldx a multiple of 8 and below 2^20, and the last-level
 * stream 4-byte aligned; otherwise IXH_EUNSUPPORTED (the caller then decodes with
 * ixh_decode and multiplies itself).  K is cut into up to 16 slices whose fp32 partial
 * sums are combined in slice order through `workspace` (ixh_gemm_workspace_bytes).
 */
int ixh_gemm(const IxhPacked *packed, const int32_t *prefix, const uint16_t *x, int32_t m, int64_t ldx,
             uint16_t *y, int64_t ldy, void *workspace, size_t workspace_bytes, ixh_stream_t stream);

size_t ixh_gemm_workspace_bytes(const IxhPacked *packed, int32_t m);

/*
 * The encoder on the device, in two calls because the stream lengths depend on the data.
 * Together they replace int8x_quantize (ixrun/quantize.py:41-122, with pack_bits_stream
 * and pack_bitmap of ixrun/bitpack.py:13-61, :87-89) for a bf16 weight that is already in
 * device memory, and write byte for byte what that CPU encoder writes; the rank table of
 * compute_row_prefixes(packed, 512) (ixrun/fused.py:67-78) comes out on the way.
 *
 * ixh_encode_scan: w is bf16 [out_f, in_f], contiguous.  Writes
 *   scale        bf16( max(max|w|, bf16(1e-8)) / 127 )                   (quantize.py:64)
 *   prefix       the chunk-512 rank table, (n_levels-1) rows of E = ixh_prefix_entries(N, 512)
 *                entries; the last entry of row i, prefix[i*E + E-1], is the number of level-i
 *                elements ("counts[i]"); the last level holds what is left of N
 * The caller reads those totals (its own synchronisation), then allocates, for i < n_levels-1,
 * bitmap i of ceil((N - counts[0] - .. - counts[i-1]) / 32) words and stream i of
 * ceil(counts[i] * level_bits[i] / 32) words, and counts[n_levels-1] bytes for the last level.
 *
 * ixh_encode_pack: dst names those buffers (they are WRITTEN, despite the const of the
 * struct's fields), the scale and the table written by ixh_encode_scan for the same w.
 * No write goes past the lengths given in dst.
 */
size_t ixh_encode_workspace_bytes(int64_t out_f, int64_t in_f, int32_t n_levels);

int ixh_encode_scan(const uint16_t *w, int64_t out_f, int64_t in_f, int32_t n_levels, const int32_t *level_bits,
                    uint16_t *scale, int32_t *prefix, void *workspace, size_t workspace_bytes,
                    ixh_stream_t stream);

int ixh_encode_pack(const uint16_t *w, const IxhPacked *dst, const int32_t *prefix, ixh_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* IXHIP_H */
