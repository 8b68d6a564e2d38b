// C boundary of the library: argument checks, kernel selection, error text.
// Declarations and the reference interfaces they replace: include/ixhip.h; the testing hook: include/ixhip_test.h.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <cstdlib>
#include <mutex>

#include "../../include/ixhip_test.h"
#include "ixh_dev.h"
#include "ixh_fast358.h"
#include "ixh_prefill358.h"

namespace ixh {

static thread_local char g_error[512] = "";

std::atomic<int> g_opt_decode_kernel{kDecodeAuto};
std::atomic<int> g_opt_gemv_shared_x{8};
std::atomic<int> g_opt_gemv_strips{0};
std::atomic<int> g_opt_gemv_tiles{0};
std::atomic<int> g_opt_gemv_tile_rows{0};
std::atomic<int> g_opt_gemv_tile_cus{0};
std::atomic<int> g_opt_gemv_tile_split{0};
std::atomic<int> g_opt_gemv_dense_tiles{0};
std::atomic<int> g_opt_gemm_tiles{0};
extern std::atomic<int> g_opt_gemv_slots;
extern std::atomic<int> g_opt_gemv_slot_waves;

void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

// Validate an IxhPacked and turn it into the kernel-argument form.
static int to_dev(const IxhPacked *pk, Dev *out, bool need_scale = true) {
    if (!pk) { set_error("packed is NULL"); return IXH_EINVAL; }
    const int L = pk->n_levels;
    if (L < 2 || L > IXH_MAX_LEVELS) { set_error("n_levels %d not in 2..%d", L, IXH_MAX_LEVELS); return IXH_EINVAL; }
    if (pk->level_bits[L - 1] != 8) { set_error("last level must be 8-bit, got %d", pk->level_bits[L - 1]); return IXH_EINVAL; }
    for (int i = 0; i < L - 1; ++i) {
        const int b = pk->level_bits[i];
        if (b < 1 || b > 7 || (i > 0 && b < pk->level_bits[i - 1])) {
            set_error("level_bits[%d] = %d: widths must ascend within 1..7 before the final 8", i, b);
            return IXH_EINVAL;
        }
    }
    if (pk->out_f < 0 || pk->in_f < 0) { set_error("negative shape"); return IXH_EINVAL; }
    const uint64_t n = (uint64_t)pk->out_f * (uint64_t)pk->in_f;
    if (n >= (1ull << 31)) { set_error("out_f * in_f = %llu does not fit the 31-bit rank tables", (unsigned long long)n); return IXH_EINVAL; }
    if (n != 0 && need_scale && !pk->scale) { set_error("scale is NULL"); return IXH_EINVAL; }
    Dev d;
    memset(&d, 0, sizeof(d));
    d.n_levels = L;
    d.out_f = (uint32_t)pk->out_f;
    d.in_f = (uint32_t)pk->in_f;
    d.n = (uint32_t)n;
    for (int i = 0; i < L; ++i) d.bits[i] = pk->level_bits[i];
    for (int i = 0; i < L - 1; ++i) {
        if (pk->bitmap_words[i] >= (1ull << 31) || pk->stream_words[i] >= (1ull << 31)) {
            set_error("stream %d longer than 2^31 words", i);
            return IXH_EINVAL;
        }
        if ((pk->bitmap_words[i] && !pk->bitmaps[i]) || (pk->stream_words[i] && !pk->streams[i])) {
            set_error("level %d: non-empty stream with NULL pointer", i);
            return IXH_EINVAL;
        }
        d.bm[i] = pk->bitmaps[i];
        d.bm_words[i] = (uint32_t)pk->bitmap_words[i];
        d.st[i] = pk->streams[i];
        d.st_words[i] = (uint32_t)pk->stream_words[i];
    }
    if (pk->last_bytes >= (1ull << 31)) { set_error("last stream longer than 2^31 bytes"); return IXH_EINVAL; }
    if (pk->last_bytes && !pk->last) { set_error("last stream non-empty with NULL pointer"); return IXH_EINVAL; }
    // bitmap 0 must cover every element; shorter would make the kernels read past it
    if (d.bm_words[0] < (d.n + 31u) / 32u) {
        set_error("bitmap 0 has %u words, %u elements need %u", d.bm_words[0], d.n, (d.n + 31u) / 32u);
        return IXH_EINVAL;
    }
    d.last = pk->last;
    d.last_bytes = (uint32_t)pk->last_bytes;
    d.scale = pk->scale;
    *out = d;
    return IXH_OK;
}

static bool is_358(const Dev &d) { return d.n_levels == 3 && d.bits[0] == 3 && d.bits[1] == 5 && d.bits[2] == 8; }

}  // namespace ixh

using namespace ixh;

extern "C" {

int ixh_version(void) { return 100; }

const char *ixh_last_error(void) { return g_error; }

int ixh_set_option(const char *name, int64_t value) {
    if (!name) { set_error("option name is NULL"); return IXH_EINVAL; }
    if (strcmp(name, "decode_kernel") == 0) {
        if (value < kDecodeAuto || value > kDecodeGeneric) { set_error("decode_kernel %lld not in 0..4", (long long)value); return IXH_EINVAL; }
        g_opt_decode_kernel.store((int)value, std::memory_order_relaxed);
        return IXH_OK;
    }
    if (strcmp(name, "gemv_shared_x") == 0) {
        if (value < 0 || value > 8) { set_error("gemv_shared_x %lld not in 0..8", (long long)value); return IXH_EINVAL; }
        g_opt_gemv_shared_x.store((int)value, std::memory_order_relaxed);
        return IXH_OK;
    }
    if (strcmp(name, "gemv_tiles") == 0) {
        if (value < -1 || value > 1) { set_error("gemv_tiles %lld not in -1..1", (long long)value); return IXH_EINVAL; }
        g_opt_gemv_tiles.store((int)value, std::memory_order_relaxed);
        return IXH_OK;
    }
    if (strcmp(name, "gemv_tile_rows") == 0) {
        if (value != 0 && value != 2 && value != 3 && value != 4) { set_error("gemv_tile_rows %lld not 0, 2, 3 or 4", (long long)value); return IXH_EINVAL; }
        g_opt_gemv_tile_rows.store((int)value, std::memory_order_relaxed);
        return IXH_OK;
    }
    if (strcmp(name, "gemv_tile_split") == 0) {
        if (value < 0 || value > 8) { set_error("gemv_tile_split %lld not in 0..8", (long long)value); return IXH_EINVAL; }
        g_opt_gemv_tile_split.store((int)value, std::memory_order_relaxed);
        return IXH_OK;
    }
    if (strcmp(name, "gemv_tile_cus") == 0) {
        if (value < 0 || value > 4096) { set_error("gemv_tile_cus %lld not in 0..4096", (long long)value); return IXH_EINVAL; }
        g_opt_gemv_tile_cus.store((int)value, std::memory_order_relaxed);
        return IXH_OK;
    }
    if (strcmp(name, "gemv_dense_tiles") == 0) {
        if (value < -1 || value > 1) { set_error("gemv_dense_tiles %lld not in -1..1", (long long)value); return IXH_EINVAL; }
        g_opt_gemv_dense_tiles.store((int)value, std::memory_order_relaxed);
        return IXH_OK;
    }
    if (strcmp(name, "gemm_tiles") == 0) {
        if (value < -1 || value > 2) { set_error("gemm_tiles %lld not in -1..2", (long long)value); return IXH_EINVAL; }
        g_opt_gemm_tiles.store((int)value, std::memory_order_relaxed);
        return IXH_OK;
    }
    if (strcmp(name, "gemv_slots") == 0) {
        if (value < -1 || value > 1) { set_error("gemv_slots %lld not in -1..1", (long long)value); return IXH_EINVAL; }
        g_opt_gemv_slots.store((int)value, std::memory_order_relaxed);
        return IXH_OK;
    }
    if (strcmp(name, "gemv_slot_waves") == 0) {
        if (value != 0 && (value < 8 || value > 16)) { set_error("gemv_slot_waves %lld not 0 or 8..16", (long long)value); return IXH_EINVAL; }
        g_opt_gemv_slot_waves.store((int)value, std::memory_order_relaxed);
        return IXH_OK;
    }
    if (strcmp(name, "gemv_strips") == 0) {
        if (value < -1 || value > 6) { set_error("gemv_strips %lld not in -1..6", (long long)value); return IXH_EINVAL; }
        g_opt_gemv_strips.store((int)value, std::memory_order_relaxed);
        return IXH_OK;
    }
    set_error("unknown option '%s'", name);
    return IXH_EINVAL;
}

int64_t ixh_prefix_entries(int64_t n, int64_t chunk) {
    if (n < 0 || chunk <= 0) return -1;
    return (n + chunk - 1) / chunk + 1;
}

int ixh_prefix_build(const IxhPacked *packed, int64_t chunk, int32_t *prefix, ixh_stream_t stream) {
    Dev d;
    int rc = to_dev(packed, &d, false);  // the table is counted from the bitmaps alone
    if (rc) return rc;
    if (chunk <= 0 || chunk >= (1ll << 31)) { set_error("chunk %lld out of range", (long long)chunk); return IXH_EINVAL; }
    if (!prefix) { set_error("prefix is NULL"); return IXH_EINVAL; }
    rc = launch_prefix_build(d, (uint32_t)chunk, prefix, (hipStream_t)stream);
    if (rc) set_error("prefix_build: launch failed");
    return rc;
}

static int decode_any(const IxhPacked *packed, const int32_t *prefix, int64_t chunk, int8_t *out_i8, uint16_t *out_bf16,
                      GroupScales gs, ixh_stream_t stream) {
    Dev d;
    int rc = to_dev(packed, &d, gs.fp16 == nullptr);
    if (rc) return rc;
    if (chunk <= 0 || chunk >= (1ll << 31)) { set_error("chunk %lld out of range", (long long)chunk); return IXH_EINVAL; }
    if (d.n == 0) return IXH_OK;
    if (!prefix) { set_error("prefix is NULL"); return IXH_EINVAL; }
    if (!out_i8 && !out_bf16) { set_error("both outputs are NULL"); return IXH_EINVAL; }
    // Which decoder: by the tensor, unless the option "decode_kernel" names one (so that tests and measurements can
    // take each of them; a named kernel that does not support the call is skipped).
    const int want = g_opt_decode_kernel.load(std::memory_order_relaxed);
    auto allowed = [&](int which) { return want == kDecodeAuto || want == which; };
    const bool forced = want != kDecodeAuto;
    // level 1 holds at least 97 % of the elements (from the size of its stream)
    const bool mostly_l1 = (uint64_t)d.st_words[0] * 32u / 3u >= (uint64_t)d.n / 100u * 97u;
    if (allowed(kDecodeRows) && (forced || mostly_l1) && !gs.fp16 && decode_rows358_supports(d, (uint32_t)chunk, out_i8, out_bf16))
        // first level of 3 bits, almost all level 1, whole unit-quads: the row-block decoder (ixh_decode_rows358.hip)
        rc = launch_decode_rows358(d, prefix, out_bf16, (hipStream_t)stream);
    else if (allowed(kDecodeDense) && (forced || !mostly_l1) && decode_dense358_supports(d, (uint32_t)chunk, out_i8, out_bf16, gs))
        // (3,5,8) with many elements above level 1: the level-by-level decoder (ixh_dense358.hip)
        rc = launch_decode_dense358(d, prefix, out_bf16, gs, (hipStream_t)stream);
    else if (allowed(kDecodeDense) && (forced || !mostly_l1) && !gs.fp16 && decode_dense34568_supports(d, (uint32_t)chunk, out_i8, out_bf16))
        // the same for the five-level scheme (3,4,5,6,8) (ixh_dense5.hip)
        rc = launch_decode_dense34568(d, prefix, out_bf16, (hipStream_t)stream);
    else if ((allowed(kDecodeStaged) || allowed(kDecodeRows) || allowed(kDecodeDense)) &&
             decode_staged_supports(d, (uint32_t)chunk, out_i8, out_bf16, gs))
        rc = launch_decode_staged(d, prefix, out_bf16, gs, (hipStream_t)stream);
    else
        rc = launch_decode(d, prefix, (uint32_t)chunk, out_i8, out_bf16, gs, (hipStream_t)stream);
    if (rc == IXH_ELAUNCH) set_error("decode: launch failed");
    return rc;
}

int ixh_decode(const IxhPacked *packed, const int32_t *prefix, int64_t chunk, int8_t *out_i8,
               uint16_t *out_bf16, ixh_stream_t stream) {
    return decode_any(packed, prefix, chunk, out_i8, out_bf16, GroupScales{nullptr, 0}, stream);
}

int ixh_decode_gs(const IxhPacked *packed, const int32_t *prefix, int64_t chunk, const uint16_t *group_scales,
                  int64_t group_size, uint16_t *out_bf16, ixh_stream_t stream) {
    if (!group_scales) { set_error("group_scales is NULL"); return IXH_EINVAL; }
    if (group_size <= 0 || group_size >= (1ll << 31)) { set_error("group_size %lld out of range", (long long)group_size); return IXH_EINVAL; }
    if (!out_bf16) { set_error("out_bf16 is NULL"); return IXH_EINVAL; }
    return decode_any(packed, prefix, chunk, nullptr, out_bf16, GroupScales{group_scales, (uint32_t)group_size}, stream);
}

static int gemv_checks(const Dev &d, int64_t chunk, int32_t m) {
    if (m < 1 || m > 16) { set_error("m = %d not in 1..16", m); return IXH_EINVAL; }
    if (chunk <= 0 || chunk > (int64_t)d.in_f || d.in_f % chunk != 0) {
        set_error("chunk %lld must divide in_f %u", (long long)chunk, d.in_f);
        return IXH_EINVAL;
    }
    return IXH_OK;
}

size_t ixh_gemv_workspace_bytes(const IxhPacked *packed, int64_t chunk, int32_t m, uint32_t flags) {
    Dev d;
    if (to_dev(packed, &d)) return 0;
    if (d.n == 0 || gemv_checks(d, chunk, m)) return 0;
    if (flags & IXH_GEMV_ATOMIC) return 0;
    const size_t n_chunks = d.in_f / (uint32_t)chunk;
    if (n_chunks == 1) return 0;
    return n_chunks * (size_t)m * d.out_f * sizeof(float);
}

// Which of the kernel families for tensors that are almost all level 1 may take a call.
struct Level1Family {
    bool mostly_l1, fast, fast_any;
};
static Level1Family level1_family(const Dev &d, int64_t chunk, int32_t m, uint32_t flags) {
    Level1Family f;
    // The (3,5,8) kernels are built for tensors that are almost all level 1 (every other element costs
    // them a queue record); denser mixes go to the general kernel unless the caller insists.
    f.mostly_l1 = (uint64_t)d.st_words[0] * 32u / 3u >= (uint64_t)d.n / 100u * 97u;
    f.fast = !(flags & (IXH_GEMV_FORCE_GENERIC | IXH_GEMV_STAGED | IXH_GEMV_DENSE)) && is_358(d) &&
             fast358_supports(d, (uint32_t)chunk, m) &&
             (f.mostly_l1 || (flags & (IXH_GEMV_COLUMN_KERNEL | IXH_GEMV_FORCE_358)));
    // any other scheme whose first level has 3 bits, almost all level 1: the row-block kernel with the resolver that
    // walks the nested bitmaps (the column-block kernel is (3,5,8) only, so 5..8 rows go on to the any-scheme kernel)
    f.fast_any = !f.fast && !is_358(d) && d.n_levels >= 2 && d.bits[0] == 3 &&
                 !(flags & (IXH_GEMV_FORCE_GENERIC | IXH_GEMV_STAGED | IXH_GEMV_DENSE | IXH_GEMV_COLUMN_KERNEL)) &&
                 fast358_supports(d, (uint32_t)chunk, m) && (f.mostly_l1 || (flags & IXH_GEMV_FORCE_358));
    return f;
}

// partial_ws: the workspace may be smaller than ixh_gemv_workspace_bytes says (the built-in buffer of
// ixh_gemv_noalloc): kernels whose workgroups share a block of rows then share it among as many pieces as it holds,
// kernels that need no workspace run as ever, and only a call whose kernel needs all of it fails.
static int gemv_any(const IxhPacked *packed, const int32_t *prefix, int64_t chunk, const uint16_t *x, int32_t m,
                    int64_t ldx, uint16_t *y, int64_t ldy, float *y32, void *workspace, size_t workspace_bytes,
                    uint32_t flags, ixh_stream_t stream, bool partial_ws = false) {
    Dev d;
    int rc = to_dev(packed, &d);
    if (rc) return rc;
    if (d.n == 0) {
        if (d.out_f != 0 && m >= 1 && m <= 16 && !(flags & IXH_GEMV_ATOMIC) && y) {
            // no inputs: every output is an empty sum
            for (int j = 0; j < m; ++j)
                if (launch_fill_u16(y + (int64_t)j * ldy, d.out_f, 0, (hipStream_t)stream)) return IXH_ELAUNCH;
        }
        return IXH_OK;
    }
    rc = gemv_checks(d, chunk, m);
    if (rc) return rc;
    if (!prefix || !x) { set_error("prefix or x is NULL"); return IXH_EINVAL; }
    if (ldx < (int64_t)d.in_f && m > 1) { set_error("ldx %lld < in_f %u", (long long)ldx, d.in_f); return IXH_EINVAL; }
    const bool atomic = (flags & IXH_GEMV_ATOMIC) != 0;
    size_t need = 0;
    bool ws_full = true;
    uint32_t ws_pieces = 0;
    if (atomic) {
        if (!y32) { set_error("IXH_GEMV_ATOMIC needs y32"); return IXH_EINVAL; }
    } else {
        if (!y) { set_error("y is NULL"); return IXH_EINVAL; }
        if (ldy < (int64_t)d.out_f && m > 1) { set_error("ldy %lld < out_f %u", (long long)ldy, d.out_f); return IXH_EINVAL; }
        need = ixh_gemv_workspace_bytes(packed, chunk, m, flags);
        ws_full = !need || (workspace && workspace_bytes >= need);
        if (!ws_full && !partial_ws) {
            set_error("workspace of %zu bytes needed, %zu given", need, workspace ? workspace_bytes : (size_t)0);
            return IXH_EWORKSPACE;
        }
        if (workspace) {  // pieces of m x out_f partial sums that the workspace holds
            const size_t piece = (size_t)m * d.out_f * sizeof(float), n_chunks = d.in_f / (uint32_t)chunk;
            ws_pieces = (uint32_t)(workspace_bytes / piece < n_chunks ? workspace_bytes / piece : n_chunks);
        }
    }
    rc = IXH_EUNSUPPORTED;
    const Level1Family fam = level1_family(d, chunk, m, flags);
    const bool mostly_l1 = fam.mostly_l1, fast = fam.fast, fast_any = fam.fast_any;
    if ((fast || fast_any) && !(flags & IXH_GEMV_COLUMN_KERNEL)) {
        // The row-block kernels: a workgroup owns whole rows, so the split-K contract (add into the caller's fp32
        // vector) costs them one addition per output.  First the strip kernel (products on the matrix pipe, up to 16
        // activation rows where they fit LDS beside the tables), then the kernels that multiply lane by lane: up to
        // four rows, five to eight with the activations shared in LDS, nine to sixteen eight or four rows at a time
        // (atomic mode excepted: a later group that does not fit must not leave an earlier one added).
        uint16_t *const yb = atomic ? nullptr : y;
        float *const yf = atomic ? y32 : nullptr;
        // (the workspace holds in_f / chunk pieces of m x out_f sums)
        rc = launch_gemv_358_tiles(d, prefix, x, m, ldx, yb, ldy, yf, atomic || !ws_pieces ? nullptr : (float *)workspace,
                                   ws_pieces, (hipStream_t)stream);
        if (rc == IXH_EUNSUPPORTED) rc = launch_gemv_358_strips(d, prefix, x, m, ldx, yb, ldy, yf, (hipStream_t)stream);
        if (rc == IXH_EUNSUPPORTED && m <= 8)
            rc = launch_gemv_358_rows(d, prefix, x, m, ldx, yb, ldy, yf, (hipStream_t)stream);
        if (rc == IXH_EUNSUPPORTED && m > 8 && !atomic) {
            for (int group = 8; group >= 4 && rc == IXH_EUNSUPPORTED; group -= 4) {
                rc = IXH_OK;
                for (int j = 0; j < m && rc == IXH_OK; j += group) {
                    const int mj = m - j < group ? m - j : group;
                    rc = launch_gemv_358_strips(d, prefix, x + (int64_t)j * ldx, mj, ldx, y + (int64_t)j * ldy, ldy, nullptr,
                                                (hipStream_t)stream);
                    if (rc == IXH_EUNSUPPORTED)
                        rc = launch_gemv_358_rows(d, prefix, x + (int64_t)j * ldx, mj, ldx, y + (int64_t)j * ldy, ldy,
                                                  nullptr, (hipStream_t)stream);
                }
            }
        }
    }
    if (rc == IXH_EUNSUPPORTED && !ws_full) {  // every kernel from here on keeps one piece per chunk of a row
        set_error("gemv_noalloc: the kernel for this call needs %zu bytes of partial sums, the built-in buffer holds "
                  "%zu; call ixh_gemv with a workspace of your own", need, workspace_bytes);
        return IXH_EWORKSPACE;
    }
    if (fast && rc == IXH_EUNSUPPORTED)
        rc = launch_gemv_358(d, prefix, (uint32_t)chunk, x, m, ldx, y, ldy, y32, (float *)workspace, atomic,
                             (hipStream_t)stream);
    if (rc == IXH_EUNSUPPORTED && !(flags & (IXH_GEMV_FORCE_GENERIC | IXH_GEMV_STAGED)) &&
        (!mostly_l1 || (flags & IXH_GEMV_DENSE)) && gemv_dense358_supports(d, (uint32_t)chunk, m, x))
        // (3,5,8), one activation row, many elements above level 1: level-by-level products over compacted x
        rc = launch_gemv_dense358(d, prefix, x, y, y32, (float *)workspace, atomic, (hipStream_t)stream);
    if (rc == IXH_EUNSUPPORTED && !(flags & (IXH_GEMV_FORCE_GENERIC | IXH_GEMV_STAGED)) &&
        (!mostly_l1 || (flags & IXH_GEMV_DENSE)) && gemv_dense34568_supports(d, (uint32_t)chunk, m, x))
        // the same for the five-level scheme (3,4,5,6,8)
        rc = launch_gemv_dense34568(d, prefix, x, y, y32, (float *)workspace, atomic, (hipStream_t)stream);
    if (rc == IXH_EUNSUPPORTED && !atomic && !(flags & (IXH_GEMV_FORCE_GENERIC | IXH_GEMV_STAGED)) &&
        (!mostly_l1 || (flags & IXH_GEMV_DENSE)) &&
        (g_opt_gemv_dense_tiles.load(std::memory_order_relaxed) > 0 ||
         (g_opt_gemv_dense_tiles.load(std::memory_order_relaxed) == 0 && m >= 4)) &&
        gemv_dense358_tiles_supports(d, (uint32_t)chunk, m, x, ldx))
        // (3,5,8), 4..16 activation rows (2..16 when the option says so), many elements above level 1: 16 rows' spans
        // gathered to position order in LDS, products on the matrix pipe; its time does not grow with the rows
        rc = launch_gemv_dense358_tiles(d, prefix, x, m, ldx, y, ldy, (float *)workspace, (hipStream_t)stream);
    if (rc == IXH_EUNSUPPORTED && !atomic && !(flags & (IXH_GEMV_FORCE_GENERIC | IXH_GEMV_STAGED)) &&
        (!mostly_l1 || (flags & IXH_GEMV_DENSE)) && g_opt_gemv_dense_tiles.load(std::memory_order_relaxed) >= 0 &&
        gemv_dense34568_tiles_supports(d, (uint32_t)chunk, m, x, ldx))
        // the same for the five-level scheme (3,4,5,6,8), from two rows on (it has no kernel of its own for two and three)
        rc = launch_gemv_dense34568_tiles(d, prefix, x, m, ldx, y, ldy, (float *)workspace, (hipStream_t)stream);
    if (rc == IXH_EUNSUPPORTED && !atomic && !(flags & (IXH_GEMV_FORCE_GENERIC | IXH_GEMV_STAGED)) &&
        (!mostly_l1 || (flags & IXH_GEMV_DENSE)) && gemv_dense358_rows_supports(d, (uint32_t)chunk, m, x, ldx))
        // (3,5,8), 2..8 activation rows, many elements above level 1: weights gathered to position order per span
        rc = launch_gemv_dense358_rows(d, prefix, x, m, ldx, y, ldy, (float *)workspace, (hipStream_t)stream);
    if (rc == IXH_EUNSUPPORTED && !(flags & IXH_GEMV_FORCE_GENERIC) && gemv_staged_supports(d, (uint32_t)chunk, x, ldx))
        // any scheme, any mix, whole 512-element units: streams staged in LDS, eight elements per lane
        rc = launch_gemv_staged(d, prefix, x, m, ldx, y, ldy, y32, (float *)workspace, atomic, (hipStream_t)stream);
    if (rc == IXH_EUNSUPPORTED) {  // other chunk sizes, ragged rows, unaligned x
        rc = launch_gemv_generic(d, prefix, (uint32_t)chunk, x, m, ldx, y, ldy, y32, (float *)workspace, atomic,
                                 (hipStream_t)stream);
    }
    if (rc == IXH_ELAUNCH) set_error("gemv: launch failed");
    return rc;
}

int ixh_gemv(const IxhPacked *packed, const int32_t *prefix, int64_t chunk, const uint16_t *x, int32_t m,
             int64_t ldx, uint16_t *y, int64_t ldy, float *y32, void *workspace, size_t workspace_bytes,
             uint32_t flags, ixh_stream_t stream) {
    return gemv_any(packed, prefix, chunk, x, m, ldx, y, ldy, y32, workspace, workspace_bytes, flags, stream);
}

// ---- ixh_gemv for callers that may not allocate: the partial sums go to a buffer that is part of the library ----
// The array lives in the code object, once per GPU the library runs on, until the process ends.  In host code its
// name is only a handle for hipGetSymbolAddress: kernels and everything else take the per-device address looked
// up below, never the name.
static __device__ __align__(256) unsigned char scratch[IXH_NOALLOC_WORKSPACE_BYTES];

constexpr int kMaxDevices = 64;
static void *g_scratch_ptr[kMaxDevices];  // address of `scratch` on each device, looked up on first use there
static std::mutex g_scratch_lock;

// the current device's copy of `scratch`
static int scratch_of_current_device(void **out) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        set_error("gemv_noalloc: no current device (or its index %d is beyond %d)", dev, kMaxDevices - 1);
        return IXH_ELAUNCH;
    }
    std::lock_guard<std::mutex> guard(g_scratch_lock);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            set_error("gemv_noalloc: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(e));
            return IXH_ELAUNCH;
        }
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return IXH_OK;
}

int ixh_gemv_noalloc(const IxhPacked *packed, const int32_t *prefix, int64_t chunk, const uint16_t *x, int32_t m,
                     int64_t ldx, uint16_t *y, int64_t ldy, uint32_t flags, ixh_stream_t stream) {
    if (flags & IXH_GEMV_ATOMIC) {
        set_error("gemv_noalloc: IXH_GEMV_ATOMIC takes no workspace; call ixh_gemv");
        return IXH_EINVAL;
    }
    Dev d;
    if (to_dev(packed, &d) == IXH_OK && d.n != 0 && gemv_checks(d, chunk, m) == IXH_OK) {
        // only the row-block kernels (no workspace, or as many pieces as there is room for) can take a call whose
        // full set of partial sums is larger than the buffer
        const size_t need = ixh_gemv_workspace_bytes(packed, chunk, m, flags);
        const Level1Family fam = level1_family(d, chunk, m, flags);
        if (need > (size_t)IXH_NOALLOC_WORKSPACE_BYTES && (!(fam.fast || fam.fast_any) || (flags & IXH_GEMV_COLUMN_KERNEL))) {
            set_error("gemv_noalloc: the kernel for this call needs %zu bytes of partial sums, the built-in buffer "
                      "holds %zu; call ixh_gemv with a workspace of your own", need, (size_t)IXH_NOALLOC_WORKSPACE_BYTES);
            return IXH_EWORKSPACE;
        }
    }
    void *ws = nullptr;
    const int rc = scratch_of_current_device(&ws);
    if (rc) return rc;
    // every partial sum the second kernel reads was written by the first in the same call: nothing to clear
    // (a call whose kernel needs more partial sums than the buffer holds fails inside with IXH_EWORKSPACE, before
    // any launch; the row-block kernels need none, the tile kernel shares the buffer among the pieces it holds)
    return gemv_any(packed, prefix, chunk, x, m, ldx, y, ldy, nullptr, ws, (size_t)IXH_NOALLOC_WORKSPACE_BYTES, flags,
                    stream, true);
}

size_t ixh_gemm_workspace_bytes(const IxhPacked *packed, int32_t m) {
    Dev d;
    if (to_dev(packed, &d) || d.n == 0 || m < 1) return 0;
    return max(prefill_workspace_bytes(d, (uint32_t)m), prefill358_workspace_bytes(d, (uint32_t)m));
}

// The kernel of ixh_prefill358.hip: tensors that are almost all level 1 (the full decode of such tensors and the
// products of few activation rows switch at the same share) and large enough to give most CUs a 128-row tile and a
// few unit columns; measured against k_prefill on 4096 x 4096 ... 8192 x 28672, 32 ... 2048 activation rows: ahead
// everywhere above 2^24 elements, at 2^24 from 512 rows on, behind below.
static bool gemm_takes_tiles(const Dev &d, const uint16_t *x, int64_t ldx, int32_t m, const void *workspace) {
    const int want = g_opt_gemm_tiles.load(std::memory_order_relaxed);
    if (want < 0 || !prefill358_supports(d, x, ldx) || ((uintptr_t)workspace & 15u) != 0) return false;
    if (want > 0) return true;
    const bool mostly_l1 = (uint64_t)d.st_words[0] * 32u / 3u >= (uint64_t)d.n / 100u * 97u;
    return mostly_l1 && (d.n > (1u << 24) || (d.n == (1u << 24) && m >= 512));
}

int ixh_gemm(const IxhPacked *packed, const int32_t *prefix, const uint16_t *x, int32_t m, int64_t ldx, uint16_t *y,
             int64_t ldy, void *workspace, size_t workspace_bytes, ixh_stream_t stream) {
    Dev d;
    int rc = to_dev(packed, &d);
    if (rc) return rc;
    if (m < 1) { set_error("m = %d < 1", m); return IXH_EINVAL; }
    if (!y) { set_error("y is NULL"); return IXH_EINVAL; }
    if (ldy < (int64_t)d.out_f && m > 1) { set_error("ldy %lld < out_f %u", (long long)ldy, d.out_f); return IXH_EINVAL; }
    if (d.n == 0) {
        for (int j = 0; j < m && d.out_f; ++j)
            if (launch_fill_u16(y + (int64_t)j * ldy, d.out_f, 0, (hipStream_t)stream)) return IXH_ELAUNCH;
        return IXH_OK;
    }
    if (!prefix || !x) { set_error("prefix or x is NULL"); return IXH_EINVAL; }
    if (ldx < (int64_t)d.in_f && m > 1) { set_error("ldx %lld < in_f %u", (long long)ldx, d.in_f); return IXH_EINVAL; }
    const bool tiles = gemm_takes_tiles(d, x, ldx, m, workspace);
    if (!tiles && !prefill_supports(d, x, ldx)) {
        set_error("gemm: needs in_f %% 512 == 0, x 16-byte aligned, ldx %% 8 == 0, last stream 4-byte aligned");
        return IXH_EUNSUPPORTED;
    }
    const size_t need = tiles ? prefill358_workspace_bytes(d, (uint32_t)m) : prefill_workspace_bytes(d, (uint32_t)m);
    if (!workspace || workspace_bytes < need) {
        set_error("workspace of %zu bytes needed, %zu given", need, workspace ? workspace_bytes : (size_t)0);
        return IXH_EWORKSPACE;
    }
    if (tiles)
        rc = launch_prefill358(d, prefix, x, (uint32_t)m, ldx, y, ldy, (float *)workspace,
                               g_opt_gemm_tiles.load(std::memory_order_relaxed) == 2 ? 1u : 0u, (hipStream_t)stream);
    else
        rc = launch_prefill(d, prefix, x, (uint32_t)m, ldx, y, ldy, (float *)workspace, (hipStream_t)stream);
    if (rc == IXH_ELAUNCH) set_error("gemm: launch failed");
    return rc;
}

static int encode_levels_ok(int32_t n_levels, const int32_t *level_bits) {
    if (n_levels < 2 || n_levels > IXH_MAX_LEVELS) { set_error("n_levels %d not in 2..%d", n_levels, IXH_MAX_LEVELS); return IXH_EINVAL; }
    if (!level_bits) { set_error("level_bits is NULL"); return IXH_EINVAL; }
    if (level_bits[n_levels - 1] != 8) { set_error("last level must be 8-bit, got %d", level_bits[n_levels - 1]); return IXH_EINVAL; }
    for (int i = 0; i < n_levels - 1; ++i) {
        if (level_bits[i] < 1 || level_bits[i] > 7 || (i > 0 && level_bits[i] < level_bits[i - 1])) {
            set_error("level_bits[%d] = %d: widths must ascend within 1..7 before the final 8", i, level_bits[i]);
            return IXH_EINVAL;
        }
    }
    return IXH_OK;
}

size_t ixh_encode_workspace_bytes(int64_t out_f, int64_t in_f, int32_t n_levels) {
    if (out_f <= 0 || in_f <= 0 || n_levels < 2 || n_levels > IXH_MAX_LEVELS) return 0;
    const uint64_t n = (uint64_t)out_f * (uint64_t)in_f;
    if (n >= (1ull << 31)) return 0;
    return encode_workspace_bytes(n, n_levels);
}

int ixh_encode_scan(const uint16_t *w, int64_t out_f, int64_t in_f, int32_t n_levels, const int32_t *level_bits,
                    uint16_t *scale, int32_t *prefix, void *workspace, size_t workspace_bytes,
                    ixh_stream_t stream) {
    int rc = encode_levels_ok(n_levels, level_bits);
    if (rc) return rc;
    if (out_f <= 0 || in_f <= 0) { set_error("encode: empty weight (the reference's max() raises on it too)"); return IXH_EINVAL; }
    const uint64_t n = (uint64_t)out_f * (uint64_t)in_f;
    if (n >= (1ull << 31)) { set_error("out_f * in_f = %llu does not fit the 31-bit rank tables", (unsigned long long)n); return IXH_EINVAL; }
    if (!w || !scale || !prefix) { set_error("encode: w, scale or prefix is NULL"); return IXH_EINVAL; }
    const size_t need = encode_workspace_bytes(n, n_levels);
    if (!workspace || workspace_bytes < need) {
        set_error("workspace of %zu bytes needed, %zu given", need, workspace ? workspace_bytes : (size_t)0);
        return IXH_EWORKSPACE;
    }
    int bits[IXH_MAX_LEVELS];
    for (int i = 0; i < n_levels; ++i) bits[i] = level_bits[i];
    rc = launch_encode_scan(w, (uint32_t)n, n_levels, bits, scale, prefix, workspace, (hipStream_t)stream);
    if (rc == IXH_ELAUNCH) set_error("encode_scan: launch failed");
    return rc;
}

int ixh_encode_pack(const uint16_t *w, const IxhPacked *dst, const int32_t *prefix, ixh_stream_t stream) {
    Dev d;
    int rc = to_dev(dst, &d);
    if (rc) return rc;
    if (d.n == 0) { set_error("encode: empty weight"); return IXH_EINVAL; }
    if (!w || !prefix) { set_error("encode: w or prefix is NULL"); return IXH_EINVAL; }
    rc = launch_encode_pack(w, d, prefix, (hipStream_t)stream);
    if (rc == IXH_ELAUNCH) set_error("encode_pack: launch failed");
    return rc;
}

}  // extern "C"
