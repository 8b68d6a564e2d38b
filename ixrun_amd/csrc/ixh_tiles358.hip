// (3,5,8) fused decode + skinny GEMM for gfx950, tile variant: 16 weight rows x 16 activation rows per matrix
// instruction, so that up to 16 activation rows cost what one costs.
//
// Work split.  A workgroup owns whole rows, or, where rows are few per CU, shares a taller block of rows with k - 1
// others, each taking a run of the rows' column blocks (their fp32 sums go to a workspace as [piece][m][row] and
// k_reduce_chunks adds them in piece order): taller blocks fill tiles of 16 and need fewer parts (below).  Its rows are cut into tiles of 16, 8 or 4 (one size per launch); a tile of
// 16 / s rows takes s column blocks side by side in a step (slots), so that the 16 columns of the matrix instruction
// are always 16 different (row, block) pairs, and serves up to 16 / s activation rows: row a of the other operand is
// activation row a % (16 / s) at the columns of slot a / (16 / s), and the products whose slots agree are the sums.
// Short tiles fill the lanes where a workgroup's rows are not a multiple of 16 (5120 rows on 256 CUs: 20 each).  A
// wave belongs to one tile and to one share of the steps for its whole life, so its 16 x 16 accumulator never leaves
// its registers: wave = tile * n_sub + sub, and the steps of a part are dealt in runs to the n_sub waves of a tile.
// Lane (n, kg), n = lane % 16, kg = lane / 16, decodes strip kg (128 columns) of (row, block) pair n, word by word, exactly
// as in ixh_strips358.hip: bitmap words and table entry into registers, ranks from popcounts (the strips of a unit are
// 16 lanes apart: their counts travel through ds_bpermute), 16 stream bytes per word, v_alignbit, splice, pair table.
//
// Products.  v_mfma_f32_16x16x32_bf16 takes eight weights of every lane (B: column n, k group kg) and eight activations
// of every lane (A: activation row n, the same eight columns of strip kg) and adds into D[4 kg + i][n], i = 0..3:
// four instructions per 32-column word whatever the number of activation rows.  Activation rows that do not exist
// read a strip of zeros.
//
// Activations.  In LDS, in padded strips as in the strip kernel, 16 bytes of shift between rows; when all rows do not
// fit beside the tables they are held one part of the columns at a time, and the workgroup walks the parts in turn
// (a barrier, the next part's copy, a barrier).
//
// Elements above level 1 go to the wave's record queue and are resolved by the wave itself (it owns its tile): 64 at a
// time their weights are looked up lane by lane, then they go through the matrix pipe like the others (TileSink), into
// the same accumulators.  At the end every wave stores its accumulators; after one barrier the outputs are summed over
// the sub-ranges in order.  Every addition has a fixed place: a call gives the same bits every time.
#include <math.h>

#include "ixh_rows_common.h"

namespace ixh {

// ixh_set_option("gemv_tile_rows"): 0 = the planner's choice, 2 / 3 / 4 = tiles of 4 / 8 / 16 rows only
extern std::atomic<int> g_opt_gemv_tile_rows;
// ixh_set_option("gemv_tile_cus"): the number of CUs the planner spreads the rows over; 0 = the device's
extern std::atomic<int> g_opt_gemv_tile_cus;
// ixh_set_option("gemv_tile_split"): the number of workgroups that share a block of rows, each taking a run of its
// column blocks; 0 = the planner's choice
extern std::atomic<int> g_opt_gemv_tile_split;

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));

constexpr int kTMaxWaves = 16;
constexpr uint32_t kTMaxRows = 128;  // rows per workgroup at most (8 tiles)
constexpr int kTMaxM = 16;
constexpr uint32_t kTQueue = 256;  // records in a wave's queue: a task's records must fit (4 words x 64 lanes)
constexpr size_t kTLdsLimit = 160 * 1024;
// bytes between the 128-column strips of an activation row: 16-byte reads need 16-byte aligned strips, and 272 = 68
// dwords puts the four strips of a column block four banks apart, as the 16-byte shift between rows does for the rows
constexpr uint32_t kTStripBytes = 272;

constexpr uint32_t kFlagPieces = 0x100u;  // y32 is a workspace of pieces: plain stores at the workgroup's piece

struct TilesLds {
    uint32_t tq1, tq2, side, xs, xs_row, zero, partial, waves, wave_bytes, tasks_off, round_off, total;
};

// x_blocks: column blocks of the activation rows that LDS holds at a time
__host__ __device__ inline TilesLds tiles_layout(uint32_t rows_cap, uint32_t n_chunks, uint32_t x_blocks, uint32_t n_sub,
                                                 uint32_t n_waves, int m, uint32_t qcap) {
    TilesLds L;
    const uint32_t tbl = ((rows_cap * n_chunks + 1u + 3u) & ~3u) * 4u;  // one entry past the slice: its end ranks
    L.tq1 = kRLutBytes + kRSpliceBytes;
    L.tq2 = L.tq1 + tbl;
    L.side = L.tq2 + tbl;
    L.xs = L.side + kRSideBytes;
    // bytes between activation rows: the padded strips, then 16 bytes so that the 16 rows a b128 read takes
    // start four banks apart
    L.xs_row = ((x_blocks * 4u * kTStripBytes + 127u) & ~127u) + 16u;
    // [n_sub][rows_cap][m] fp32, the waves' accumulators at the end (n_sub: waves per tile x slots per wave): over the
    // activations, which nobody reads any more then
    L.partial = L.xs;
    const uint32_t partial_bytes = (n_sub * rows_cap * (uint32_t)m * 4u + 15u) & ~15u;
    // a strip of zeros: what the lanes of absent activation rows read
    L.zero = L.xs + max((uint32_t)m * L.xs_row, partial_bytes);
    L.waves = (L.zero + kTStripBytes + 15u) & ~15u;
    L.tasks_off = qcap * 8u;  // behind the queue of 8-byte records
    L.round_off = (L.tasks_off + kRTasks2 * 2u + 15u) & ~15u;  // the elements of a round: {weight | column, address}
    L.wave_bytes = L.round_off + kWave * 8u;
    L.total = L.waves + n_waves * L.wave_bytes;
    return L;
}

// The resolved elements above level 1 of a round go through the matrix pipe like the others, into the same
// accumulators: every lane writes its element's weight, the column n of the product it belongs to and the LDS address of
// its activation in row 0 to the wave's list of the round; then, sixteen elements per instruction, lane (n, kg) reads
// elements 4 kg .. 4 kg + 3 (32 consecutive bytes, the same for the 16 lanes of a k group) and gathers the activations
// of its row as one operand and, as the other, the weights of the elements that belong to column n (zero for the rest).
// (Fetching the four elements from the lanes that hold them, eight ds_bpermute a group, took 1.6 times as long.)
struct TileSink {
    static constexpr bool active = true;
    f32x4 acc;           // the wave's accumulators: taken over for the time of the resolver, handed back after it
    uint32_t n, kg;
    uint32_t x_off;      // bytes from activation row 0 to the lane's activation row
    bool x_on;           // that row exists
    uint32_t idle_addr;  // an address that can be read
    uint32_t wn, xa;     // the lane's element of the round: weight bits | column << 16, address
    uint32_t n_chunks;
    uint32_t round_addr;  // the wave's list of a round's elements, 8 bytes each
    // a record's second word: column n of the product << 27 | row in the workgroup << 20 | column / 32 << 9 | level-1
    // elements between the unit's start and the word
    __device__ __forceinline__ void unpack(uint32_t packed, uint32_t unit0, uint32_t tq1_addr, uint32_t &r0, uint32_t &unit,
                                           uint32_t &k0, uint32_t &row_field) {
        const uint32_t lrow = (packed >> 20) & 127u, kw = (packed >> 9) & 2047u;
        unit = unit0 + lrow * n_chunks + (kw >> 4);
        r0 = unit * kFastChunk + ((kw & 15u) << 5) - lds_u32(tq1_addr + (unit - unit0) * 4u) - (packed & 511u);
        k0 = kw << 5;
        row_field = ((packed >> 27) << 12) | lrow;
    }
    __device__ __forceinline__ void put(uint32_t w_bits, uint32_t row_field, uint32_t addr) {
        wn = w_bits | ((row_field >> 12) << 16);
        xa = addr;
    }
    __device__ __forceinline__ void idle() {
        wn = 0u;
        xa = idle_addr;
    }
    // lanes: the lanes below this number may hold an element
    __device__ __forceinline__ void flush(uint32_t lanes) {
        *reinterpret_cast<__attribute__((address_space(3))) u32x2 *>((uintptr_t)(round_addr + (kg * 16u + n) * 8u)) = u32x2{wn, xa};
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            if ((uint32_t)g * 16u >= lanes) break;
            const uint32_t at = round_addr + ((uint32_t)g * 16u + kg * 4u) * 8u;
            const u32x4 p = lds_u128(at), q = lds_u128(at + 16u);  // {wn, xa} of elements 4 kg, 4 kg + 1 | + 2, + 3
            const uint32_t x0 = lds_u16(p.y + x_off), x1 = lds_u16(p.w + x_off);
            const uint32_t x2 = lds_u16(q.y + x_off), x3 = lds_u16(q.w + x_off);
            const uint32_t w0 = (p.x >> 16) == n ? (p.x & 0xFFFFu) : 0u, w1 = (p.z >> 16) == n ? p.z << 16 : 0u;
            const uint32_t w2 = (q.x >> 16) == n ? (q.x & 0xFFFFu) : 0u, w3 = (q.z >> 16) == n ? q.z << 16 : 0u;
            const u32x2 ap = {x_on ? (x0 | (x1 << 16)) : 0u, x_on ? (x2 | (x3 << 16)) : 0u};
            const u32x2 bp = {w0 | w1, w2 | w3};
            acc = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4, ap), __builtin_bit_cast(s16x4, bp), acc, 0, 0, 0);
        }
    }
};

template <bool ANY>
__global__ void __launch_bounds__(kTMaxWaves * kWave)
k_gemv358_tiles(Dev P, const int32_t *__restrict__ prefix, uint32_t n_chunks, uint32_t rows_per_wg, uint32_t n_sub,
                uint32_t x_blocks, uint32_t lg_rows, uint32_t flags, uint32_t k_plan,
                const uint16_t *__restrict__ x, int m, int64_t ldx,
                uint16_t *__restrict__ y, int64_t ldy, float *__restrict__ y32) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const uint32_t n_waves = blockDim.x >> 6;
    const uint32_t n = lane & 15u, kg = lane >> 4;
    // a tile is tile_rows = 4, 8 or 16 weight rows by 16 / tile_rows column blocks side by side: column n of the matrix
    // instruction is weight row n % tile_rows in column block n / tile_rows of the step (its slot)
    const uint32_t tile_rows = 1u << lg_rows, slots = 16u >> lg_rows;
    const uint32_t r = n & (tile_rows - 1u);

    // k_split workgroups share a block of rows, k_blocks column blocks of every row each; with kFlagPieces their
    // sums go to y32 as a workspace ([piece][m][row] fp32) for the kernel that adds the pieces in order
    // (k_plan: k_split | k_blocks << 8)
    const uint32_t k_split = k_plan & 255u, k_blocks = k_plan >> 8;
    const uint32_t row_group = blockIdx.x / k_split;
    const uint32_t kb_end = min(n_chunks, (blockIdx.x - row_group * k_split + 1u) * k_blocks);
    const uint32_t row0 = row_group * rows_per_wg;
    const uint32_t rows_here = min(rows_per_wg, P.out_f - row0), rows_cap = rows_per_wg;
    constexpr uint32_t qcap = kTQueue;
    const TilesLds L = tiles_layout(rows_cap, n_chunks, x_blocks, n_sub * slots, n_waves, m, qcap);

    // the pair table is addressed with (index bits | lane bits): it must sit at LDS address 0
    if ((uint32_t)(uintptr_t)(lds_ptr_t)smem != 0) {
        for (uint32_t t = tid; t < rows_here * (uint32_t)m; t += blockDim.x) {
            const uint32_t piece = (flags & kFlagPieces) ? blockIdx.x % k_split : 0u;
            if (y32) y32[((size_t)piece * m + t % m) * P.out_f + row0 + t / m] = __uint_as_float(0x7FC00000u);  // NaN
            else y[(int64_t)(t % m) * ldy + row0 + t / m] = 0x7FC0;
        }
        return;
    }
    const uint16_t scale_bits = *P.scale;  // asked for with the first requests, not where the pair table is built
    uint32_t *const lut = reinterpret_cast<uint32_t *>(smem);            // [64][32]
    uint4 *const splice = reinterpret_cast<uint4 *>(smem + kRLutBytes);  // [33][2]
    uint32_t *const tq1 = reinterpret_cast<uint32_t *>(smem + L.tq1);
    uint32_t *const tq2 = reinterpret_cast<uint32_t *>(smem + L.tq2);
    uint8_t *const wave_base = smem + L.waves + wave * L.wave_bytes;
    uint4 *const queue = reinterpret_cast<uint4 *>(wave_base);
    uint16_t *const tasks = reinterpret_cast<uint16_t *>(wave_base + L.tasks_off);

    const uint32_t unit0 = row0 * n_chunks;
    const uint32_t entries = P.out_f * n_chunks + 1;
    const uint32_t n_local = rows_here * n_chunks;
    // the ranks at the ends of the workgroup's rows (what its share of the side streams is worked out from): asked for
    // here, so that the share's words can be asked for with the rest of the set-up
    uint32_t q1b = 0, q2b = 0, q1e = 0, q2e = 0;
    if (!ANY) {
        q1b = (uint32_t)prefix[unit0], q2b = (uint32_t)prefix[entries + unit0];
        q1e = (uint32_t)prefix[unit0 + n_local], q2e = (uint32_t)prefix[entries + unit0 + n_local];
    }

    const __amdgpu_buffer_rsrc_t b1_rsrc =
        __builtin_amdgcn_make_buffer_rsrc((void *)P.bm[0], 0, (int)(P.bm_words[0] * 4u), 0x00020000);
    const __amdgpu_buffer_rsrc_t l1_rsrc =
        __builtin_amdgcn_make_buffer_rsrc((void *)P.st[0], 0, (int)(P.st_words[0] * 4u), 0x00020000);
    const __amdgpu_buffer_rsrc_t tb_rsrc =
        __builtin_amdgcn_make_buffer_rsrc((void *)prefix, 0, (int)(entries * 4u), 0x00020000);

    // ---- this wave's tile and its share of the column blocks of a part ----
    const uint32_t tile = wave / n_sub, sub = wave - tile * n_sub;
    const uint32_t trow0 = tile << lg_rows;
    const bool tile_live = trow0 < rows_here;                      // a wave beyond the workgroup's rows has nothing to do
    const bool row_live = trow0 + r < rows_here;                   // this lane's row exists
    const uint32_t lrow = min(trow0 + r, rows_here - 1);           // clamped: a lane without a row decodes zeros
    // the two things the loop needs of the lane's row: the index of its first unit (table entries, and bitmap words at
    // 16 a unit) and the row's part of a record
    const uint32_t base_u = row0 * n_chunks + lrow * n_chunks;
    const uint32_t rec_hi = (n << 27) | (lrow << 20);
    uint32_t part_first = (blockIdx.x - row_group * k_split) * k_blocks;  // the part's column blocks
    uint32_t part_count = min(x_blocks, kb_end - part_first);
    uint32_t c_begin = 0, c_end = 0;                                // this wave's run of them
    auto take_share = [&]() {  // in steps of `slots` column blocks
        const uint32_t steps = (part_count + slots - 1u) >> (4u - lg_rows);
        const uint32_t base = steps / n_sub, rem = steps - base * n_sub;
        c_begin = min(part_first + part_count, part_first + ((sub * base + min(sub, rem)) << (4u - lg_rows)));
        c_end = min(part_first + part_count, c_begin + ((base + (sub < rem ? 1u : 0u)) << (4u - lg_rows)));
        if (!tile_live) c_end = c_begin;
    };
    take_share();

    // what a lane needs for one task (its tile x one column block): requested first, so that it travels early
    struct TaskIn {
        uint32_t col;    // first column of the lane's strip; bit 31: the lane has no task (its row does not exist, or
                         // its slot's column block lies past the wave's run)
        uint32_t q1u;    // rank table entry of the row's unit
        u32x4 bm;        // the four bitmap words of the lane's strip
    };
    auto request = [&](uint32_t c0, TaskIn &T) {
        // the lane's k group and slot, worked out from a lane number the compiler cannot connect with the one
        // above: two instructions here instead of two registers held through the loop
        uint32_t l2 = threadIdx.x;
        asm volatile("" : "+v"(l2));
        const uint32_t kg2 = (l2 >> 4) & 3u, slot2 = (l2 & 15u) >> lg_rows;
        const uint32_t c = min(c0 + slot2, c_end - 1u);  // clamped: a lane without a block reads what exists
        T.col = c * kFastChunk + kg2 * 128u;
        T.q1u = __builtin_amdgcn_raw_buffer_load_b32(tb_rsrc, (int)((base_u + c) * 4u), 0, 0);
        T.bm = __builtin_amdgcn_raw_buffer_load_b128(b1_rsrc, (int)((((base_u + c) << 4) + kg2 * 4u) * 4u), 0, 0);
        if (!row_live || c0 + slot2 >= c_end) T.col |= 0x80000000u;
    };
    TaskIn T;
    if (c_begin < c_end) request(c_begin, T);

    // ---- workgroup set-up: activations, table slices, side streams, pair table, splice masks ----
    // activation rows of the part's columns into padded strips: 16-byte piece p of row i holds columns 8p .. 8p+7.
    // Eight loads of a thread in flight at a time, then their stores: one piece a trip to memory (a loop of load and
    // store) made a part of five column blocks at 16 activation rows eight trips long.  Row and piece are stepped, not
    // divided out, for every load.  (Named registers, not an array: the array went to scratch memory; a slot that no
    // thread of the workgroup needs is skipped by a scalar branch.)
#define IXH_T_LOAD(u)                                                                                              \
    const bool any##u = done + (uint32_t)(u) * stride < total;                                                      \
    uint4 v##u = make_uint4(0, 0, 0, 0);                                                                            \
    uint32_t at##u = ~0u;                                                                                           \
    if (any##u) {                                                                                                   \
        const bool live = tb + (uint32_t)(u) * stride < total;                                                      \
        v##u = *reinterpret_cast<const uint4 *>(x + (int64_t)(live ? i : 0u) * ldx + (first_piece + (live ? p : 0u)) * 8u); \
        if (live) at##u = L.xs + i * L.xs_row + (p >> 4) * kTStripBytes + (p & 15u) * 16u;                          \
        i += di;                                                                                                    \
        p += dp;                                                                                                    \
        if (p >= pieces) {                                                                                          \
            p -= pieces;                                                                                            \
            ++i;                                                                                                    \
        }                                                                                                           \
    }
#define IXH_T_STORE(u) \
    if (at##u != ~0u) *reinterpret_cast<uint4 *>(smem + at##u) = v##u;
#define IXH_T_LOAD_ALL IXH_T_LOAD(0) IXH_T_LOAD(1) IXH_T_LOAD(2) IXH_T_LOAD(3) IXH_T_LOAD(4) IXH_T_LOAD(5) IXH_T_LOAD(6) IXH_T_LOAD(7)
#define IXH_T_STORE_ALL IXH_T_STORE(0) IXH_T_STORE(1) IXH_T_STORE(2) IXH_T_STORE(3) IXH_T_STORE(4) IXH_T_STORE(5) IXH_T_STORE(6) IXH_T_STORE(7)
#define IXH_T_COPY_STATE                                                                                            \
    const uint32_t pieces = part_count * (kFastChunk / 8), first_piece = part_first * (kFastChunk / 8);             \
    uint32_t t0 = threadIdx.x;                                                                                      \
    asm volatile("" : "+v"(t0)); /* worked out anew at every call: no register is held for it across the loop */    \
    const uint32_t total = (uint32_t)m * pieces, stride = blockDim.x;                                               \
    const uint32_t di = stride / pieces, dp = stride - di * pieces;                                                 \
    uint32_t i = t0 / pieces, p = t0 - i * pieces;                                                                  \
    uint32_t tb = t0, done = 0;
    auto load_activations = [&]() __attribute__((always_inline)) {
        IXH_T_COPY_STATE
        for (; tb < total; tb += 8u * stride, done += 8u * stride) {
            IXH_T_LOAD_ALL
            IXH_T_STORE_ALL
        }
    };
    // The set-up's loads are all asked for before the first of them is stored: the first eight pieces of a thread's
    // activations, its first table entries, its first two words of the side streams.  One phase after the other, each
    // waiting for its own loads, the set-up was four trips to memory long.
    IXH_T_COPY_STATE
    IXH_T_LOAD_ALL
    const uint32_t n_tbl = n_local + 1u;
    const uint32_t tbl_i = min(tid, n_local);
    const uint32_t tbl_1 = (uint32_t)prefix[unit0 + tbl_i];
    const uint32_t tbl_2 = ANY ? 0u : (uint32_t)prefix[entries + unit0 + tbl_i];
    // this workgroup's share of bitmap 1 and of the 5-bit / 8-bit streams: small when few elements are above level 1,
    // then it is staged in LDS and resolving them touches no global memory
    SideView sv;
    sv.staged = false;
    sv.base = L.side;
    sv.b2w0 = sv.l2w0 = sv.l3w0 = 0;
    const uint32_t *const last32 = reinterpret_cast<const uint32_t *>(P.last);
    const uint32_t last_words = (P.last_bytes + 3u) >> 2;  // whole dwords (allocations are 256-byte granular)
    auto side_word = [&](uint32_t t) -> uint32_t {  // word t of the staged share (past a stream's end: zero)
        if (t < 256) {
            const uint32_t w = sv.b2w0 + t;
            return w < P.bm_words[1] ? P.bm[1][w] : 0u;
        }
        if (t < 768) {
            const uint32_t w = sv.l2w0 + (t - 256);
            return w < P.st_words[1] ? P.st[1][w] : 0u;
        }
        const uint32_t w = sv.l3w0 + (t - 768);
        return w < last_words ? last32[w] : 0u;
    };
    uint32_t side_0 = 0, side_1 = 0;
    if (!ANY) {
        const uint32_t nl1b = row0 * P.in_f - q1b, nl1e = (row0 + rows_here) * P.in_f - q1e;
        sv.b2w0 = nl1b >> 5;
        sv.l2w0 = (uint32_t)(((uint64_t)q2b * 5u) >> 5);
        sv.l3w0 = (nl1b - q2b) >> 2;
        const uint32_t n_b2 = ((nl1e + 31) >> 5) - sv.b2w0;
        const uint32_t n_l2 = (uint32_t)((((uint64_t)q2e * 5u) + 31) >> 5) - sv.l2w0;
        const uint32_t n_l3 = ((nl1e - q2e + 3) >> 2) - sv.l3w0;
        // one word of slack each: the resolver reads the word after a code's first word unconditionally
        sv.staged = (flags & kFlagStageSide) && n_b2 < 256 && n_l2 < 511 && n_l3 <= 256;
        if (sv.staged) {
            if (tid < kRSideBytes / 4) side_0 = side_word(tid);
            if (tid + blockDim.x < kRSideBytes / 4) side_1 = side_word(tid + blockDim.x);
        }
    }
    // what needs no memory: the strip of zeros (the pair table and the splice masks follow below)
    for (uint32_t t = tid; t < kTStripBytes / 4; t += blockDim.x) reinterpret_cast<uint32_t *>(smem + L.zero)[t] = 0u;
    // the stores, in the order of the requests, and what one request per thread did not cover
    IXH_T_STORE_ALL
    for (tb += 8u * stride, done += 8u * stride; tb < total; tb += 8u * stride, done += 8u * stride) {
        IXH_T_LOAD_ALL
        IXH_T_STORE_ALL
    }
    if (tid < n_tbl) {
        tq1[tid] = tbl_1;
        if (!ANY) tq2[tid] = tbl_2;
    }
    for (uint32_t i2 = tid + blockDim.x; i2 < n_tbl; i2 += blockDim.x) {
        tq1[i2] = (uint32_t)prefix[unit0 + i2];
        if (!ANY) tq2[i2] = (uint32_t)prefix[entries + unit0 + i2];
    }
    if (!ANY && sv.staged) {
        uint32_t *side = reinterpret_cast<uint32_t *>(smem + L.side);
        if (tid < kRSideBytes / 4) side[tid] = side_0;
        if (tid + blockDim.x < kRSideBytes / 4) side[tid + blockDim.x] = side_1;
        for (uint32_t t = tid + 2u * blockDim.x; t < kRSideBytes / 4; t += blockDim.x) side[t] = side_word(t);
    }
#undef IXH_T_COPY_STATE
#undef IXH_T_LOAD_ALL
#undef IXH_T_STORE_ALL
#undef IXH_T_LOAD
#undef IXH_T_STORE
    const float scale = bf16_bits_to_f32(scale_bits);
    for (uint32_t i = tid; i < 64 * 32; i += blockDim.x) {
        const int c0 = (i >> 5) & 7, c1 = i >> 8;
        const uint32_t w0 = c0 < 7 ? f32_to_bf16_bits((float)(c0 - 3) * scale) : 0u;
        const uint32_t w1 = c1 < 7 ? f32_to_bf16_bits((float)(c1 - 3) * scale) : 0u;
        lut[i] = w0 | (w1 << 16);
    }
    if (tid <= 32) {
        // entry e < 32: masks for a zero at element e (code bits 3e..3e+2): the bits below it, and its field;
        // entry 32: the identity (nothing to splice)
        const uint32_t pos = 3 * tid;
        uint32_t lm[3], f[3];
#pragma unroll
        for (int dd = 0; dd < 3; ++dd) {
            const uint32_t base = 32u * dd;
            lm[dd] = pos <= base ? 0u : (pos >= base + 32 ? ~0u : (1u << (pos - base)) - 1u);
            f[dd] = (pos + 3 <= base || pos >= base + 32) ? 0u : (pos >= base ? 7u << (pos - base) : 7u >> (base - pos));
        }
        splice[2 * tid] = make_uint4(lm[0], lm[1], lm[2], 0u);
        splice[2 * tid + 1] = make_uint4(f[0], f[1], f[2], 0u);
    }

    const uint32_t lut_lane = (lane & 31u) << 2;
    const uint32_t splice_addr = kRLutBytes;
    const uint32_t tq1_addr = L.tq1, tq2_addr = L.tq2;
    const uint32_t xs_addr = L.xs;
    // as row n of the other operand, lane n of each k group feeds activation row n % tile_rows at the columns of its
    // own slot's block (absent activation rows read zeros): the product of row a and column n of the operands means
    // something where their slots agree
    const uint32_t x_lane = r < (uint32_t)m ? L.xs + r * L.xs_row : L.zero;
    const uint32_t x_step = r < (uint32_t)m ? kTStripBytes : 0u;  // bytes from strip to strip

    f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};  // D[4 kg + i][n]: activation rows 4 kg .. 4 kg + 3 x this lane's weight row

    uint32_t qcount = 0;  // wave-uniform
    auto resolve = [&]() {
        TileSink sink{acc, n, kg, r * L.xs_row, r < (uint32_t)m, xs_addr, 0u, xs_addr, n_chunks,
                      L.waves + wave * L.wave_bytes + L.round_off};
        const TaskPool none{0, 0, 0, 1, 0, 0};
        if (ANY)
            resolve_rows_to<kTMaxM, false, true, 2, false, kTStripBytes>(
                sink, P, sv, tq1_addr, tq2_addr, unit0, queue, qcount, 0u, tasks, xs_addr, L.xs_row,
                part_first * kFastChunk, m, scale, lane, prefix, entries, none);
        else if (sv.staged)
            resolve_rows_to<kTMaxM, true, false, 2, false, kTStripBytes>(
                sink, P, sv, tq1_addr, tq2_addr, unit0, queue, qcount, 0u, tasks, xs_addr, L.xs_row,
                part_first * kFastChunk, m, scale, lane, nullptr, 0, none);
        else
            resolve_rows_to<kTMaxM, false, false, 2, false, kTStripBytes>(
                sink, P, sv, tq1_addr, tq2_addr, unit0, queue, qcount, 0u, tasks, xs_addr, L.xs_row,
                part_first * kFastChunk, m, scale, lane, nullptr, 0, none);
        acc = sink.acc;
        qcount = 0;
    };

    auto splice_once = [&](uint32_t &w0, uint32_t &w1, uint32_t &w2, uint32_t &zrem) {
        const uint32_t e = zrem != 0 ? (uint32_t)__builtin_ctz(zrem) : 32u;
        zrem &= zrem - 1;
        const u32x4 lm = lds_u128(splice_addr + e * 32), fm = lds_u128(splice_addr + e * 32 + 16);
        const uint32_t s0 = w0 << 3;
        const uint32_t s1 = __builtin_amdgcn_alignbit(w1, w0, 29);
        const uint32_t s2 = __builtin_amdgcn_alignbit(w2, w1, 29);
        w0 = (w0 & lm.x) | (s0 & ~lm.x);
        w1 = (w1 & lm.y) | (s1 & ~lm.y);
        w2 = (w2 & lm.z) | (s2 & ~lm.z);
        w0 = (w0 & ~fm.x) | (kZeroCodes0 & fm.x);
        w1 = (w1 & ~fm.y) | (kZeroCodes1 & fm.y);
        w2 = (w2 & ~fm.z) | (kZeroCodes2 & fm.z);
    };

    // (the barrier that ends the set-up comes after the first task's codes have been asked for, below)

    // A task in flight: the ranks at which its words start and the stream bytes asked for with them.
    struct Stage {
        uint32_t word[4];  // bitmap words
        uint32_t first;    // level-1 elements before the strip's first word (global rank)
        u32x4 code[4];     // the 16 stream bytes that hold each word's codes (address = 3 x rank)
        uint32_t col;      // as in TaskIn
        uint32_t records;  // wave-uniform: lanes x words with elements above level 1, the records the task will queue
    };
    // second step of a task: from table entry and bitmap words to the ranks, and the requests for the codes
    auto launch_codes = [&](const TaskIn &T, Stage &S) {
        S.col = T.col;
        u32x4 b = T.bm;
        if ((int)T.col < 0) b = u32x4{~0u, ~0u, ~0u, ~0u};  // a lane without a task: no records, and zero codes below
        S.word[0] = b.x; S.word[1] = b.y; S.word[2] = b.z; S.word[3] = b.w;
        S.records = (uint32_t)(__popcll(__ballot(b.x != ~0u)) + __popcll(__ballot(b.y != ~0u)) +
                               __popcll(__ballot(b.z != ~0u)) + __popcll(__ballot(b.w != ~0u)));
        const uint32_t p1 = __popc(b.x), p2 = p1 + __popc(b.y), p3 = p2 + __popc(b.z), p4 = p3 + __popc(b.w);
        // level-1 elements of the unit's strips before this one: they are 16, 32 and 48 lanes down
        const uint32_t d1 = (uint32_t)__builtin_amdgcn_ds_bpermute((int)((lane - 16u) * 4u), (int)p4);
        const uint32_t d2 = (uint32_t)__builtin_amdgcn_ds_bpermute((int)((lane - 32u) * 4u), (int)p4);
        const uint32_t d3 = (uint32_t)__builtin_amdgcn_ds_bpermute((int)((lane - 48u) * 4u), (int)p4);
        const uint32_t before = (kg >= 1 ? d1 : 0u) + (kg >= 2 ? d2 : 0u) + (kg >= 3 ? d3 : 0u);
        const uint32_t first = T.q1u + before;
        S.first = first;
        const uint32_t rank[4] = {first, first + p1, first + p2, first + p3};
#pragma unroll
        for (int k = 0; k < 4; ++k)
            S.code[k] = __builtin_amdgcn_raw_buffer_load_b128(l1_rsrc, (int)(((rank[k] * 3u) >> 5) * 4u), 0, 0);
    };

    // third step: decode and multiply the task's words
    auto compute = [&](Stage &S) {
        // the lane's strip of its activation row in LDS
        const uint32_t x_strip = x_lane + (((S.col & 0x7FFFFFFFu) >> 7) - part_first * 4u) * x_step;
        // a lane without a task looks up pair (7, 7) whatever it decodes: the table's zero
        const uint32_t lut_x = lut_lane | ((uint32_t)((int)S.col >> 31) & 0x1F80u);
        uint32_t rk = S.first;  // level-1 elements before the word
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const u32x4 dq = S.code[k];
            const uint32_t off = rk * 3u;  // v_alignbit takes the low five bits
            uint32_t w0 = __builtin_amdgcn_alignbit(dq.y, dq.x, off);
            uint32_t w1 = __builtin_amdgcn_alignbit(dq.z, dq.y, off);
            uint32_t w2 = __builtin_amdgcn_alignbit(dq.w, dq.z, off);
            uint32_t zrem = ~S.word[k];
            const uint64_t any = __ballot(zrem != 0);
            if (any != 0) {  // lanes with elements above level 1 leave a record
                if (zrem != 0) {
                    const uint32_t kw = (S.col >> 5) + (uint32_t)k;  // column / 32
                    const uint32_t rel = rk - lds_u32(tq1_addr + (base_u - unit0 + (S.col >> 9)) * 4u);
                    push_record8(queue, qcount + lanes_below(any), zrem, rec_hi | (kw << 9) | rel);
                }
                qcount += (uint32_t)__popcll(any);
                do splice_once(w0, w1, w2, zrem);
                while (__ballot(zrem != 0) != 0);
            }
            // sixteen code pairs through the pair table and the word's activations, eight columns per matrix
            // instruction; in two halves, so that a half's operands are all that is in registers at a time
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                u32x4 xa[2];
#pragma unroll
                for (int s = 0; s < 2; ++s)
                    xa[s] = lds_u128(x_strip + (uint32_t)k * 64u + (uint32_t)(2 * half + s) * 16u);
                uint32_t wp[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    const int bit = 6 * (8 * half + u), ob = bit & 31, dd = bit >> 5;
                    const uint32_t lo = dd == 0 ? w0 : (dd == 1 ? w1 : w2);
                    const uint32_t hi = dd == 0 ? w1 : w2;
                    uint32_t a;  // pair index at bits 12..7
                    if (ob > 26) a = __builtin_amdgcn_alignbit(hi, lo, ob - 7);
                    else if (ob >= 7) a = lo >> (ob - 7);
                    else a = lo << (7 - ob);
                    wp[u] = lds_u32((a & 0x1F80u) | lut_x);
                }
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                    const u32x4 b4 = u32x4{wp[4 * s], wp[4 * s + 1], wp[4 * s + 2], wp[4 * s + 3]};
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, xa[s]),
                                                                 __builtin_bit_cast(bf16x8, b4), acc, 0, 0, 0);
                }
                if (half == 0) __builtin_amdgcn_sched_barrier(0);
            }
            rk += (uint32_t)__popc(S.word[k]);
        }
    };

    // Three steps per task, each one task ahead of the next: table entry + bitmap words (request), ranks and code
    // requests (launch_codes), decode (compute).  Two stages take turns, so nothing is copied between iterations.
    // The first task's codes are asked for before the barrier that ends the set-up, and travel across it (no fence:
    // this wave's LDS stores have completed, and the loads in flight are nobody else's business).
    auto lds_barrier = [&]() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };
    for (bool later = false;; later = true) {
        const bool mine = c_begin < c_end;
        Stage A, B;
        if (mine) {
            launch_codes(T, A);
            if (c_begin + slots < c_end) request(c_begin + slots, T);
        }
        if (later) {
            // the next part of the columns (the last part's elements above level 1 have met its activations): the
            // copy travels together with the first task's codes
            lds_barrier();  // nobody reads the old part any more
            load_activations();
        }
        lds_barrier();  // the set-up, or the part's activations, are in LDS
        if (mine) {
            // The queue is emptied between tasks, where one stage is dead and registers are free: before a task whose
            // records (at most 4 x 64 = the queue's capacity) would not fit behind those that wait.
            for (uint32_t c = c_begin; c < c_end; c += 2 * slots) {
                if (qcount + A.records > qcap) resolve();
                if (c + slots < c_end) {
                    launch_codes(T, B);
                    if (c + 2 * slots < c_end) request(c + 2 * slots, T);
                }
                compute(A);
                if (c + slots < c_end) {
                    if (qcount + B.records > qcap) resolve();
                    if (c + 2 * slots < c_end) {
                        launch_codes(T, A);
                        if (c + 3 * slots < c_end) request(c + 3 * slots, T);
                    }
                    compute(B);
                }
            }
        }
        if (part_first + part_count >= kb_end) break;
        // this part's elements above level 1 meet its activations while they are there
        resolve();
        part_first = (uint32_t)__builtin_amdgcn_readfirstlane((int)(part_first + part_count));
        part_count = min(x_blocks, kb_end - part_first);
        take_share();
        if (c_begin < c_end) request(c_begin, T);
    }
    resolve();

    // ---- the wave's accumulators into the sub-range's slot; after the barrier the outputs are summed over the
    // sub-ranges, each with what its wave added for the elements above level 1 ----
    __syncthreads();  // the accumulators go where the activations were
    {
        // the lane holds rows 4 kg .. 4 kg + 3 of the product's column n: those of its own slot are the sums of
        // activation rows (4 kg + i) % tile_rows.  The lane's place is worked out anew (from a lane number the
        // compiler cannot connect with the one above), so that no register carries it through the kernel.
        uint32_t l2 = threadIdx.x & 63u;
        asm volatile("" : "+v"(l2));
        const uint32_t n2 = l2 & 15u, kg2 = l2 >> 4, r2 = n2 & (tile_rows - 1u), slot2 = n2 >> lg_rows;
        if (trow0 + r2 < rows_here) {
            float *const partial = reinterpret_cast<float *>(smem + L.partial) +
                                   ((sub * slots + slot2) * rows_cap + trow0 + r2) * (uint32_t)m;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint32_t a = 4u * kg2 + i, j = a & (tile_rows - 1u);
                if ((a >> lg_rows) == slot2 && j < (uint32_t)m) partial[j] = acc[i];
            }
        }
    }
    __syncthreads();
    for (uint32_t t = tid; t < rows_here * (uint32_t)m; t += blockDim.x) {
        const uint32_t row = t / (uint32_t)m, i = t - row * (uint32_t)m;
        float sum = 0.0f;
        for (uint32_t s = 0; s < n_sub; ++s) {
            for (uint32_t q = 0; q < slots; ++q)
                sum += reinterpret_cast<const float *>(smem + L.partial)[((s * slots + q) * rows_cap + row) * (uint32_t)m + i];
        }
        if (y32 && (flags & kFlagPieces)) y32[((size_t)(blockIdx.x % k_split) * m + i) * P.out_f + row0 + row] = sum;
        else if (y32) atomicAdd(&y32[(size_t)i * P.out_f + row0 + row], sum);
        else y[(int64_t)i * ldy + row0 + row] = (uint16_t)f32_to_bf16_bits(sum);
    }
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
struct TilesPlan {
    uint32_t rows, n_sub, x_blocks, qcap, waves, lg_rows, k_split, k_blocks;
    float cost;
};

// Rows per workgroup (whole rounds of one workgroup per CU, a multiple of four), the tile shape, waves per tile, the
// part of the activation rows that LDS holds at a time, and the number of workgroups that share a block of rows, each
// taking a run of its column blocks.  A tile of 16 >> k rows takes 1 << k column blocks per step and serves 16 >> k
// activation rows, so short tiles suit workgroups whose rows are not a multiple of 16 when the rows of activations are
// few.  A wave's time goes with the steps it decodes, and every further part costs two barriers and a copy: the plan
// with the fewest steps per wave, a part counted as 0.6 of a step (costs that also count the steps of all waves of
// a CU, or of a SIMD, chose slower plans on the shapes measured).  Sharing the rows' columns among k workgroups makes
// the row blocks k times as tall, which fills tiles of 16 that a short block leaves mostly empty and takes k times
// fewer parts per workgroup; it costs the second launch that adds the pieces (kSplitCost steps).
// In steps: a further part (the wait at its two barriers and the loop's restart), a round's set-up and final sums,
// the second launch.
constexpr float kPartCost = 0.6f, kSetupCost = 2.5f, kSplitCost = 0.9f;
static TilesPlan plan_tiles(uint32_t out_f, uint32_t n_chunks, uint32_t n_cu, int m, int lg_only, uint32_t max_split,
                            uint32_t split_only) {
    const uint32_t n_quads = (out_f + 3) / 4, max_quads = kTMaxRows / 4;
    TilesPlan best{0, 0, 0, 0, 0, 4, 1, 0, 0.0f};
    for (uint32_t k_split = 1; k_split <= min(min(max_split, 8u), n_chunks); ++k_split) {
        if (split_only != 0 && k_split != split_only) continue;
        const uint32_t k_blocks = (n_chunks + k_split - 1) / k_split;
        if ((n_chunks + k_blocks - 1) / k_blocks != k_split) continue;  // a piece would be empty
        const uint32_t per_round = max(1u, n_cu / k_split);             // blocks of rows at a time
        const uint32_t rounds = (n_quads + per_round * max_quads - 1) / (per_round * max_quads);
        const uint32_t rows = 4u * max(1u, min(max_quads, (n_quads + rounds * per_round - 1) / (rounds * per_round)));
        for (uint32_t lg = 4; lg >= 2; --lg) {
            if (lg_only >= 2 && (uint32_t)lg_only != lg) continue;
            const uint32_t tile_rows = 1u << lg, slots = 16u >> lg;
            if ((uint32_t)m > tile_rows) break;
            const uint32_t tiles = (rows + tile_rows - 1) / tile_rows;
            if (tiles > (uint32_t)kTMaxWaves) continue;
            for (uint32_t parts = 1; parts <= k_blocks; ++parts) {
                const uint32_t x_blocks = (k_blocks + parts - 1) / parts;
                if ((k_blocks + x_blocks - 1) / x_blocks != parts) continue;  // the same parts with fewer blocks each: seen
                const uint32_t steps = (x_blocks + slots - 1) / slots;      // of the longest part
                TilesPlan here{0, 0, 0, 0, 0, lg, k_split, k_blocks, 0.0f};
                for (uint32_t n_sub = min((uint32_t)kTMaxWaves / tiles, steps); n_sub >= 1 && here.waves == 0; --n_sub) {
                    const uint32_t qcap = kTQueue;
                    if (tiles_layout(rows, n_chunks, x_blocks, n_sub * slots, tiles * n_sub, m, qcap).total > kTLdsLimit)
                        continue;
                    // no more waves than shorten the longest run of steps
                    const uint32_t run = (steps + n_sub - 1) / n_sub;
                    const uint32_t subs = (steps + run - 1) / run;
                    uint32_t per_wave = 0;  // of the longest piece, the first
                    for (uint32_t first = 0; first < k_blocks; first += x_blocks) {
                        const uint32_t st = (min(x_blocks, k_blocks - first) + slots - 1) / slots;
                        per_wave += (st + subs - 1) / subs;
                    }
                    here.rows = rows, here.n_sub = subs, here.x_blocks = x_blocks, here.qcap = qcap;
                    here.waves = tiles * subs;
                    here.cost = (float)rounds * ((float)per_wave + (float)(parts - 1) * kPartCost + kSetupCost) +
                                (k_split > 1 ? kSplitCost : 0.0f);
                }
                if (here.waves != 0 && (best.waves == 0 || here.cost < best.cost)) best = here;
                if (here.waves != 0 && here.waves >= tiles * min((uint32_t)kTMaxWaves / tiles, steps) && parts > 1 &&
                    here.cost > best.cost)
                    break;  // more parts only add to the cost from here on
            }
        }
    }
    return best;
}

template <bool ANY>
static int launch_tiles(const Dev &P, const int32_t *prefix, uint32_t n_chunks, const TilesPlan &plan, const uint16_t *x,
                        int m, int64_t ldx, uint16_t *y, int64_t ldy, float *y32, float *ws, hipStream_t s) {
    static const bool raised =  // per instantiation
        hipFuncSetAttribute(reinterpret_cast<const void *>(k_gemv358_tiles<ANY>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)kTLdsLimit) == hipSuccess;
    if (!raised) return IXH_EUNSUPPORTED;
    const uint32_t groups = (P.out_f + plan.rows - 1) / plan.rows;
    const size_t lds =
        tiles_layout(plan.rows, n_chunks, plan.x_blocks, plan.n_sub * (16u >> plan.lg_rows), plan.waves, m, plan.qcap).total;
    if (lds > kTLdsLimit) return IXH_EUNSUPPORTED;
    // every piece has column blocks (the kernel's part loop counts on it)
    if (plan.k_split < 1 || plan.k_blocks < 1 || (uint64_t)(plan.k_split - 1) * plan.k_blocks >= n_chunks ||
        (uint64_t)plan.k_split * plan.k_blocks < n_chunks)
        return IXH_EUNSUPPORTED;
    const bool pieces = plan.k_split > 1 && !y32;
    if (pieces && !ws) return IXH_EUNSUPPORTED;
    uint32_t flags = 0;
    if (((uintptr_t)P.last & 3u) == 0) flags |= kFlagStageSide;
    if (pieces) flags |= kFlagPieces;
    hipLaunchKernelGGL((k_gemv358_tiles<ANY>), dim3(groups * plan.k_split), dim3(plan.waves * kWave), lds, s, P, prefix,
                       n_chunks, plan.rows, plan.n_sub, plan.x_blocks, plan.lg_rows, flags,
                       plan.k_split | (plan.k_blocks << 8), x, m, ldx, pieces ? nullptr : y, ldy, pieces ? ws : y32);
    if (hipGetLastError() != hipSuccess) return IXH_ELAUNCH;
    return pieces ? launch_reduce_chunks(ws, plan.k_split, m, P.out_f, y, ldy, s) : IXH_OK;
}

// The tile kernel: up to 16 activation rows, rows of whole 512-column blocks, row counts that are multiples of four;
// IXH_EUNSUPPORTED sends the caller on to the other row-block kernels.  ws: room for ws_pieces x m x out_f fp32 sums
// (none: every workgroup takes whole rows).
int launch_gemv_358_tiles(const Dev &P, const int32_t *prefix, const uint16_t *x, int m, int64_t ldx, uint16_t *y,
                          int64_t ldy, float *y32, float *ws, uint32_t ws_pieces, hipStream_t s) {
    if (m < 1 || m > kTMaxM || P.out_f % 4u != 0 || P.in_f % kFastChunk != 0 || P.in_f > 65536u) return IXH_EUNSUPPORTED;
    if (((uintptr_t)x & 15u) != 0 || (m > 1 && (ldx & 7) != 0)) return IXH_EUNSUPPORTED;
    const int opt = g_opt_gemv_tiles.load(std::memory_order_relaxed);  // ixh_set_option("gemv_tiles")
    if (opt < 0) return IXH_EUNSUPPORTED;
    const bool any = !(P.n_levels == 3 && P.bits[1] == 5);  // not (3,5,8): the resolver that walks the nested bitmaps
    static const int n_cu = [] {
        int dev = 0, v = 256;
        if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev);
        return v;
    }();
    const uint32_t n_chunks = P.in_f / kFastChunk;
    const int cus_opt = g_opt_gemv_tile_cus.load(std::memory_order_relaxed);
    const int split_opt = g_opt_gemv_tile_split.load(std::memory_order_relaxed);
    // pieces need the workspace, or the caller's fp32 sums, which the workgroups add to one by one anyway
    const uint32_t max_split = y32 ? 8u : (ws ? ws_pieces : 1u);
    const TilesPlan plan = plan_tiles(P.out_f, n_chunks, (uint32_t)(cus_opt > 0 ? cus_opt : n_cu), m,
                                      g_opt_gemv_tile_rows.load(std::memory_order_relaxed), max(1u, max_split),
                                      (uint32_t)(split_opt > 0 ? split_opt : 0));
    if (plan.waves == 0) return IXH_EUNSUPPORTED;
    // by itself from three activation rows on (one or two: the kernels that multiply lane by lane are as fast or faster)
    // and where a workgroup's rows fill its tiles of 16 at least half; forced (option 1) wherever it fits
    const uint32_t tile_rows = 1u << plan.lg_rows;
    if (opt == 0 && (m <= 2 || plan.rows * 2u < ((plan.rows + tile_rows - 1u) / tile_rows) * tile_rows))
        return IXH_EUNSUPPORTED;
    return any ? launch_tiles<true>(P, prefix, n_chunks, plan, x, m, ldx, y, ldy, y32, ws, s)
               : launch_tiles<false>(P, prefix, n_chunks, plan, x, m, ldx, y, ldy, y32, ws, s);
}

}  // namespace ixh
