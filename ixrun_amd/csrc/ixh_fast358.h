// Specialised (3,5,8) fused decode+GEMV for gfx950 (see ixh_fast358.hip).
#pragma once
#include "ixh_dev.h"

namespace ixh {

constexpr uint32_t kFastChunk = 512;  // elements per table unit the kernel is built around

// true when launch_gemv_358 can serve the request (otherwise the caller uses the general kernel)
bool fast358_supports(const Dev &P, uint32_t chunk, int m);
// x / ld alignment is checked at launch; returns IXH_EUNSUPPORTED if it does not fit
int launch_gemv_358(const Dev &P, const int32_t *prefix, uint32_t chunk, const uint16_t *x, int m, int64_t ldx,
                    uint16_t *y, int64_t ldy, float *y32, float *ws, bool atomic, hipStream_t s);
// single-launch row-block kernel (ixh_rows358.hip); IXH_EUNSUPPORTED if the shape does not fit it.  y32 == nullptr:
// bf16 results to y; otherwise the fp32 row sums are added into y32 [m, out_f] (one addition per output) and y is
// not touched
int launch_gemv_358_rows(const Dev &P, const int32_t *prefix, const uint16_t *x, int m, int64_t ldx, uint16_t *y,
                         int64_t ldy, float *y32, hipStream_t s);
// slot kernel (ixh_slots358.hip): the row-block decode with the products on the matrix pipe, up to four activation
// rows, rows a multiple of four; same contract
int launch_gemv_358_slots(const Dev &P, const int32_t *prefix, const uint16_t *x, int m, int64_t ldx, uint16_t *y,
                          int64_t ldy, float *y32, hipStream_t s);
// strip kernel (ixh_strips358.hip): up to four activation rows, products on the matrix pipe; same contract
int launch_gemv_358_strips(const Dev &P, const int32_t *prefix, const uint16_t *x, int m, int64_t ldx, uint16_t *y,
                           int64_t ldy, float *y32, hipStream_t s);
// tile kernel (ixh_tiles358.hip): 16 weight rows x up to 16 activation rows per matrix instruction; same contract.
// ws: room for ws_pieces x m x out_f fp32 sums (or none), for plans in which several workgroups share a block of rows
int launch_gemv_358_tiles(const Dev &P, const int32_t *prefix, const uint16_t *x, int m, int64_t ldx, uint16_t *y,
                          int64_t ldy, float *y32, float *ws, uint32_t ws_pieces, hipStream_t s);
// level-by-level kernel for one activation row and mixes with many elements above level 1 (ixh_dense358.hip)
bool gemv_dense358_supports(const Dev &P, uint32_t chunk, int m, const uint16_t *x);
int launch_gemv_dense358(const Dev &P, const int32_t *prefix, const uint16_t *x, uint16_t *y, float *y32, float *ws,
                         bool atomic, hipStream_t s);
// the same for the five-level scheme (3,4,5,6,8), one activation row (ixh_dense5.hip)
bool gemv_dense34568_supports(const Dev &P, uint32_t chunk, int m, const uint16_t *x);
int launch_gemv_dense34568(const Dev &P, const int32_t *prefix, const uint16_t *x, uint16_t *y, float *y32, float *ws,
                           bool atomic, hipStream_t s);
bool decode_dense34568_supports(const Dev &P, uint32_t chunk, const int8_t *o8, const uint16_t *o16);
int launch_decode_dense34568(const Dev &P, const int32_t *prefix, uint16_t *o16, hipStream_t s);
bool gemv_dense34568_tiles_supports(const Dev &P, uint32_t chunk, int m, const uint16_t *x, int64_t ldx);
int launch_gemv_dense34568_tiles(const Dev &P, const int32_t *prefix, const uint16_t *x, int m, int64_t ldx, uint16_t *y,
                                 int64_t ldy, float *ws, hipStream_t s);
bool gemv_dense358_tiles_supports(const Dev &P, uint32_t chunk, int m, const uint16_t *x, int64_t ldx);
int launch_gemv_dense358_tiles(const Dev &P, const int32_t *prefix, const uint16_t *x, int m, int64_t ldx, uint16_t *y,
                               int64_t ldy, float *ws, hipStream_t s);
bool gemv_dense358_rows_supports(const Dev &P, uint32_t chunk, int m, const uint16_t *x, int64_t ldx);
int launch_gemv_dense358_rows(const Dev &P, const int32_t *prefix, const uint16_t *x, int m, int64_t ldx, uint16_t *y,
                              int64_t ldy, float *ws, hipStream_t s);
bool decode_rows358_supports(const Dev &P, uint32_t chunk, const int8_t *o8, const uint16_t *o16);
int launch_decode_rows358(const Dev &P, const int32_t *prefix, uint16_t *o16, hipStream_t s);
bool decode_dense358_supports(const Dev &P, uint32_t chunk, const int8_t *o8, const uint16_t *o16, GroupScales gs);
int launch_decode_dense358(const Dev &P, const int32_t *prefix, uint16_t *o16, GroupScales gs, hipStream_t s);
int launch_reduce_chunks(const float *ws, uint32_t n_chunks, int m, uint32_t out_f, uint16_t *y, int64_t ldy,
                         hipStream_t s);

}  // namespace ixh
