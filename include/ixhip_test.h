/*
 * ixhip_test -- the testing and measurement hook of libixhip.so.
 *
 * Not part of the product interface declared in ixhip.h: nothing here has a counterpart in the reference, and a
 * caller that only decodes and multiplies never needs it.  The library's own tests, its benchmark and its profiles
 * use it to run one kernel where the library would choose another.  The switches are process-wide and read at every
 * call, so a program that sets one changes every later call of every thread: set them from test harnesses only.
 */
#ifndef IXHIP_TEST_H
#define IXHIP_TEST_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/*
 * Overrides, for the whole process, a choice the
 * library otherwise makes from the tensor (the defaults are what every other caller gets):
 *   "decode_kernel"  0 = by the tensor (default), 1 = the row-block decoder, 2 = the level-by-level decoder,
 *                    3 = the staged decoder, 4 = the wave-per-unit decoder; a named decoder that cannot take a
 *                    call is skipped for that call
 *   "gemv_shared_x"  most activation rows (0..8, default 8) that ixh_gemv gives to the row-block kernel that
 *                    shares the activations through on-chip memory; 0 = never
 *   "gemv_tiles"     the tile kernel (16, 8 or 4 weight rows x up to 16, 8 or 4 activation rows per matrix
 *                    instruction): -1 = never, 0 = where it pays (three activation rows or more, tiles at least half
 *                    full; default), 1 = wherever it fits
 *   "gemv_tile_rows" the tile kernel's tile shape: 0 = the planner's choice (default), 2 / 3 / 4 = tiles of 4 / 8 / 16
 *                    weight rows only (a shape that cannot serve the call's activation rows hands the call on)
 *   "gemv_tile_split" the number of workgroups of the tile kernel that share a block of rows, each taking a run of its
 *                    column blocks, their sums added by a second launch (needs the workspace of ixh_gemv): 0 = the
 *                    planner's choice (default), 1..8 = that many where the workspace allows
 *   "gemv_tile_cus"  the number of CUs over which the tile kernel's planner spreads the rows: 0 = the device's
 *                    (default), 1..4096 = that many (small tensors then get workgroups with several tiles); also the
 *                    number of workgroups of the dense-mix matrix-pipe kernel
 *   "gemv_dense_tiles" the level-by-level kernels for dense mixes that multiply on the matrix pipe (2..16
 *                    activation rows): -1 = never, 0 = (3,5,8) from four rows on, (3,4,5,6,8) from two (default),
 *                    1 = both from two rows on
 *   "gemv_strips"    the strip kernel (up to eight activation rows a pass): -1 = never, 0 = for three rows or more
 *                    where the tile kernel does not run and the shape fits (default), 1..6 = wherever it fits
 *   "gemv_slots"     the row-block kernel that multiplies on the matrix pipe (one to four activation rows): -1 = never,
 *                    0 = where it is the fastest (two rows on layers that give a workgroup at least 128 unit quads;
 *                    default), 1 = wherever it fits
 *   "gemv_slot_waves" waves per workgroup of that kernel: 0 = the planner's choice (default), 8..16 = that many
 * Returns IXH_EINVAL for an unknown name or a value out of range.  Calls already running are not affected.
 */
int ixh_set_option(const char *name, int64_t value);

#ifdef __cplusplus
}
#endif

#endif /* IXHIP_TEST_H */
