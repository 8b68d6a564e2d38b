// The 128-row tile kernel of ixh_gemm for tensors that are almost all level 1 with a 3-bit first level
// (ixh_prefill358.hip), and the reduction kernel of ixh_prefill.hip.  Internal to the library.
#pragma once
#include "ixh_dev.h"

namespace ixh {

int launch_prefill_reduce(const float *ws, uint32_t m_rows, uint32_t out_f, uint32_t n_slices, uint16_t *y, int64_t ldy,
                          hipStream_t s);
size_t prefill358_workspace_bytes(const Dev &P, uint32_t m_rows);
bool prefill358_supports(const Dev &P, const uint16_t *x, int64_t ldx);
// flags & 1: no value lists, every element above level 1 is computed where it is needed (testing)
int launch_prefill358(const Dev &P, const int32_t *prefix, const uint16_t *x, uint32_t m_rows, int64_t ldx, uint16_t *y,
                      int64_t ldy, float *ws, uint32_t flags, hipStream_t s);
// ixh_set_option("gemm_tiles"): -1 = never, 0 = where it pays, 1 = wherever it fits, 2 = as 1 without value lists
extern std::atomic<int> g_opt_gemm_tiles;

}  // namespace ixh
