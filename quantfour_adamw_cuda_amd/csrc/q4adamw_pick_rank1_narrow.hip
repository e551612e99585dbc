// The instantiations of fused_4bit_rank1_kernel<..., kTileNarrow> (rank-1 update) and their selection.
#include <hip/hip_runtime.h>

#include "q4adamw_pick.h"
#include "q4adamw_step.h"

namespace q4 {

template <bool EXT, bool SR, bool EXACT>
static Rank1Kernel pick_pg(int p_dtype, int g_dtype) {
  Q4_PICK_PG(fused_4bit_rank1_kernel, EXT, SR, kTileNarrow, EXACT)
}

template <bool EXT, bool SR>
static Rank1Kernel pick_exact(int p_dtype, int g_dtype, bool exact) {
  return exact ? pick_pg<EXT, SR, true>(p_dtype, g_dtype) : pick_pg<EXT, SR, false>(p_dtype, g_dtype);
}

Rank1Kernel pick_rank1_narrow(int p_dtype, int g_dtype, bool ext, bool sr, bool exact) {
  if (sr) return ext ? pick_exact<true, true>(p_dtype, g_dtype, exact) : pick_exact<false, true>(p_dtype, g_dtype, exact);
  return ext ? pick_exact<true, false>(p_dtype, g_dtype, exact) : pick_exact<false, false>(p_dtype, g_dtype, exact);
}

}  // namespace q4
