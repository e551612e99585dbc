// Which kernel a call takes.  The step kernels are templates over element types, gradient
// options, rounding and the parameter update's form; their instantiations are spread over
// several translation units (q4adamw_pick_*.hip) so that a build compiles them side by side.
#pragma once
#include "q4adamw_args.h"

namespace q4 {

typedef void (*FusedKernel)(const FusedArgs);
typedef void (*SmallKernel)(const SmallArgs);
typedef void (*Rank1Kernel)(const Rank1Args);
typedef void (*Rank1StatKernel)(const Rank1StatArgs);

// Kernel of a family for the (parameter, gradient) element types of a call: the tags
// 0 = fp32, 1 = bf16, 2 = fp16 become template arguments.
#define Q4_PICK_PG(KERNEL, ...)                                                   \
  switch (p_dtype * 3 + g_dtype) {                                                \
    case 0: return KERNEL<0, 0, __VA_ARGS__>;                                     \
    case 1: return KERNEL<0, 1, __VA_ARGS__>;                                     \
    case 2: return KERNEL<0, 2, __VA_ARGS__>;                                     \
    case 3: return KERNEL<1, 0, __VA_ARGS__>;                                     \
    case 4: return KERNEL<1, 1, __VA_ARGS__>;                                     \
    case 5: return KERNEL<1, 2, __VA_ARGS__>;                                     \
    case 6: return KERNEL<2, 0, __VA_ARGS__>;                                     \
    case 7: return KERNEL<2, 1, __VA_ARGS__>;                                     \
    default: return KERNEL<2, 2, __VA_ARGS__>;                                    \
  }

// ext: gradient options; sr: stochastic rounding; exact: the parameter update with every
// operation rounded as IEEE 754 rounds it
FusedKernel pick_fused(int p_dtype, int g_dtype, bool ext, bool sr, bool exact);
// the rank-1 update kernels: tiles anywhere in a matrix of rows at least a tile long
// (pick_rank1_wide), matrices narrower than a tile (pick_rank1_narrow), tiles aligned to the
// rows of a matrix (pick_rank1_rows), rows of any length (pick_rank1_any)
Rank1Kernel pick_rank1_wide(int p_dtype, int g_dtype, bool ext, bool sr, bool exact);
Rank1Kernel pick_rank1_narrow(int p_dtype, int g_dtype, bool ext, bool sr, bool exact);
Rank1Kernel pick_rank1_rows(int p_dtype, int g_dtype, bool ext, bool sr, bool exact);
Rank1Kernel pick_rank1_any(int p_dtype, int g_dtype, bool ext, bool sr, bool exact);

}  // namespace q4
