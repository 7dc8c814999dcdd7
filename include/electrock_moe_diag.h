/*
 * electrock_moe_diag.h -- diagnostic switches of em_moe_forward and its variants, for benchmarks and tests.
 * Not part of the drop-in surface: a serving caller never sets them.  They are flag bits like those of
 * electrock_moe.h and may be OR-ed into the `flags` argument of the layer entry points.
 */
#ifndef ELECTROCK_MOE_DIAG_H
#define ELECTROCK_MOE_DIAG_H

#include "electrock_moe.h"

/* Stage masks: skip a stage and reuse what an earlier call with the same shapes left in `workspace`
 * (used to time one stage in isolation). */
#define EM_FLAG_SKIP_ROUTER    (1u << 8)
#define EM_FLAG_SKIP_ALIGN     (1u << 9)
#define EM_FLAG_SKIP_GEMM1     (1u << 10)
#define EM_FLAG_SKIP_GEMM2     (1u << 11)
#define EM_FLAG_SKIP_COMBINE   (1u << 12)
/* Kernel choice: the shape-generic GEMM kernels at every batch size (the cross-check of the tuned ones). */
#define EM_FLAG_FORCE_GENERIC  (1u << 16)
/* The 256-row kernels run one workgroup per tile instead of one per CU walking a tile queue. */
#define EM_FLAG_NO_PERSIST     (1u << 17)
/* The sort of the layer call runs on one workgroup at every batch size. */
#define EM_FLAG_ONE_GROUP_SORT (1u << 18)

#endif /* ELECTROCK_MOE_DIAG_H */
