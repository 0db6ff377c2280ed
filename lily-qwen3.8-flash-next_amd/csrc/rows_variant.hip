// rows_variant.hip - one (logits type, kernel kind) pair of the row kernel, with and without
// the row sum.  Compiled once per pair (-DLILY_DT=0|1 -DLILY_KIND=0|1|2) so that the pairs
// build in parallel; rows_dispatch.hip picks among them.
#include "row_kernel.h"

#if !defined(LILY_DT) || !defined(LILY_KIND)
#error "compile with -DLILY_DT=<lily_dtype> -DLILY_KIND=<0|1|2>"
#endif

#define LILY_CAT_(a, b, c, d) a##b##c##d
#define LILY_CAT(a, b, c, d) LILY_CAT_(a, b, c, d)

namespace lily {

hipError_t LILY_CAT(launch_rows_dt, LILY_DT, _kind, LILY_KIND)(hipStream_t stream, bool lse, uint32_t rows,
                                                              const LaunchCfg& cfg,
                                                              const InlineRows* inline_rows,
                                                              size_t dyn_bytes) {
    return lse ? launch_variant<LILY_DT, LILY_KIND, true>(stream, rows, cfg, inline_rows, dyn_bytes)
               : launch_variant<LILY_DT, LILY_KIND, false>(stream, rows, cfg, inline_rows, dyn_bytes);
}

}  // namespace lily
