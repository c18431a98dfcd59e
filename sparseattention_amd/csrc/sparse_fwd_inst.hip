// One translation unit per (element type, mask source, tile hand-out) of the block-sparse forward, so that the
// variants compile in parallel: built with -DSA_FWD_DT={0,1} (bf16, fp16), -DSA_FWD_PK={0,1} (bool mask,
// bit-packed PARTIAL tiles) and -DSA_FWD_PS={0,1} (one workgroup per Q tile, persistent workgroups).
#include "sparse_fwd_kernel.h"

#if !defined(SA_FWD_DT) || !defined(SA_FWD_PK) || !defined(SA_FWD_PS)
#error "compile with -DSA_FWD_DT=<0|1> -DSA_FWD_PK=<0|1> -DSA_FWD_PS=<0|1>"
#endif

namespace sa {
template hipError_t launch_fwd_variant<SA_FWD_DT, (SA_FWD_PK != 0), (SA_FWD_PS != 0)>(const FwdParams &, int, int,
                                                                                      hipStream_t);
}  // namespace sa
