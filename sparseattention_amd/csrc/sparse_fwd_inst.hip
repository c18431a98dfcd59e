// One translation unit per (element type, mask source) of the block-sparse forward, so that the variants
// compile in parallel: built four times with -DSA_FWD_DT={0,1} (bf16, fp16) and -DSA_FWD_PK={0,1}
// (bool mask, bit-packed PARTIAL tiles).
#include "sparse_fwd_kernel.h"

#if !defined(SA_FWD_DT) || !defined(SA_FWD_PK)
#error "compile with -DSA_FWD_DT=<0|1> -DSA_FWD_PK=<0|1>"
#endif

namespace sa {
template hipError_t launch_fwd_variant<SA_FWD_DT, (SA_FWD_PK != 0)>(const FwdParams &, int, int, hipStream_t);
}  // namespace sa
