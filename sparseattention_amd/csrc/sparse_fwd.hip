// Dispatch of the block-sparse forward to the translation unit that holds the kernels for the element type
// and for the source of the PARTIAL tiles' mask entries (see sparse_fwd_inst.hip).
#include "kernels.h"

namespace sa {

template <int DT, bool PK>
hipError_t launch_fwd_variant(const FwdParams &p, int D, int BQ, hipStream_t stream);
extern template hipError_t launch_fwd_variant<0, false>(const FwdParams &, int, int, hipStream_t);
extern template hipError_t launch_fwd_variant<0, true>(const FwdParams &, int, int, hipStream_t);
extern template hipError_t launch_fwd_variant<1, false>(const FwdParams &, int, int, hipStream_t);
extern template hipError_t launch_fwd_variant<1, true>(const FwdParams &, int, int, hipStream_t);

hipError_t launch_fwd(const FwdParams &p, int dtype, int D, int BQ, hipStream_t stream) {
    const bool pk = p.packed != nullptr;
    if (dtype == 0) return pk ? launch_fwd_variant<0, true>(p, D, BQ, stream) : launch_fwd_variant<0, false>(p, D, BQ, stream);
    if (dtype == 1) return pk ? launch_fwd_variant<1, true>(p, D, BQ, stream) : launch_fwd_variant<1, false>(p, D, BQ, stream);
    return hipErrorInvalidValue;
}

}  // namespace sa
