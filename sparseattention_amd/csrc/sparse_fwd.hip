// Dispatch of the block-sparse forward to the translation unit that holds the kernels for the element type,
// for the source of the PARTIAL tiles' mask entries and for the way Q tiles are handed out (sparse_fwd_inst.hip).
#include "kernels.h"

namespace sa {

template <int DT, bool PK, bool PS>
hipError_t launch_fwd_variant(const FwdParams &p, int D, int BQ, hipStream_t stream);
#define SA_DECL(DT, PK, PS) \
    extern template hipError_t launch_fwd_variant<DT, PK, PS>(const FwdParams &, int, int, hipStream_t);
SA_DECL(0, false, false) SA_DECL(0, false, true) SA_DECL(0, true, false) SA_DECL(0, true, true)
SA_DECL(1, false, false) SA_DECL(1, false, true) SA_DECL(1, true, false) SA_DECL(1, true, true)
#undef SA_DECL

namespace {
template <int DT>
hipError_t by_flags(const FwdParams &p, int D, int BQ, hipStream_t stream) {
    const bool pk = p.packed != nullptr, ps = p.sched != nullptr;
    if (pk) return ps ? launch_fwd_variant<DT, true, true>(p, D, BQ, stream) : launch_fwd_variant<DT, true, false>(p, D, BQ, stream);
    return ps ? launch_fwd_variant<DT, false, true>(p, D, BQ, stream) : launch_fwd_variant<DT, false, false>(p, D, BQ, stream);
}
}  // namespace

hipError_t launch_fwd(const FwdParams &p, int dtype, int D, int BQ, hipStream_t stream) {
    if (dtype == 0) return by_flags<0>(p, D, BQ, stream);
    if (dtype == 1) return by_flags<1>(p, D, BQ, stream);
    return hipErrorInvalidValue;
}

}  // namespace sa
