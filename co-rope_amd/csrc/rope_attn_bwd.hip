#include "common.hpp"
#include "kernels.hpp"
namespace corope {
hipError_t launch_bwd_dkdv(const BwdParams&, int, bool, hipStream_t) { return hipErrorNotSupported; }
hipError_t launch_bwd_dq(const BwdParams&, int, bool, hipStream_t) { return hipErrorNotSupported; }
}  // namespace corope
