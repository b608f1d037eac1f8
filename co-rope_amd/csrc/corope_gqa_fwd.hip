#include "common.hpp"
#include "kernels.hpp"
namespace corope {
hipError_t launch_corope_gqa_fwd(const CoropeParams&, int, hipStream_t) { return hipErrorNotSupported; }
}  // namespace corope
