// fp32 path (placeholder until the fp32 kernels land): reports "not supported".
#include "sba_device.hpp"
#include "sba_params.hpp"
namespace sba {
hipError_t launch_fwd_f32(const FwdParams&, int, hipStream_t) { return hipErrorNotSupported; }
hipError_t launch_bwd_f32(const BwdParams&, int, int, hipStream_t) { return hipErrorNotSupported; }
}  // namespace sba
