#include "fa_common.hpp"
#include "fa_launch.hpp"
namespace acct {
hipError_t launch_bwd(const FaArgs& a, int dtype, int D, bool general, hipStream_t st) { return hipErrorNotSupported; }
}
