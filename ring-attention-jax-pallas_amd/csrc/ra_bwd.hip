#include "ra_launch.h"
namespace ra {
hipError_t launch_bwd_delta(const void*, int, long long, long long, long long, TensorArg, float*, int, int, int, int, hipStream_t) { return hipErrorNotSupported; }
hipError_t launch_bwd_step(const BwdArgs&, int, bool, hipStream_t) { return hipErrorNotSupported; }
hipError_t launch_bwd_finalize(const float*, void*, long long, long long, long long, int, int, int, int, hipStream_t) { return hipErrorNotSupported; }
}
