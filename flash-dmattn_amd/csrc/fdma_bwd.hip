#include "fdma_common.h"
#include "fdma_params.h"
namespace fdma {
hipError_t launch_bwd(const BwdParams &, int, hipStream_t) { return hipErrorNotSupported; }
}
