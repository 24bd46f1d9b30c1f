#include "fdma_common.h"
#include "fdma_params.h"
namespace fdma {
bool use_decode_path(int, int, int) { return false; }
int decode_num_splits(int, int, int) { return 1; }
hipError_t launch_fwd_decode(const FwdParams &, int, hipStream_t) { return hipErrorNotSupported; }
}
