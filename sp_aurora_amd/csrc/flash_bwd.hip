#include "spa_common.h"
hipError_t spa_launch_flash_bwd(BwdParams p, int D, int dtype, hipStream_t stream) { return hipErrorInvalidValue; }
