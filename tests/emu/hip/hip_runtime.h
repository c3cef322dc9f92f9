// Test infrastructure: stands in for <hip/hip_runtime.h> when the kernels are compiled for the host
// (see ../hip_emu.h).
#include "../hip_emu.h"
