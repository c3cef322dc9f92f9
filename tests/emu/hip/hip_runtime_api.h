// Test infrastructure: stands in for <hip/hip_runtime_api.h> when host code that uses the HIP runtime
// (the C++ classes of include/libmolgrid) is compiled against the emulation (see ../hip_emu.h).
#include "../hip_emu.h"
