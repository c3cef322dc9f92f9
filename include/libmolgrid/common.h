// Shared definitions of the C++ host layer: HIP error checking, float3 helpers.
//
// This layer keeps the class and member names of libmolgrid's public headers for the gridding
// path and forwards the numeric work to the C ABI in molgrid_hip.h.  `isCUDA = true` in a Grid
// type means "HIP device pointer".  Compile host code with -D__HIP_PLATFORM_AMD__ (hipcc does it
// itself) and link libmolgrid_hip.so and libamdhip64.so.
#ifndef LIBMOLGRID_COMMON_H_
#define LIBMOLGRID_COMMON_H_

#include <hip/hip_runtime_api.h>

#include <sstream>
#include <stdexcept>
#include <string>

#include "molgrid_hip.h"

namespace libmolgrid {

/// integer (or anything streamable) to string, used in error messages
template <typename T>
inline std::string itoa(const T& v) {
  std::ostringstream s;
  s << v;
  return s.str();
}

/// throw std::runtime_error for a failed HIP runtime call (reference: LMG_CUDA_CHECK,
/// include/libmolgrid/common.h:41-47)
inline void hip_check(hipError_t e, const char* file, int line) {
  if (e != hipSuccess)
    throw std::runtime_error(std::string("HIP Error: ") + hipGetErrorString(e) + " at " + file +
                             ":" + itoa(line));
}
#define LMG_HIP_CHECK(call) ::libmolgrid::hip_check((call), __FILE__, __LINE__)

/// map a return code of the C ABI to the exception type the reference throws
inline void abi_check(int rc, const char* what) {
  if (rc == MG_OK) return;
  const std::string msg = std::string(what) + ": " + mg_error_string(rc);
  if (rc == MG_ERR_OUT_OF_RANGE) throw std::out_of_range(msg);
  if (rc < 0) throw std::invalid_argument(msg);
  throw std::runtime_error("HIP Error: " + msg);
}

/// select the device used by the calling thread (reference: set_gpu_device / get_gpu_device)
inline void set_gpu_device(int device) { LMG_HIP_CHECK(hipSetDevice(device)); }
inline int get_gpu_device() {
  int d = 0;
  LMG_HIP_CHECK(hipGetDevice(&d));
  return d;
}

}  // namespace libmolgrid

#endif
