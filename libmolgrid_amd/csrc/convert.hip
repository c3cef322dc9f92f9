// float <-> double copies for callers that hold double precision grids.  The reference
// instantiates its GPU overloads for Grid<double, ...> outputs, gradients and coordinates as well
// (src/grid_maker.cu:293-294, 445-446, 460-466, 600; src/transform.cu:96) and computes in float
// there too; here such arrays are staged through float copies around the float kernels.
#include "kernels.h"

namespace mg {
namespace {

constexpr int kThreads = 256;

template <typename From, typename To>
__global__ __launch_bounds__(kThreads) void convert_kernel(const From* __restrict__ src,
                                                           To* __restrict__ dst, size_t n) {
  const size_t stride = (size_t)gridDim.x * kThreads;
  for (size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += stride)
    dst[i] = (To)src[i];
}

template <typename From, typename To>
hipError_t launch(const From* src, To* dst, size_t n, hipStream_t stream) {
  if (n == 0) return hipSuccess;
  size_t blocks = (n + kThreads - 1) / kThreads;
  if (blocks > 65536) blocks = 65536;
  hipLaunchKernelGGL((convert_kernel<From, To>), dim3((unsigned)blocks), dim3(kThreads), 0, stream,
                     src, dst, n);
  return hipGetLastError();
}

}  // namespace

hipError_t launch_widen(const float* src, double* dst, size_t n, hipStream_t stream) {
  return launch<float, double>(src, dst, n, stream);
}
hipError_t launch_narrow(const double* src, float* dst, size_t n, hipStream_t stream) {
  return launch<double, float>(src, dst, n, stream);
}

}  // namespace mg
