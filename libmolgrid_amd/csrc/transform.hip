// Rigid transform of packed atom coordinates, one launch for a whole batch.
//
// Forward:  out = rotate_q(in - center) + center + translation
//           (include/libmolgrid/quaternion.h:152-158, src/transform.cpp:57-79)
// Backward: out = rotate_{q^-1}(in + (-translation - center)) + center
//           (src/transform.cpp:85-108)
// Every product and sum is a separate float rounding in the reference's order,
// so the result is the same float the host loop produces.
#include "device_common.h"
#include "kernels.h"

namespace mg {

namespace {

constexpr int kThreads = 256;

template <bool INVERSE>
__global__ __launch_bounds__(kThreads) void transform_kernel(
    BatchArg batch, Vec4Arg quats, Vec3Arg centers, Vec3Arg translations, int dotranslate,
    const float* in, float* out) {
  const int b = blockIdx.y;
  int begin, end;
  example_range(batch, b, begin, end);
  const float4 q = load4(quats, b);
  const float3 c = load3(centers, b);
  float3 t = make_float3(0.f, 0.f, 0.f);
  if (dotranslate) t = load3(translations, b);
  const float4 qinv = quat_inverse(q);

  if (!INVERSE) {
    for (int a = begin + blockIdx.x * kThreads + threadIdx.x; a < end; a += gridDim.x * kThreads) {
#pragma clang fp contract(off)
      const float x = in[3 * a], y = in[3 * a + 1], z = in[3 * a + 2];
      const float3 r = quat_rotate(q, qinv, x - c.x, y - c.y, z - c.z);
      out[3 * a] = r.x + c.x + t.x;
      out[3 * a + 1] = r.y + c.y + t.y;
      out[3 * a + 2] = r.z + c.z + t.z;
    }
  } else {
    // rotating by the inverse quaternion: its own inverse is conj(qinv)/norm(qinv)
    const float4 qinvinv = quat_inverse(qinv);
    float3 un;
    {
#pragma clang fp contract(off)
      un = make_float3(-t.x - c.x, -t.y - c.y, -t.z - c.z);
    }
    for (int a = begin + blockIdx.x * kThreads + threadIdx.x; a < end; a += gridDim.x * kThreads) {
#pragma clang fp contract(off)
      const float x = in[3 * a] + un.x, y = in[3 * a + 1] + un.y, z = in[3 * a + 2] + un.z;
      const float3 r = quat_rotate(qinv, qinvinv, x, y, z);
      out[3 * a] = r.x + c.x;
      out[3 * a + 1] = r.y + c.y;
      out[3 * a + 2] = r.z + c.z;
    }
  }
}

}  // namespace

hipError_t launch_transform(const BatchArg& batch, int nbatch, int launch_atoms,
                            const Vec4Arg& quats, const Vec3Arg& centers,
                            const Vec3Arg& translations, bool dotranslate, bool inverse,
                            const float* in, float* out, hipStream_t stream) {
  int blocks = (launch_atoms + kThreads - 1) / kThreads;
  if (blocks < 1) blocks = 1;
  if (blocks > 1024) blocks = 1024;
  dim3 grid(blocks, nbatch), block(kThreads);
  if (inverse)
    hipLaunchKernelGGL(transform_kernel<true>, grid, block, 0, stream, batch, quats, centers,
                       translations, (int)dotranslate, in, out);
  else
    hipLaunchKernelGGL(transform_kernel<false>, grid, block, 0, stream, batch, quats, centers,
                       translations, (int)dotranslate, in, out);
  return hipGetLastError();
}

}  // namespace mg
