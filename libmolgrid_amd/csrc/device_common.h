// Shared device-side helpers for the gfx950 gridding kernels.
#ifndef LIBMOLGRID_AMD_DEVICE_COMMON_H_
#define LIBMOLGRID_AMD_DEVICE_COMMON_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "gfx950_asm.h"
#include "molgrid_hip.h"

namespace mg {

constexpr int kWave = 64;

// A per-example float3 / float4 parameter: either one device row per example
// or one host value used for every example.
struct Vec3Arg {
  const float* dev;
  float host[3];
};
struct Vec4Arg {
  const float* dev;
  float host[4];
};

__device__ __forceinline__ float3 load3(const Vec3Arg& a, int b) {
  if (a.dev) return make_float3(a.dev[3 * b], a.dev[3 * b + 1], a.dev[3 * b + 2]);
  return make_float3(a.host[0], a.host[1], a.host[2]);
}
__device__ __forceinline__ float4 load4(const Vec4Arg& a, int b) {
  if (a.dev) return make_float4(a.dev[4 * b], a.dev[4 * b + 1], a.dev[4 * b + 2], a.dev[4 * b + 3]);
  return make_float4(a.host[0], a.host[1], a.host[2], a.host[3]);
}

// Which atoms belong to example b.
struct BatchArg {
  const int32_t* offsets;  // device, nbatch+1 entries, or nullptr
  int32_t per_example;     // atoms per example when offsets == nullptr
};
__device__ __forceinline__ void example_range(const BatchArg& a, int b, int& begin, int& end) {
  if (a.offsets) {
    begin = a.offsets[b];
    end = a.offsets[b + 1];
  } else {
    begin = b * a.per_example;
    end = begin + a.per_example;
  }
}

// Which example the workgroups of launch slot `slot` (blockIdx.y) work on.  Workgroups start in
// launch order and the time of one grows with the atoms of its example, so a ragged batch is
// taken largest example first: the workgroups still running when the launch drains are then the
// cheapest ones.  Ties keep their order; batches with equal sizes, or with more examples than a
// wave has lanes, keep the launch order.  Every lane of the wave must call this.
__device__ __forceinline__ int example_for_slot(const BatchArg& a, int slot, int nbatch, int lane) {
  if (a.offsets == nullptr || nbatch < 2 || nbatch > kWave) return slot;
  const int me = lane < nbatch ? lane : nbatch - 1;
  const int mine = a.offsets[me + 1] - a.offsets[me];
  int before = 0;   // examples that come before this lane's in (size descending, index) order
  for (int i = 0; i < nbatch; ++i) {
    const int other = __builtin_amdgcn_readlane(mine, i);
    before += (other > mine || (other == mine && i < lane)) ? 1 : 0;
  }
  const unsigned long long hit = __ballot(lane < nbatch && before == slot);
  return hit ? (int)__builtin_ctzll(hit) : slot;
}

// Scalars every gridding kernel needs (a flattened mg_gridmaker plus derived
// values computed once on the host).
struct GridArg {
  float resolution;
  float half_dimension;  // (float)(dimension / 2.0)
  float radius_scale;
  float grm;  // gaussian_radius_multiple (positive)
  float frm;  // final_radius_multiple
  float A, B, C, D, E;
  int dim;
  int ntypes;
};

// Quaternion product in the reference's association order
// (include/libmolgrid/quaternion.h:82-91); no contraction so that the result is
// the same float the host computes.
__device__ __forceinline__ float4 quat_mul(float4 p, float4 q) {
#pragma clang fp contract(off)
  float a = p.x, b = p.y, c = p.z, d = p.w;
  float ar = q.x, br = q.y, cr = q.z, dr = q.w;
  float4 o;
  o.x = +a * ar - b * br - c * cr - d * dr;
  o.y = +a * br + b * ar + c * dr - d * cr;
  o.z = +a * cr - b * dr + c * ar + d * br;
  o.w = +a * dr + b * cr - c * br + d * ar;
  return o;
}

// conj(q)/norm(q), i.e. the inverse (quaternion.h:145-149, 161-165).
__device__ __forceinline__ float4 quat_inverse(float4 q) {
#pragma clang fp contract(off)
  float n = q.x * q.x + q.y * q.y + q.z * q.z + q.w * q.w;
  return make_float4(q.x / n, -q.y / n, -q.z / n, -q.w / n);
}

// q * (0,x,y,z) * inverse(q) with `qinv` precomputed by the caller.
__device__ __forceinline__ float3 quat_rotate(float4 q, float4 qinv, float x, float y, float z) {
  float4 r = quat_mul(quat_mul(q, make_float4(0.f, x, y, z)), qinv);
  return make_float3(r.y, r.z, r.w);
}

// Cartesian coordinate of grid index i along one axis: origin + i*resolution
// with two roundings (src/grid_maker.cpp:191-193).
__device__ __forceinline__ float grid_coord(float origin, int i, float resolution) {
#pragma clang fp contract(off)
  float s = (float)i * resolution;
  return origin + s;
}

// ((dx*dx + dy*dy) + dz*dz), uncontracted (src/grid_maker.cu:82-92).
__device__ __forceinline__ float sq_distance_exact(float dx, float dy, float dz) {
#pragma clang fp contract(off)
  float r = dx * dx;
  r = r + dy * dy;
  r = r + dz * dz;
  return r;
}

// Per-axis voxel range [lo, hi) an atom may touch (src/grid_maker.cu:66-79).
__device__ __forceinline__ void bounds_1d(float origin, float coord, float densityrad,
                                          float resolution, int dim, int& lo, int& hi) {
#pragma clang fp contract(off)
  lo = 0;
  hi = 0;
  float low = coord - densityrad - origin;
  if (low > 0) lo = (int)min((float)dim, floorf(low / resolution));
  float high = coord + densityrad - origin;
  if (high > 0) hi = (int)min((float)dim, ceilf(high / resolution));
}

}  // namespace mg

#endif
