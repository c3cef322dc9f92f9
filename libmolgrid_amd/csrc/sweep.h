// Wave-level helpers of the atom-centred kernels (one wavefront per atom): a reduction over the
// 64 lanes and the sweep of an atom's voxel box.
#ifndef LIBMOLGRID_AMD_SWEEP_H_
#define LIBMOLGRID_AMD_SWEEP_H_

#include <hip/hip_runtime.h>

#include "device_common.h"

namespace mg {

// DPP controls (gfx9 encoding)
constexpr int kDppQuadPerm1032 = 0xB1;  // quad_perm:[1,0,3,2]
constexpr int kDppQuadPerm2301 = 0x4E;  // quad_perm:[2,3,0,1]
constexpr int kDppRowHalfMirror = 0x141;
constexpr int kDppRowMirror = 0x140;
constexpr int kDppRowBcast15 = 0x142;
constexpr int kDppRowBcast31 = 0x143;

template <int CTRL, int ROW_MASK>
__device__ __forceinline__ double dpp_add(double v) {
  // lanes outside ROW_MASK (or without a source lane) contribute 0
  const int lo = __builtin_amdgcn_update_dpp(0, __double2loint(v), CTRL, ROW_MASK, 0xF, false);
  const int hi = __builtin_amdgcn_update_dpp(0, __double2hiint(v), CTRL, ROW_MASK, 0xF, false);
  return v + __hiloint2double(hi, lo);
}

// Sum of v over the 64 lanes of the wave, returned to every lane.  The lanes' float partial sums
// are added in double: the cross-lane step adds no rounding of its own (the reference's
// sequential float loop, src/grid_maker.cu:898-919, carries more).
__device__ __forceinline__ double wave_sum64(float value) {
  double v = (double)value;
  v = dpp_add<kDppQuadPerm1032, 0xF>(v);
  v = dpp_add<kDppQuadPerm2301, 0xF>(v);
  v = dpp_add<kDppRowHalfMirror, 0xF>(v);
  v = dpp_add<kDppRowMirror, 0xF>(v);   // every lane of a 16-lane row holds the row total
  v = dpp_add<kDppRowBcast15, 0xA>(v);  // rows 1 and 3 add the total of rows 0 and 2
  v = dpp_add<kDppRowBcast31, 0xC>(v);  // rows 2 and 3 add the total of rows 0..1
  return __hiloint2double(__builtin_amdgcn_readlane(__double2hiint(v), 63),
                          __builtin_amdgcn_readlane(__double2loint(v), 63));
}
__device__ __forceinline__ float wave_sum(float v) { return (float)wave_sum64(v); }

// Sweep of an atom's voxel box [lo, lo+n) by one wave.  Each lane owns one (y, z) column of the
// box (64 columns per pass) and marches along x, so everything that depends on y and z only --
// dy, dz, dy^2+dz^2, the lane's element offset -- is worked out once per pass, while the x offset
// of a plane is the same in every lane: it is computed by lane i for plane i before the march
// and read back as a scalar.  body(dx, dy, dz, dist2, plane_off, lane_off, live) is called for
// every voxel; dx and plane_off (element offset of the plane) are wave-uniform, lane_off is the
// lane's element offset inside the plane, and lanes past the last column get live = false and an
// infinite dist2 (their offsets point at a valid voxel of the box).
template <typename Body>
__device__ __forceinline__ void sweep_box(const GridArg& g, int lane, float ox, float oy, float oz,
                                          float ax, float ay, float az, int lo0, int lo1, int lo2,
                                          int ni, int nj, int nk, Body body) {
  const int dim = g.dim;
  const int columns = nj * nk;
  for (int i0 = 0; i0 < ni; i0 += kWave) {
    const int planes = min(kWave, ni - i0);
    const int dx_lane = __float_as_int(grid_coord(ox, lo0 + i0 + lane, g.resolution) - ax);
    for (int c0 = 0; c0 < columns; c0 += kWave) {
      const bool live = c0 + lane < columns;
      const int c = live ? c0 + lane : columns - 1;
      const int j = c / nk, k = c - j * nk;
      const float dy = grid_coord(oy, lo1 + j, g.resolution) - ay;
      const float dz = grid_coord(oz, lo2 + k, g.resolution) - az;
      const float dyz2 = live ? dy * dy + dz * dz : INFINITY;
      const unsigned lane_off = (unsigned)((lo1 + j) * dim + lo2 + k);
      for (int i = 0; i < planes; ++i) {
        const float dx = __int_as_float(__builtin_amdgcn_readlane(dx_lane, i));
        const unsigned plane_off = (unsigned)(lo0 + i0 + i) * (unsigned)(dim * dim);
        body(dx, dy, dz, fmaf(dx, dx, dyz2), plane_off, lane_off, live);
      }
    }
  }
}

// sweep_box for callers that read one float per voxel from `chan` (one grid channel): the reads
// of kSweepChunk planes are issued together before any of them is used, so that a wave has
// several planes in flight instead of one round trip to memory per voxel.
constexpr int kSweepChunk = 8;
template <typename Body>
__device__ __forceinline__ void sweep_channel(const GridArg& g, const float* __restrict__ chan,
                                              int lane, float ox, float oy, float oz, float ax,
                                              float ay, float az, int lo0, int lo1, int lo2, int ni,
                                              int nj, int nk, Body body) {
  const int dim = g.dim;
  const int columns = nj * nk;
  const unsigned plane_stride = (unsigned)(dim * dim);
  for (int i0 = 0; i0 < ni; i0 += kWave) {
    const int planes = min(kWave, ni - i0);
    const int dx_lane = __float_as_int(grid_coord(ox, lo0 + i0 + lane, g.resolution) - ax);
    for (int c0 = 0; c0 < columns; c0 += kWave) {
      const bool live = c0 + lane < columns;
      const int c = live ? c0 + lane : columns - 1;
      const int j = c / nk, k = c - j * nk;
      const float dy = grid_coord(oy, lo1 + j, g.resolution) - ay;
      const float dz = grid_coord(oz, lo2 + k, g.resolution) - az;
      const float dyz2 = live ? dy * dy + dz * dz : INFINITY;
      const unsigned lane_off = (unsigned)((lo1 + j) * dim + lo2 + k);
      for (int i = 0; i < planes; i += kSweepChunk) {
        const float* first = chan + (size_t)(unsigned)(lo0 + i0 + i) * plane_stride;
        float gv[kSweepChunk];
#pragma unroll
        for (int u = 0; u < kSweepChunk; ++u)
          if (i + u < planes) gv[u] = (first + (size_t)u * plane_stride)[lane_off];
#pragma unroll
        for (int u = 0; u < kSweepChunk; ++u) {
          if (i + u < planes) {
            const float dx = __int_as_float(__builtin_amdgcn_readlane(dx_lane, i + u));
            body(dx, dy, dz, fmaf(dx, dx, dyz2), gv[u], live);
          }
        }
      }
    }
  }
}

}  // namespace mg

#endif
