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

// Voxel range [lo, lo + n) along one axis whose centres lie within `reach` of `coord` (n <= 0:
// none).  Tighter than the reference's index box (src/grid_maker.cu:66-79), which adds a voxel
// beyond the reach on either side; such voxels contribute nothing to a gradient.  The slack keeps
// a voxel whose distance equals the reach to rounding.
__device__ __forceinline__ void reach_range(float origin, float coord, float reach, float inv_res,
                                            int dim, int& lo, int& n) {
  constexpr float kSlack = 1e-3f;
  // (clamped on both sides as floats: a coordinate or a reach that is huge, infinite or not a
  // number must not reach the conversion)
  const float first = fminf(fmaxf(ceilf((coord - reach - origin) * inv_res - kSlack), 0.f), (float)dim);
  const float last = fmaxf(fminf(floorf((coord + reach - origin) * inv_res + kSlack), (float)(dim - 1)), -1.f);
  lo = (int)first;
  n = (int)last - lo + 1;
}

// Sweep of the voxels within `reach` of an atom by one wave: like sweep_box, but over the range
// of reach_range instead of the reference's index box, and only over the (y, z) columns that come
// within reach of the atom -- a circle's worth instead of the square's.  The columns are tested
// 64 at a time and compacted into `cols`, a list of 2 * kWave ints in LDS that belongs to the
// calling wave alone; every full 64 (and the rest at the end) is marched along x, one column per
// lane.  The set of voxels visited is a superset (by a relative slack of 1e-5 on reach^2 and
// 1e-3 voxel on the range) of those with dist <= reach, so a body that adds nothing beyond the
// reach gives the sums of sweep_box over the index box, in another order.
// body(dx, dy, dz, dist2, plane_off, lane_off, live) as for sweep_box.
template <typename Body>
__device__ __forceinline__ void sweep_reach(const GridArg& g, int lane, volatile int* cols,
                                            float ox, float oy, float oz, float ax, float ay,
                                            float az, float reach, Body body) {
  const int dim = g.dim;
  const float inv_res = 1.0f / g.resolution;
  int lo0, lo1, lo2, ni, nj, nk;
  reach_range(ox, ax, reach, inv_res, dim, lo0, ni);
  reach_range(oy, ay, reach, inv_res, dim, lo1, nj);
  reach_range(oz, az, reach, inv_res, dim, lo2, nk);
  if (ni <= 0 || nj <= 0 || nk <= 0) return;
  const float reach2 = reach * reach * 1.00001f;
  const int ncols = nj * nk;
  const float inv_nk = __builtin_amdgcn_rcpf((float)nk);
  for (int i0 = 0; i0 < ni; i0 += kWave) {
    const int planes = min(kWave, ni - i0);
    const int dx_lane = __float_as_int(grid_coord(ox, lo0 + i0 + lane, g.resolution) - ax);
    // one pass: lanes below `count` take the columns cols[0 .. count)
    auto march = [&](int count) {
      wave_lds_fence();                          // the list is complete
      const bool live = lane < count;
      const int packed = cols[live ? lane : 0];
      const int j = packed >> 16, k = packed & 0xffff;
      const float dy = grid_coord(oy, lo1 + j, g.resolution) - ay;
      const float dz = grid_coord(oz, lo2 + k, g.resolution) - az;
      const float dyz2 = live ? dy * dy + dz * dz : INFINITY;
      const unsigned lane_off = (unsigned)((lo1 + j) * dim + lo2 + k);
      // (unrolled so that the loads of a few planes are in flight together)
#pragma unroll 4
      for (int i = 0; i < planes; ++i) {
        const float dx = __int_as_float(__builtin_amdgcn_readlane(dx_lane, i));
        const unsigned plane_off = (unsigned)(lo0 + i0 + i) * (unsigned)(dim * dim);
        body(dx, dy, dz, fmaf(dx, dx, dyz2), plane_off, lane_off, live);
      }
    };
    int pending = 0;
    for (int c0 = 0; c0 < ncols; c0 += kWave) {
      wave_lds_fence();                          // the entries moved to the front have been read
      const int cand = c0 + lane;
      const int j = (int)(((float)cand + 0.5f) * inv_nk), k = cand - j * nk;
      const float dy = grid_coord(oy, lo1 + j, g.resolution) - ay;
      const float dz = grid_coord(oz, lo2 + k, g.resolution) - az;
      const bool within = cand < ncols && dy * dy + dz * dz <= reach2;
      const unsigned long long m = __ballot(within);
      if (within) cols[pending + __popcll(m & ((1ull << lane) - 1ull))] = (j << 16) | k;
      pending += __popcll(m);
      if (pending >= kWave) {
        march(kWave);
        pending -= kWave;
        const int moved = cols[kWave + lane];
        if (lane < pending) cols[lane] = moved;
      }
    }
    if (pending > 0) march(pending);
  }
}

// Whether the sweeps must follow the reference's index box (src/grid_maker.cu:66-79) instead of the
// reach: the box is what decides which voxels count where it is NOT wider than the support of the
// density or where the density does not fade to zero at its edge.  That is a binary sphere with a
// final radius multiple of at most one (the box is smaller than the sphere, or coincides with it,
// and then the rounding of its edges decides about the voxels on them), and a Gaussian cut off
// without a tail (final multiple = Gaussian multiple): the box [floor(lo), ceil(hi)) leaves out a
// voxel that sits exactly at +reach on an axis, where such a density and its gradient are not zero.
__device__ __forceinline__ bool needs_index_box(const GridArg& g, bool binary) {
  return (binary && g.frm <= 1.0f) || g.frm <= g.grm;
}

// sweep_reach, or -- `index_box` -- the reference's index box for the radius `reach` (sweep_box).
template <typename Body>
__device__ __forceinline__ void sweep_reach(const GridArg& g, int lane, volatile int* cols,
                                            float ox, float oy, float oz, float ax, float ay,
                                            float az, float reach, bool index_box, Body body) {
  if (index_box) {
    int lo0, hi0, lo1, hi1, lo2, hi2;
    bounds_1d(ox, ax, reach, g.resolution, g.dim, lo0, hi0);
    bounds_1d(oy, ay, reach, g.resolution, g.dim, lo1, hi1);
    bounds_1d(oz, az, reach, g.resolution, g.dim, lo2, hi2);
    if (hi0 > lo0 && hi1 > lo1 && hi2 > lo2)
      sweep_box(g, lane, ox, oy, oz, ax, ay, az, lo0, lo1, lo2, hi0 - lo0, hi1 - lo1, hi2 - lo2, body);
    return;
  }
  sweep_reach(g, lane, cols, ox, oy, oz, ax, ay, az, reach, body);
}

}  // namespace mg

#endif
