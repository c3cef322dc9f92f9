// Pieces shared by the index-typed and vector-typed forward splat kernels.
#ifndef LIBMOLGRID_AMD_SPLAT_COMMON_H_
#define LIBMOLGRID_AMD_SPLAT_COMMON_H_

#include "device_common.h"

namespace mg {

constexpr int kTile = 8;                          // voxels per tile side
constexpr int kTileVox = kTile * kTile * kTile;   // 512
constexpr int kSplatThreads = 512;                // one lane per voxel
constexpr int kSplatWaves = kSplatThreads / kWave;
constexpr int kCandCap = 1024;                    // atom indices kept per scan round
constexpr int kChunk = 256;                       // atoms turned into LDS records at a time
constexpr float kNeg2Log2e = -2.0f * 1.4426950408889634f;
constexpr float kCullSlack = 1.00001f;            // keeps every cull a superset of the exact test

typedef float v4f __attribute__((ext_vector_type(4)));

// LDS position of voxel (x,y,z) of the tile inside one channel plane.  Bit 2 of
// the in-plane index is flipped on odd x so that the 32 lanes of a half wave
// (two x planes of a 4x4x4 sub-tile) land in 32 different banks.
__device__ __forceinline__ int lds_voxel(int x, int y, int z) {
  return x * 64 + ((y * 8 + z) ^ ((x & 1) << 2));
}

// Squared distance from point p to the axis-aligned box [lo, hi]; a lower bound
// of the squared distance to every voxel centre inside the box because float
// subtraction, squaring and addition are monotone.
__device__ __forceinline__ float box_distance2(float px, float py, float pz, float lox, float loy,
                                               float loz, float hix, float hiy, float hiz) {
  const float dx = fmaxf(fmaxf(lox - px, px - hix), 0.f);
  const float dy = fmaxf(fmaxf(loy - py, py - hiy), 0.f);
  const float dz = fmaxf(fmaxf(loz - pz, pz - hiz), 0.f);
  return sq_distance_exact(dx, dy, dz);
}

// Per-thread geometry of the tile / sub-tile / voxel it works on.
struct SplatGeom {
  int x0, y0, z0;        // first voxel of the tile
  int vxi, vyi, vzi;     // this lane's voxel (grid index)
  int slot;              // its position in an LDS channel plane
  bool voxel_live, wave_live;
  float ox, oy, oz;      // grid origin
  float vx, vy, vz;      // voxel centre
  float tlo[3], thi[3];  // tile box
  float wlo[3], whi[3];  // this wave's 4x4x4 sub-tile box
};

__device__ __forceinline__ SplatGeom make_geom(const GridArg& g, float3 center, int tile,
                                               int tiles_per_side, int wave, int lane) {
  SplatGeom s;
  const int tz = tile % tiles_per_side;
  const int ty = (tile / tiles_per_side) % tiles_per_side;
  const int tx = tile / (tiles_per_side * tiles_per_side);
  const int dim = g.dim;
  s.ox = center.x - g.half_dimension;
  s.oy = center.y - g.half_dimension;
  s.oz = center.z - g.half_dimension;
  s.x0 = tx * kTile;
  s.y0 = ty * kTile;
  s.z0 = tz * kTile;
  s.tlo[0] = grid_coord(s.ox, s.x0, g.resolution);
  s.tlo[1] = grid_coord(s.oy, s.y0, g.resolution);
  s.tlo[2] = grid_coord(s.oz, s.z0, g.resolution);
  s.thi[0] = grid_coord(s.ox, min(s.x0 + kTile, dim) - 1, g.resolution);
  s.thi[1] = grid_coord(s.oy, min(s.y0 + kTile, dim) - 1, g.resolution);
  s.thi[2] = grid_coord(s.oz, min(s.z0 + kTile, dim) - 1, g.resolution);
  const int sx = (wave >> 2) * 4, sy = ((wave >> 1) & 1) * 4, sz = (wave & 1) * 4;
  const int lx = sx + (lane >> 4), ly = sy + ((lane >> 2) & 3), lz = sz + (lane & 3);
  s.vxi = s.x0 + lx;
  s.vyi = s.y0 + ly;
  s.vzi = s.z0 + lz;
  s.voxel_live = s.vxi < dim && s.vyi < dim && s.vzi < dim;
  s.vx = grid_coord(s.ox, s.vxi, g.resolution);
  s.vy = grid_coord(s.oy, s.vyi, g.resolution);
  s.vz = grid_coord(s.oz, s.vzi, g.resolution);
  s.slot = lds_voxel(lx, ly, lz);
  s.wlo[0] = grid_coord(s.ox, s.x0 + sx, g.resolution);
  s.wlo[1] = grid_coord(s.oy, s.y0 + sy, g.resolution);
  s.wlo[2] = grid_coord(s.oz, s.z0 + sz, g.resolution);
  s.whi[0] = grid_coord(s.ox, min(s.x0 + sx + 4, dim) - 1, g.resolution);
  s.whi[1] = grid_coord(s.oy, min(s.y0 + sy + 4, dim) - 1, g.resolution);
  s.whi[2] = grid_coord(s.oz, min(s.z0 + sz + 4, dim) - 1, g.resolution);
  s.wave_live = (s.x0 + sx) < dim && (s.y0 + sy) < dim && (s.z0 + sz) < dim;
  return s;
}

// Order-preserving append of the lanes with `pass` set to the workgroup's
// candidate list: wavefront ballot, per-wave totals through LDS, prefix count.
// Returns the number appended; contains two workgroup barriers.
__device__ __forceinline__ int append_candidates(bool pass, int value, int* s_cand, int ncand,
                                                 int* s_wcount, int wave, int lane) {
  const unsigned long long m = __ballot(pass);
  if (lane == 0) s_wcount[wave] = __popcll(m);
  __syncthreads();
  int before = 0, total = 0;
#pragma unroll
  for (int w = 0; w < kSplatWaves; ++w) {
    const int c = s_wcount[w];
    before += (w < wave) ? c : 0;
    total += c;
  }
  if (pass) s_cand[ncand + before + __popcll(m & ((1ull << lane) - 1ull))] = value;
  __syncthreads();
  return total;
}

// Index-box clip of the CPU loops (src/grid_maker.cpp:181-189), packed as
// lo | hi<<16 per axis.
__device__ __forceinline__ uint3 pack_clip(const GridArg& g, float ox, float oy, float oz, float ax,
                                           float ay, float az, float radius) {
  float densityrad;
  {
#pragma clang fp contract(off)
    densityrad = radius * g.radius_scale * g.frm;
  }
  int lo[3], hi[3];
  bounds_1d(ox, ax, densityrad, g.resolution, g.dim, lo[0], hi[0]);
  bounds_1d(oy, ay, densityrad, g.resolution, g.dim, lo[1], hi[1]);
  bounds_1d(oz, az, densityrad, g.resolution, g.dim, lo[2], hi[2]);
  return make_uint3((unsigned)lo[0] | ((unsigned)hi[0] << 16),
                    (unsigned)lo[1] | ((unsigned)hi[1] << 16),
                    (unsigned)lo[2] | ((unsigned)hi[2] << 16));
}
__device__ __forceinline__ uint3 pack_clip(const GridArg& g, const SplatGeom& s, float ax, float ay,
                                           float az, float radius) {
  return pack_clip(g, s.ox, s.oy, s.oz, ax, ay, az, radius);
}

__device__ __forceinline__ bool inside_clip(int xi, int yi, int zi, uint3 cl) {
  return xi >= (int)(cl.x & 0xffff) && xi < (int)(cl.x >> 16) &&
         yi >= (int)(cl.y & 0xffff) && yi < (int)(cl.y >> 16) &&
         zi >= (int)(cl.z & 0xffff) && zi < (int)(cl.z >> 16);
}
__device__ __forceinline__ bool inside_clip(const SplatGeom& s, uint3 cl) {
  return inside_clip(s.vxi, s.vyi, s.vzi, cl);
}

// Density of one atom at one voxel (calc_point, src/grid_maker.cu:95-130).
//   w  = ar^2 in binary mode, 1/ar^2 otherwise (ar = radius * radius_scale)
//   ar = only read in EXACT mode
// BINARY: 1 if ((dx^2+dy^2)+dz^2) < ar^2, on uncontracted floats -> bit exact.
// EXACT (density): the reference's own cut-off predicates on the same floats
//   (dist = sqrtf(rsq) > ar*frm -> 0; dist <= ar*grm -> Gaussian).
// otherwise: u = rsq/ar^2 and the cut-offs are tested on u; the density and its
//   slope are continuous at both cut-offs, so a voxel within rounding of one
//   changes by far less than the comparison tolerance.
template <bool BINARY, bool EXACT>
__device__ __forceinline__ float density(const GridArg& g, float dx, float dy, float dz, float w,
                                         float ar, float frm2, float grm2) {
  if (BINARY) {
    const float rsq = sq_distance_exact(dx, dy, dz);
    return rsq < w ? 1.0f : 0.0f;
  } else if (EXACT) {
    const float rsq = sq_distance_exact(dx, dy, dz);
    const float dist = sqrtf(rsq);
    float rcut, rgauss;
    {
#pragma clang fp contract(off)
      rcut = ar * g.frm;
      rgauss = ar * g.grm;
    }
    if (dist > rcut) return 0.f;
    if (dist <= rgauss) return __builtin_amdgcn_exp2f(rsq * w * kNeg2Log2e);
    const float dr = dist / ar;
    return fmaxf((g.A * dr + g.B) * dr + g.C, 0.f);
  } else {
    const float rsq = dx * dx + dy * dy + dz * dz;
    const float u = rsq * w;
    if (!(u <= frm2)) return 0.f;
    const float gauss = __builtin_amdgcn_exp2f(u * kNeg2Log2e);
    const float su = __builtin_amdgcn_sqrtf(u);
    const float quad = fmaxf(fmaf(g.A, u, fmaf(g.B, su, g.C)), 0.f);
    return (u <= grm2) ? gauss : quad;
  }
}

// The same density split into "does the atom reach the voxel" (returned) and the value where it
// does, so that callers can leave untouched sums alone.  `quad_c` is g.C (in a vector register).
template <bool BINARY, bool EXACT>
__device__ __forceinline__ bool density_hit(const GridArg& g, float dx, float dy, float dz, float w,
                                            float ar, float frm2, float grm2, float quad_c,
                                            float& val) {
  if (BINARY) {
    const float rsq = sq_distance_exact(dx, dy, dz);
    val = 1.0f;
    return rsq < w;
  } else if (EXACT) {
    val = density<false, true>(g, dx, dy, dz, w, ar, frm2, grm2);
    return val != 0.f;
  } else {
    const float rsq = dx * dx + dy * dy + dz * dz;
    const float u = rsq * w;
    const float gauss = __builtin_amdgcn_exp2f(u * kNeg2Log2e);
    const float su = __builtin_amdgcn_sqrtf(u);
    const float quad = fmaxf(fmaf(g.A, u, fmaf(g.B, su, quad_c)), 0.f);
    val = (u <= grm2) ? gauss : quad;
    return u <= frm2;
  }
}

}  // namespace mg

#endif
