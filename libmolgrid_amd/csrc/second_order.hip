// Atom relevance and the gradients of the backward pass on gfx950.
//
// Both are atom-centred like the backward pass itself: one wavefront per atom sweeps the atom's
// voxel box (sweep.h), lanes keep private partial sums and a DPP tree combines them.
//
//   relevance           src/grid_maker.cpp:392-432, 680-704: every voxel the atom reaches hands
//                       the atom the share (own density / total density) of its relevance.
//   backward_gradients  src/grid_maker.cpp:529-661: the backward pass maps (coords, types, diff)
//                       to (atom_gradients, type_gradients); given upstream gradients of those two,
//                       this is the gradient with respect to diff (diffdiff, scattered with float
//                       atomics like the reference's GPU kernel, src/grid_maker.cu:652-753), to
//                       the coordinates (atom_diffdiff) and to the types (type_diffdiff = 0).
#include "kernels.h"
#include "splat_common.h"
#include "sweep.h"

namespace mg {

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / kWave;

int atom_blocks(int launch_atoms) {
  int blocks = (launch_atoms + kWaves - 1) / kWaves;
  if (blocks < 1) blocks = 1;
  if (blocks > 4096) blocks = 4096;
  return blocks;
}

// calc_point (src/grid_maker.cu:95-130) float for float: the relevance divides the atom's density
// by the grid's, and where the atom is the voxel's only contributor the quotient has to come out
// as exactly 1 however small both are -- so no contraction, the exponent through double as in the
// reference, and the same clamp.
template <bool BINARY>
__device__ __forceinline__ float calc_point_reference(const GridArg& g, float dx, float dy,
                                                      float dz, float ar) {
#pragma clang fp contract(off)
  const float rsq = sq_distance_exact(dx, dy, dz);
  if (BINARY) return rsq < ar * ar ? 1.0f : 0.0f;
  const float dist = sqrtf(rsq);
  if (dist > ar * g.frm) return 0.0f;
  if (dist <= ar * g.grm) {
    const float ex = (float)(-2.0 * dist * dist / (ar * ar));
    return expf(ex);
  }
  const float dr = dist / ar;
  const float q = (g.A * dr + g.B) * dr + g.C;
  return q > 0.f ? q : 0.f;
}

template <bool BINARY>
__global__ __launch_bounds__(kThreads) void relevance_kernel(
    GridArg g, BatchArg batch, Vec3Arg centers, const float* __restrict__ coords,
    const float* __restrict__ type_index, const float* __restrict__ radii,
    const float* __restrict__ density_grid, const float* __restrict__ diff,
    float* __restrict__ relevance) {
  __shared__ int s_cols[kWaves][2 * kWave];      // column list of each wave (sweep_reach)
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int b = blockIdx.y;
  int begin, end;
  example_range(batch, b, begin, end);
  const float3 center = load3(centers, b);
  const float ox = center.x - g.half_dimension;
  const float oy = center.y - g.half_dimension;
  const float oz = center.z - g.half_dimension;
  const int dim = g.dim;
  const size_t chan_stride = (size_t)dim * dim * dim;
  const size_t example = (size_t)b * g.ntypes * chan_stride;

  for (int a = begin + blockIdx.x * kWaves + wave; a < end; a += gridDim.x * kWaves) {
    float ret = 0.f;
    const float tf = roundf(type_index[a]);
    if (tf >= 0.f && tf < (float)g.ntypes) {
      const float ax = coords[3 * a], ay = coords[3 * a + 1], az = coords[3 * a + 2];
      const float radius = radii[a];
      float densityrad, ar;
      {
#pragma clang fp contract(off)
        densityrad = radius * g.radius_scale * g.frm;
        ar = radius * g.radius_scale;
      }
      // the voxels with a density above zero lie within the final radius (binary: the radius)
      if (densityrad > 0.f) {
        const float* dens = density_grid + example + (size_t)(int)tf * chan_stride;
        const float* dif = diff + example + (size_t)(int)tf * chan_stride;
        // (over the reference's index box, always: the box leaves out a voxel that sits exactly
        // at +reach on an axis, and although the atom's density is next to nothing there, so may
        // be the grid's that it is divided by)
        sweep_reach(g, lane, s_cols[wave], ox, oy, oz, ax, ay, az, densityrad, true,
                    [&](float dx, float dy, float dz, float, unsigned plane_off, unsigned lane_off,
                        bool live) {
                      const float val = calc_point_reference<BINARY>(g, dx, dy, dz, ar);
                      const float denseval = (dens + plane_off)[lane_off];
                      const float gridval = (dif + plane_off)[lane_off];
                      if (live && val > 0.f && denseval > 0.f) ret += gridval * val / denseval;
                    });
      }
    }
    ret = wave_sum(ret);
    if (lane == 0) relevance[a] = ret;
  }
}

__global__ __launch_bounds__(kThreads) void fill_zero_kernel(float* __restrict__ p, size_t n) {
  const size_t stride = (size_t)gridDim.x * kThreads;
  for (size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += stride) p[i] = 0.f;
}

// RTI: radii indexed by type (one row of ntypes radii per example) instead of by atom
template <bool RTI>
__global__ __launch_bounds__(kThreads) void grad_grad_kernel(
    GridArg g, BatchArg batch, Vec3Arg centers, const float* __restrict__ coords,
    const float* __restrict__ type_vector, const float* __restrict__ radii,
    const float* __restrict__ diff, const float* __restrict__ atom_gradients,
    const float* __restrict__ type_gradients, float* __restrict__ diffdiff,
    float* __restrict__ atom_diffdiff, float* __restrict__ type_diffdiff) {
  __shared__ int s_cols[kWaves][2 * kWave];      // column list of each wave (sweep_reach)
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int b = blockIdx.y;
  int begin, end;
  example_range(batch, b, begin, end);
  const float3 center = load3(centers, b);
  const float ox = center.x - g.half_dimension;
  const float oy = center.y - g.half_dimension;
  const float oz = center.z - g.half_dimension;
  const int dim = g.dim;
  const int T = g.ntypes;
  const size_t chan_stride = (size_t)dim * dim * dim;
  const size_t example = (size_t)b * T * chan_stride;
  const float* radii_b = RTI ? radii + (size_t)b * T : radii;

  for (int a = begin + blockIdx.x * kWaves + wave; a < end; a += gridDim.x * kWaves) {
    const float ax = coords[3 * a], ay = coords[3 * a + 1], az = coords[3 * a + 2];
    const float gx = atom_gradients[3 * a], gy = atom_gradients[3 * a + 1],
                gz = atom_gradients[3 * a + 2];
    float ddx = 0.f, ddy = 0.f, ddz = 0.f;
    // the density is linear in the type weights: no second-order term (src/grid_maker.cpp:563)
    for (int t = lane; t < T; t += kWave) type_diffdiff[(size_t)a * T + t] = 0.f;
    for (int t = 0; t < T; ++t) {
      const float tmult = type_vector[(size_t)a * T + t];
      if (tmult == 0.f) continue;   // wave-uniform
      const float tgrad = type_gradients[(size_t)a * T + t];
      const float radius = RTI ? radii_b[t] : radii_b[a];
      float densityrad, ar;
      {
#pragma clang fp contract(off)
        densityrad = radius * g.radius_scale * g.frm;
        ar = radius * g.radius_scale;
      }
      if (!(densityrad > 0.f)) continue;
      const float inv_ar = 1.0f / ar, inv_ar2 = inv_ar * inv_ar;
      const float rcut = ar * g.frm, rcore = ar * g.grm;
      const float* dif = diff + example + (size_t)t * chan_stride;
      float* dd = diffdiff + example + (size_t)t * chan_stride;
      // (over the reference's index box: the second derivatives do not vanish at the cut-off, and
      // the box leaves out a voxel that sits exactly at +reach on an axis)
      sweep_reach(g, lane, s_cols[wave], ox, oy, oz, ax, ay, az, densityrad, true,
                [&](float dx, float dy, float dz, float dist2, unsigned plane_off,
                    unsigned lane_off, bool live) {
                  // (the reference's own distance, src/grid_maker.cu:898-919: sqrtf of the
                  // uncontracted sum of squares; the terms jump at both radii, so a voxel within
                  // rounding of one must fall on the reference's side)
                  const float rsq = sq_distance_exact(dx, dy, dz);
                  const float dist = sqrtf(rsq);
                  if (!live || dist > rcut) return;   // density_grad_dist is NaN out here
                  const float G = (dif + plane_off)[lane_off];
                  // slope of the density along dist, the density, and with p = voxel - atom:
                  //   d2(density)/da_i da_j = K p_i p_j + [i == j] T3
                  float slope, val, K, T3;
                  if (dist <= rcore) {
                    const float e = __expf(-2.0f * dist2 * inv_ar2);
                    val = e;
                    slope = -4.0f * dist * inv_ar2 * e;
                    K = 16.0f * e * inv_ar2 * inv_ar2;
                    T3 = -4.0f * e * inv_ar2;
                  } else {
                    const float q = dist * inv_ar;
                    val = fmaxf((g.A * q + g.B) * q + g.C, 0.f);
                    const float c1 = g.E + g.D * q;
                    slope = c1 * inv_ar;
                    const float inv_dist = 1.0f / dist;
                    K = g.D * inv_dist * inv_dist * inv_ar2 - c1 * inv_dist * inv_dist * inv_dist * inv_ar;
                    T3 = c1 * inv_dist * inv_ar;
                  }
                  const float dot = dx * gx + dy * gy + dz * gz;
                  // gradient with respect to diff at this voxel
                  float gval = val * tgrad;
                  if (dist > 0.f) gval -= tmult * slope * dot / dist;
                  atomicAdd(dd + plane_off + lane_off, gval);
                  // gradient with respect to the atom's coordinates
                  const float wk = G * K * (tmult * dot);
                  const float w3 = G * T3 * tmult;
                  const float wt = G * tgrad;
                  ddx += wk * dx + w3 * gx + wt * (K * dx * dx + T3);
                  ddy += wk * dy + w3 * gy + wt * (K * dy * dy + T3);
                  ddz += wk * dz + w3 * gz + wt * (K * dz * dz + T3);
                });
    }
    ddx = wave_sum(ddx);
    ddy = wave_sum(ddy);
    ddz = wave_sum(ddz);
    if (lane == 0) {
      atom_diffdiff[3 * a] = ddx;
      atom_diffdiff[3 * a + 1] = ddy;
      atom_diffdiff[3 * a + 2] = ddz;
    }
  }
}

}  // namespace

hipError_t launch_backward_relevance(const GridArg& g, const BatchArg& batch, int nbatch,
                                     int launch_atoms, const Vec3Arg& centers, const float* coords,
                                     const float* type_index, const float* radii,
                                     const float* density, const float* diff, float* relevance,
                                     bool binary, hipStream_t stream) {
  dim3 grid(atom_blocks(launch_atoms), nbatch), block(kThreads);
  if (binary)
    hipLaunchKernelGGL(relevance_kernel<true>, grid, block, 0, stream, g, batch, centers, coords,
                       type_index, radii, density, diff, relevance);
  else
    hipLaunchKernelGGL(relevance_kernel<false>, grid, block, 0, stream, g, batch, centers, coords,
                       type_index, radii, density, diff, relevance);
  return hipGetLastError();
}

hipError_t launch_backward_gradients(const GridArg& g, const BatchArg& batch, int nbatch,
                                     int launch_atoms, const Vec3Arg& centers,
                                     const float* coords, const float* type_vector,
                                     const float* radii, const float* diff,
                                     const float* atom_gradients, const float* type_gradients,
                                     float* diffdiff, float* atom_diffdiff, float* type_diffdiff,
                                     bool radii_type_indexed, hipStream_t stream) {
  // the scattered sums start from zero (a fill kernel rather than a memset node, so that the
  // call can be captured in a graph)
  const size_t grid_elems = (size_t)nbatch * g.ntypes * g.dim * g.dim * g.dim;
  hipLaunchKernelGGL(fill_zero_kernel, dim3(2048), dim3(kThreads), 0, stream, diffdiff, grid_elems);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  dim3 grid(atom_blocks(launch_atoms), nbatch), block(kThreads);
  if (radii_type_indexed)
    hipLaunchKernelGGL(grad_grad_kernel<true>, grid, block, 0, stream, g, batch, centers, coords,
                       type_vector, radii, diff, atom_gradients, type_gradients, diffdiff,
                       atom_diffdiff, type_diffdiff);
  else
    hipLaunchKernelGGL(grad_grad_kernel<false>, grid, block, 0, stream, g, batch, centers, coords,
                       type_vector, radii, diff, atom_gradients, type_gradients, diffdiff,
                       atom_diffdiff, type_diffdiff);
  return hipGetLastError();
}

}  // namespace mg
