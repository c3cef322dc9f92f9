// Atom-gradient (and type-gradient) accumulation on gfx950.
//
// One wavefront owns one atom: its 64 lanes sweep the atom's voxel box
// (src/grid_maker.cu:66-79) -- every lane marches along x through one (y, z) column of the box --
// each lane keeps a private partial sum, and the partials are combined with a DPP reduction tree
// inside the wave.  No global float atomics are used, so the result is
// reproducible run to run.  Per-voxel terms follow accumulate_atom_gradient and
// density_grad_dist (src/grid_maker.cu:881-919); the CPU loops being mirrored
// are src/grid_maker.cpp:325-389 and 436-519.
#include "kernels.h"
#include "splat_common.h"
#include "sweep.h"

namespace mg {

namespace {

constexpr int kBwdThreads = 256;
constexpr int kBwdWaves = kBwdThreads / kWave;

// Per-atom constants of the gradient scale.
struct GradConsts {
  float inv_ar2;   // 1/ar^2
  float exp_k;     // -2 log2(e) / ar^2  (exp(-2u) = exp2(exp_k * dist^2))
  float gauss;     // 4/ar^2            (Gaussian part:  scale = gauss * exp(-2u) * gridval)
  float quad_a;    // -D/ar^2           (quadratic part: scale = (quad_a + quad_b/dist) * gridval)
  float quad_b;    // -E/ar
  float core2;     // (grm ar)^2: dist^2 up to here is Gaussian
  float reach2;    // (frm ar)^2: dist^2 beyond is untouched
};
__device__ __forceinline__ GradConsts grad_consts(const GridArg& g, float ar) {
  GradConsts c;
  const float inv_ar = 1.0f / ar;
  c.inv_ar2 = inv_ar * inv_ar;
  c.exp_k = c.inv_ar2 * kNeg2Log2e;
  c.gauss = 4.0f * c.inv_ar2;
  c.quad_a = -g.D * c.inv_ar2;
  c.quad_b = -g.E * inv_ar;
  c.core2 = g.grm * g.grm * ar * ar;
  c.reach2 = g.frm * g.frm * ar * ar;
  return c;
}

// Scale that turns (voxel - atom) into the gradient term of one voxel:
// -(1/dist) * d(density)/d(dist) * gridval (density_grad_dist and accumulate_atom_gradient,
// src/grid_maker.cu:881-919).  With u = dist^2/ar^2:
//   Gaussian, u <= grm^2:  d/d(dist) = -4 dist/ar^2 exp(-2u)   ->  4/ar^2 exp(-2u) gridval
//   quadratic tail:        d/d(dist) = (D dist/ar + E)/ar      -> -(D/ar^2 + E/(ar dist)) gridval
// and 0 where the reference skips the voxel (dist == 0 or beyond the cut-off).
__device__ __forceinline__ float grad_scale(const GradConsts& c, float dist2, float gridval) {
  const float e = __builtin_amdgcn_exp2f(dist2 * c.exp_k);
  const float rinv = __builtin_amdgcn_rsqf(dist2);
  const float s = (dist2 <= c.core2) ? c.gauss * e : fmaf(c.quad_b, rinv, c.quad_a);
  // dist2 == 0 (which the reference skips) needs no test: it lies in the Gaussian core, where s is
  // finite, and the caller multiplies the result by a zero offset
  return (dist2 <= c.reach2) ? s * gridval : 0.f;
}

// The same for a Gaussian that is cut off without a tail (final radius multiple = Gaussian
// multiple): there the scale jumps at the cut-off, so whether a voxel within rounding of it counts
// must be decided exactly as the reference decides it -- sqrtf of the uncontracted
// ((dx^2 + dy^2) + dz^2) against radius * radius_scale * final multiple
// (src/grid_maker.cu:881-919) --, not on squares.  `cut` is that product.
__device__ __forceinline__ float grad_scale_cut(const GradConsts& c, float dx, float dy, float dz,
                                                float cut, float gridval) {
  const float d2 = sq_distance_exact(dx, dy, dz);
  const float e = __builtin_amdgcn_exp2f(d2 * c.exp_k);
  return (sqrtf(d2) > cut) ? 0.f : c.gauss * e * gridval;
}

// Whether the kernels must take that path for this grid maker.
inline bool cut_without_tail(const GridArg& g) { return g.frm <= g.grm; }

// (CUT: the density jumps at its cut-off as well and takes the reference's predicates there)
template <bool BINARY, bool CUT>
__device__ __forceinline__ float point_density(const GridArg& g, float dx, float dy, float dz,
                                               float ar, float ar2, float inv_ar2, float frm2,
                                               float grm2) {
  return density<BINARY, CUT>(g, dx, dy, dz, BINARY ? ar2 : inv_ar2, ar, frm2, grm2);
}

constexpr int kRawBufferFlags = 0x00020000;   // untyped 32-bit elements, no swizzle (gfx9 family)

// a * b with 0 * anything = 0 (also infinities and NaNs)
__device__ __forceinline__ float mul_zero_wins(float a, float b) { return mul_legacy(a, b); }

// Atom gradients for index types.  One wave per atom.  The (y, z) columns of the atom's box that
// come within reach of the atom are compacted into a wave-private list (a circle's worth of
// columns instead of the square's), each lane takes one column of the list and marches along x;
// the offset in x of plane i is computed by lane i beforehand and read back as a scalar.  Per
// voxel the lane adds scale*dx to its x partial and scale to a running sum: dy and dz are fixed
// along the march, so the y and z partials are that sum times dy and dz.
//
// UNROTATE: the gradient is stored after Transform::backward(..., dotranslate = false) with the
// example's quaternion and rotation centre, with the arithmetic of that call (transform.hip), so
// that the result is the one the two calls give, bit for bit, with one launch less.
template <bool UNROTATE, bool CUT>
__global__ __launch_bounds__(kBwdThreads) void backward_index_kernel(
    GridArg g, BatchArg batch, Vec3Arg centers, const float* __restrict__ coords,
    const float* __restrict__ type_index, const float* __restrict__ radii,
    const float* __restrict__ diff, float* __restrict__ atom_gradients, Vec4Arg quats,
    Vec3Arg rot_centers) {
  // column list of each wave: (j << 16 | k) offsets inside the atom's box; a chunk of candidates
  // adds at most kWave entries to fewer than kWave pending ones
  __shared__ int s_cols[kBwdWaves][2 * kWave];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // scalar: so is the atom
  const int b = blockIdx.y;
  int begin, end;
  example_range(batch, b, begin, end);
  const float3 center = load3(centers, b);
  const float ox = center.x - g.half_dimension;
  const float oy = center.y - g.half_dimension;
  const float oz = center.z - g.half_dimension;
  const int dim = g.dim;
  const size_t chan_stride = (size_t)dim * dim * dim;
  const unsigned plane_stride = (unsigned)(dim * dim);
  const float* diff_b = diff + (size_t)b * g.ntypes * chan_stride;
  const float inv_res = 1.0f / g.resolution;
  volatile int* cols = s_cols[wave];
  constexpr int kPlanes = 16;   // planes of a column in flight together

  // the inverse rotation of this example, once per wave
  float4 un_q = make_float4(1.f, 0.f, 0.f, 0.f), un_qinv = un_q;
  float3 un_c = make_float3(0.f, 0.f, 0.f), un_shift = un_c;
  if (UNROTATE) {
#pragma clang fp contract(off)
    un_q = quat_inverse(load4(quats, b));
    un_qinv = quat_inverse(un_q);
    un_c = load3(rot_centers, b);
    const float zero = 0.f;
    un_shift = make_float3(-zero - un_c.x, -zero - un_c.y, -zero - un_c.z);
  }

  for (int a = begin + blockIdx.x * kBwdWaves + wave; a < end; a += gridDim.x * kBwdWaves) {
    float gx = 0.f, gy = 0.f, gz = 0.f, gauss = 0.f;
    const float tf = roundf(type_index[a]);  // backward rounds, forward floors
    if (tf >= 0.f && tf < (float)g.ntypes) {
      const float ax = coords[3 * a], ay = coords[3 * a + 1], az = coords[3 * a + 2];
      const float radius = radii[a];
      float densityrad, ar;
      {
#pragma clang fp contract(off)
        densityrad = radius * g.radius_scale * g.frm;
        ar = radius * g.radius_scale;
      }
      // scale = -(1/dist) d(density)/d(dist) (density_grad_dist, src/grid_maker.cu:881-898), in
      // terms of dist^2 and divided by 4/ar^2 (the partial sums are multiplied by it at the end):
      // Gaussian core  exp(-2 dist^2/ar^2) = exp2(exp_k dist^2);  quadratic tail
      // -(D/ar^2 + E/(ar dist)) ar^2/4 = quad_b/dist + quad_a, which falls to zero at the cut-off
      // and is negative beyond, so clamping at zero applies the cut-off.
      const float inv_ar = 1.0f / ar;
      const float inv_ar2 = inv_ar * inv_ar;
      const float exp_k = inv_ar2 * kNeg2Log2e;
      // an atom without extent (the padding rows of a padded batch) has no gradient, as in the
      // reference, whose distance test fails for every voxel of such an atom
      gauss = ar > 0.f ? 4.0f * inv_ar2 : 0.f;
      const float quad_a = -0.25f * g.D;
      const float quad_b = -0.25f * g.E * ar;
      const float core2 = g.grm * g.grm * ar * ar;
      const float reach2 = densityrad * densityrad;
      int lo0, lo1, lo2, ni, nj, nk;
      if (CUT) {
        // the reference's index box: a voxel exactly at +reach on an axis is outside it
        int hi0, hi1, hi2;
        bounds_1d(ox, ax, densityrad, g.resolution, dim, lo0, hi0);
        bounds_1d(oy, ay, densityrad, g.resolution, dim, lo1, hi1);
        bounds_1d(oz, az, densityrad, g.resolution, dim, lo2, hi2);
        ni = hi0 - lo0;
        nj = hi1 - lo1;
        nk = hi2 - lo2;
      } else {
        reach_range(ox, ax, densityrad, inv_res, dim, lo0, ni);
        reach_range(oy, ay, densityrad, inv_res, dim, lo1, nj);
        reach_range(oz, az, densityrad, inv_res, dim, lo2, nk);
      }
      if (ni > 0 && nj > 0 && nk > 0 && ar > 0.f) {
        const float* chan = diff_b + (size_t)(int)tf * chan_stride;
        const int ncols = nj * nk;
        const float inv_nk = __builtin_amdgcn_rcpf((float)nk);
        for (int i0 = 0; i0 < ni; i0 += kWave) {
          const int planes = min(kWave, ni - i0);
          const float dx_mine = grid_coord(ox, lo0 + i0 + lane, g.resolution) - ax;
          const int dx_lane = __float_as_int(dx_mine);
          // planes that lie beyond the Gaussian core as a whole skip its exponential
          const unsigned long long tail_planes = __ballot(dx_mine * dx_mine > core2);

          // one pass: lanes below `count` take the columns cols[0 .. count)
          auto march = [&](int count) {
            wave_lds_fence();                    // the list is complete
            const bool live = lane < count;
            const int packed = cols[live ? lane : 0];
            const int j = packed >> 16, k = packed & 0xffff;
            const float dy = grid_coord(oy, lo1 + j, g.resolution) - ay;
            const float dz = grid_coord(oz, lo2 + k, g.resolution) - az;
            const float dyz2 = live ? dy * dy + dz * dz : INFINITY;
            const unsigned lane_off = (unsigned)((lo1 + j) * dim + lo2 + k);
            float sum = 0.f;
            for (int i = 0; i < planes; i += kPlanes) {
              // buffer loads: the plane's offset is a scalar operand and the column's a 32-bit
              // vector one, so no address arithmetic is left to the vector unit; slots past the
              // last plane read the last plane again and are not used
              const size_t first = (size_t)(unsigned)(lo0 + i0 + i) * plane_stride;
              const size_t bytes = (chan_stride - first) * sizeof(float);
              const __amdgpu_buffer_rsrc_t planes_of_chan = __builtin_amdgcn_make_buffer_rsrc(
                  const_cast<float*>(chan + first), 0,
                  (int)(bytes < 0xffffffffull ? bytes : 0xffffffffull), kRawBufferFlags);
              const int last = planes - 1 - i;
              float gv[kPlanes];
#pragma unroll
              for (int u = 0; u < kPlanes; ++u)
                gv[u] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                    planes_of_chan, (int)(lane_off * 4u),
                    (int)((unsigned)min(u, last) * plane_stride * 4u), 0));
#pragma unroll
              for (int u = 0; u < kPlanes; ++u) {
                if (i + u < planes) {
                  const float dx = __int_as_float(__builtin_amdgcn_readlane(dx_lane, i + u));
                  const float dist2 = fmaf(dx, dx, dyz2);
                  const float tail =
                      fmaxf(fmaf(quad_b, __builtin_amdgcn_rsqf(dist2), quad_a), 0.f);
                  float s = tail;
                  if (CUT) {
                    // a Gaussian cut off without a tail: in or out by the reference's own test
                    // (grad_scale_cut), nothing beyond
                    const float d2 = sq_distance_exact(dx, dy, dz);
                    s = (!live || sqrtf(d2) > densityrad) ? 0.f : __builtin_amdgcn_exp2f(d2 * exp_k);
                  } else if (!((tail_planes >> (i + u)) & 1ull)) {
                    const float core = __builtin_amdgcn_exp2f(dist2 * exp_k);
                    s = dist2 <= core2 ? core : tail;
                  }
                  // 0 * x = 0 for every x: a voxel out of reach adds nothing whatever diff holds
                  const float sc = mul_zero_wins(s, gv[u]);
                  gx = fmaf(dx, sc, gx);
                  sum += sc;
                }
              }
            }
            gy = fmaf(dy, sum, gy);
            gz = fmaf(dz, sum, gz);
          };

          int pending = 0;
          for (int c0 = 0; c0 < ncols; c0 += kWave) {
            wave_lds_fence();                    // the entries moved to the front have been read
            const int cand = c0 + lane;
            const int j = (int)(((float)cand + 0.5f) * inv_nk), k = cand - j * nk;
            const float dy = grid_coord(oy, lo1 + j, g.resolution) - ay;
            const float dz = grid_coord(oz, lo2 + k, g.resolution) - az;
            const bool within = cand < ncols && dy * dy + dz * dz <= (CUT ? reach2 * 1.00001f : reach2);
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
    }
    gx = (float)(wave_sum64(gx) * (double)gauss);
    gy = (float)(wave_sum64(gy) * (double)gauss);
    gz = (float)(wave_sum64(gz) * (double)gauss);
    if (UNROTATE) {
      // src/transform.cpp:85-108 with dotranslate = false: rotate (g - c) by the inverse, add c
#pragma clang fp contract(off)
      const float3 r = quat_rotate(un_q, un_qinv, gx + un_shift.x, gy + un_shift.y, gz + un_shift.z);
      gx = r.x + un_c.x;
      gy = r.y + un_c.y;
      gz = r.z + un_c.z;
    }
    if (lane == 0) {
      atom_gradients[3 * a] = gx;
      atom_gradients[3 * a + 1] = gy;
      atom_gradients[3 * a + 2] = gz;
    }
  }
}

// Vector types.  TG channels are handled per pass so that the per-lane type
// gradient partials stay in registers.
template <bool BINARY, bool RTI, int TG, bool CUT>
__global__ __launch_bounds__(kBwdThreads) void backward_vector_kernel(
    GridArg g, BatchArg batch, Vec3Arg centers, const float* __restrict__ coords,
    const float* __restrict__ type_vector, const float* __restrict__ radii,
    const float* __restrict__ diff, float* __restrict__ atom_gradients,
    float* __restrict__ type_gradients) {
  __shared__ int s_cols[kBwdWaves][2 * kWave];   // column list of each wave (sweep_reach)
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // scalar: so is the atom
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
  const float* diff_b = diff + (size_t)b * T * chan_stride;
  const float* radii_b = RTI ? radii + (size_t)b * T : radii;
  const float frm2 = g.frm * g.frm, grm2 = g.grm * g.grm;

  for (int a0 = begin + blockIdx.x * kBwdWaves + wave; a0 < end; a0 += gridDim.x * kBwdWaves) {
    const int a = __builtin_amdgcn_readfirstlane(a0);
    const float ax = coords[3 * a], ay = coords[3 * a + 1], az = coords[3 * a + 2];
    const float* __restrict__ tv = type_vector + (size_t)a * T;
    float gx = 0.f, gy = 0.f, gz = 0.f;

    if (!RTI) {
      const float radius = radii_b[a];
      float densityrad, ar, ar2;
      {
#pragma clang fp contract(off)
        densityrad = radius * g.radius_scale * g.frm;
        ar = radius * g.radius_scale;
        ar2 = ar * ar;
      }
      const GradConsts gc = grad_consts(g, ar);
      const float inv_ar2 = gc.inv_ar2;
      const bool any = ar > 0.f && densityrad > 0.f;             // no extent: no gradient
      // density and gradient scale vanish beyond the final radius; where the box decides which
      // voxels count, the sweep follows the box
      const bool index_box = needs_index_box(g, BINARY);
      for (int cbase = 0; cbase < T; cbase += TG) {
        const int nchan = min(TG, T - cbase);
        float tg[TG];
#pragma unroll
        for (int t = 0; t < TG; ++t) tg[t] = 0.f;
        if (any) {
          const float* group = diff_b + (size_t)cbase * chan_stride;
          sweep_reach(g, lane, s_cols[wave], ox, oy, oz, ax, ay, az, densityrad, index_box,
                    [&](float dx, float dy, float dz, float dist2, unsigned plane_off,
                        unsigned lane_off, bool live) {
                      float val = point_density<BINARY, CUT>(g, dx, dy, dz, ar, ar2, inv_ar2, frm2, grm2);
                      if (!live) val = 0.f;
                      const float* p = group + plane_off;
                      float weighted = 0.f;  // sum_t weight_t * diff_t at this voxel
#pragma unroll
                      for (int t = 0; t < TG; ++t) {
                        if (t < nchan) {
                          const float gv = (p + (size_t)t * chan_stride)[lane_off];
                          tg[t] = fmaf(val, gv, tg[t]);
                          weighted = fmaf(tv[cbase + t], gv, weighted);
                        }
                      }
                      const float sc = CUT ? grad_scale_cut(gc, dx, dy, dz, densityrad, live ? weighted : 0.f)
                                           : grad_scale(gc, dist2, weighted);
                      gx = fmaf(dx, sc, gx);
                      gy = fmaf(dy, sc, gy);
                      gz = fmaf(dz, sc, gz);
                    });
        }
#pragma unroll
        for (int t = 0; t < TG; ++t) {
          if (t < nchan) {
            const float s = wave_sum(tg[t]);
            if (lane == 0) type_gradients[(size_t)a * T + cbase + t] = s;
          }
        }
      }
    } else {
      // radius per type: every channel has its own box
      for (int t = 0; t < T; ++t) {
        const float radius = radii_b[t];
        const float tm = tv[t];
        float densityrad, ar, ar2;
        {
#pragma clang fp contract(off)
          densityrad = radius * g.radius_scale * g.frm;
          ar = radius * g.radius_scale;
          ar2 = ar * ar;
        }
        const GradConsts gc = grad_consts(g, ar);
        const float inv_ar2 = gc.inv_ar2;
        float tgt = 0.f, tx = 0.f, ty = 0.f, tz = 0.f;
        if (ar > 0.f && densityrad > 0.f) {
          const float* chan = diff_b + (size_t)t * chan_stride;
          sweep_reach(g, lane, s_cols[wave], ox, oy, oz, ax, ay, az, densityrad,
                      needs_index_box(g, BINARY),
                        [&](float dx, float dy, float dz, float dist2, unsigned plane_off,
                            unsigned lane_off, bool live) {
                          const float gv = (chan + plane_off)[lane_off];
                          float val = point_density<BINARY, CUT>(g, dx, dy, dz, ar, ar2, inv_ar2, frm2, grm2);
                          if (!live) val = 0.f;
                          tgt = fmaf(val, gv, tgt);
                          const float sc = CUT ? grad_scale_cut(gc, dx, dy, dz, densityrad, live ? gv : 0.f)
                                               : grad_scale(gc, dist2, gv);
                          tx = fmaf(dx, sc, tx);
                          ty = fmaf(dy, sc, ty);
                          tz = fmaf(dz, sc, tz);
                        });
        }
        const float s = wave_sum(tgt);
        if (lane == 0) type_gradients[(size_t)a * T + t] = s;
        if (tm != 0.f) {
          gx = fmaf(tx, tm, gx);
          gy = fmaf(ty, tm, gy);
          gz = fmaf(tz, tm, gz);
        }
      }
    }
    gx = wave_sum(gx);
    gy = wave_sum(gy);
    gz = wave_sum(gz);
    if (lane == 0) {
      atom_gradients[3 * a] = gx;
      atom_gradients[3 * a + 1] = gy;
      atom_gradients[3 * a + 2] = gz;
    }
  }
}

int backward_blocks(int launch_atoms) {
  int blocks = (launch_atoms + kBwdWaves - 1) / kBwdWaves;
  if (blocks < 1) blocks = 1;
  if (blocks > 4096) blocks = 4096;
  return blocks;
}

template <bool BINARY, bool RTI>
hipError_t launch_vec(const GridArg& g, const BatchArg& batch, int nbatch, int launch_atoms,
                      const Vec3Arg& centers, const float* coords, const float* type_vector,
                      const float* radii, const float* diff, float* atom_gradients,
                      float* type_gradients, hipStream_t stream) {
  dim3 grid(backward_blocks(launch_atoms), nbatch), block(kBwdThreads);
  if (cut_without_tail(g))      // (a rare mode: one channel-group size serves it)
    hipLaunchKernelGGL((backward_vector_kernel<BINARY, RTI, 8, true>), grid, block, 0, stream, g,
                       batch, centers, coords, type_vector, radii, diff, atom_gradients,
                       type_gradients);
  else if (g.ntypes <= 8)
    hipLaunchKernelGGL((backward_vector_kernel<BINARY, RTI, 8, false>), grid, block, 0, stream, g, batch,
                       centers, coords, type_vector, radii, diff, atom_gradients, type_gradients);
  else if (g.ntypes <= 16)
    hipLaunchKernelGGL((backward_vector_kernel<BINARY, RTI, 16, false>), grid, block, 0, stream, g, batch,
                       centers, coords, type_vector, radii, diff, atom_gradients, type_gradients);
  else
    hipLaunchKernelGGL((backward_vector_kernel<BINARY, RTI, 32, false>), grid, block, 0, stream, g, batch,
                       centers, coords, type_vector, radii, diff, atom_gradients, type_gradients);
  return hipGetLastError();
}

}  // namespace

hipError_t launch_backward_index(const GridArg& g, const BatchArg& batch, int nbatch,
                                 int launch_atoms, const Vec3Arg& centers, const float* coords,
                                 const float* type_index, const float* radii, const float* diff,
                                 float* atom_gradients, hipStream_t stream) {
  dim3 grid(backward_blocks(launch_atoms), nbatch), block(kBwdThreads);
  const Vec4Arg no_quats{nullptr, {1.f, 0.f, 0.f, 0.f}};
  const Vec3Arg no_centers{nullptr, {0.f, 0.f, 0.f}};
  if (cut_without_tail(g))
    hipLaunchKernelGGL((backward_index_kernel<false, true>), grid, block, 0, stream, g, batch, centers,
                       coords, type_index, radii, diff, atom_gradients, no_quats, no_centers);
  else
    hipLaunchKernelGGL((backward_index_kernel<false, false>), grid, block, 0, stream, g, batch, centers,
                       coords, type_index, radii, diff, atom_gradients, no_quats, no_centers);
  return hipGetLastError();
}

hipError_t launch_backward_index_unrotated(const GridArg& g, const BatchArg& batch, int nbatch,
                                           int launch_atoms, const Vec3Arg& centers,
                                           const float* coords, const float* type_index,
                                           const float* radii, const float* diff,
                                           const Vec4Arg& quats, const Vec3Arg& rot_centers,
                                           float* atom_gradients, hipStream_t stream) {
  dim3 grid(backward_blocks(launch_atoms), nbatch), block(kBwdThreads);
  if (cut_without_tail(g))
    hipLaunchKernelGGL((backward_index_kernel<true, true>), grid, block, 0, stream, g, batch, centers,
                       coords, type_index, radii, diff, atom_gradients, quats, rot_centers);
  else
    hipLaunchKernelGGL((backward_index_kernel<true, false>), grid, block, 0, stream, g, batch, centers,
                       coords, type_index, radii, diff, atom_gradients, quats, rot_centers);
  return hipGetLastError();
}

hipError_t launch_backward_vector(const GridArg& g, const BatchArg& batch, int nbatch,
                                  int launch_atoms, const Vec3Arg& centers, const float* coords,
                                  const float* type_vector, const float* radii, const float* diff,
                                  float* atom_gradients, float* type_gradients, bool binary,
                                  bool radii_type_indexed, hipStream_t stream) {
  if (binary && radii_type_indexed)
    return launch_vec<true, true>(g, batch, nbatch, launch_atoms, centers, coords, type_vector,
                                  radii, diff, atom_gradients, type_gradients, stream);
  if (binary)
    return launch_vec<true, false>(g, batch, nbatch, launch_atoms, centers, coords, type_vector,
                                   radii, diff, atom_gradients, type_gradients, stream);
  if (radii_type_indexed)
    return launch_vec<false, true>(g, batch, nbatch, launch_atoms, centers, coords, type_vector,
                                   radii, diff, atom_gradients, type_gradients, stream);
  return launch_vec<false, false>(g, batch, nbatch, launch_atoms, centers, coords, type_vector,
                                  radii, diff, atom_gradients, type_gradients, stream);
}

}  // namespace mg
