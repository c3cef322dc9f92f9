// Forward density splat for vector-typed atoms on gfx950.
//
// Same tiling and culling as the index-typed kernel (one workgroup per 8x8x8
// tile, ballot-compacted candidate list, second cull per 4x4x4 wave sub-tile),
// but every atom feeds all channels, so each lane keeps one voxel's channel
// sums in registers: the atom's density is evaluated once and multiplied into
// TG channel accumulators with the atom's type weights, which are read through
// wave-uniform addresses.  Sums run over atoms in ascending order, as the CPU
// loop does (src/grid_maker.cpp:226-270), so binary mode (`+= weight`) is
// reproduced bit for bit.  The tile is staged through LDS and streamed out as
// float4 rows.
#include "kernels.h"
#include "splat_common.h"

namespace mg {

namespace {

// BINARY / EXACT as in density(); RTI = radii indexed by type instead of atom;
// TG = channels accumulated per pass (register array size).
template <bool BINARY, bool EXACT, bool RTI, int TG>
__global__ __launch_bounds__(kSplatThreads) void splat_vector_kernel(
    GridArg g, BatchArg batch, Vec3Arg centers, const float* __restrict__ coords,
    const float* __restrict__ type_vector, const float* __restrict__ radii,
    float* __restrict__ out, int tiles_per_side, int vec_store) {
  // [TG][512] floats of output staging, declared as 16-byte vectors so that the compiler knows
  // the alignment (the write-out reads it with one 128-bit LDS instruction per piece)
  HIP_DYNAMIC_SHARED(v4f, s_stage_v4);
  float* const s_stage = reinterpret_cast<float*>(s_stage_v4);
  __shared__ int s_cand[kCandCap];
  __shared__ float4 s_rec[kChunk];   // x, y, z, (ar^2 | 1/ar^2) (w unused when RTI)
  __shared__ int s_recatom[kChunk];  // atom index of each record
  __shared__ uint4 s_clip[(EXACT && !RTI) ? kChunk : 1];
  __shared__ unsigned char s_wlist[kSplatWaves][kChunk];
  __shared__ int s_wcount[kSplatWaves];
  __shared__ float s_type_ar[RTI ? kMaxChannelGroup : 1];  // radius*radius_scale per type
  __shared__ float s_type_w[RTI ? kMaxChannelGroup : 1];   // ar^2 | 1/ar^2 per type

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid >> 6;
  const int b = blockIdx.y;
  int begin, end;
  example_range(batch, b, begin, end);
  const SplatGeom s = make_geom(g, load3(centers, b), blockIdx.x, tiles_per_side, wave, lane);
  const int dim = g.dim;
  const int T = g.ntypes;
  const float frm2 = g.frm * g.frm;
  const float grm2 = g.grm * g.grm;
  const float cull_mult = BINARY ? 1.0f : g.frm;
  const float* radii_b = RTI ? radii + (size_t)b * T : radii;

  const size_t chan_stride = (size_t)dim * dim * dim;
  float* out_b = out + (size_t)b * T * chan_stride;

  for (int cbase = 0; cbase < T; cbase += TG) {
    const int nchan = min(TG, T - cbase);
    float acc[TG];
#pragma unroll
    for (int t = 0; t < TG; ++t) acc[t] = 0.f;

    // type-indexed radii: per-type constants of this channel group and the
    // largest reach among them (the reference culls by the maximum radius,
    // src/grid_maker.cu:421-426)
    float group_reach = 0.f;
    if (RTI) {
      __syncthreads();
      if (tid < nchan) {
        float ar, ar2;
        {
#pragma clang fp contract(off)
          ar = radii_b[cbase + tid] * g.radius_scale;
          ar2 = ar * ar;
        }
        s_type_ar[tid] = ar;
        s_type_w[tid] = BINARY ? ar2 : 1.0f / ar2;
      }
      __syncthreads();
      for (int t = 0; t < nchan; ++t) group_reach = fmaxf(group_reach, s_type_ar[t] * cull_mult);
    }

    int a0 = begin;
    do {
      int ncand = 0;
      while (a0 < end && ncand <= kCandCap - kSplatThreads) {
        const int a = a0 + tid;
        bool pass = false;
        if (a < end) {
          const float reach = RTI ? group_reach : radii_b[a] * g.radius_scale * cull_mult;
          const float d2 = box_distance2(coords[3 * a], coords[3 * a + 1], coords[3 * a + 2],
                                         s.tlo[0], s.tlo[1], s.tlo[2], s.thi[0], s.thi[1],
                                         s.thi[2]);
          pass = d2 <= reach * reach * kCullSlack;
        }
        ncand += append_candidates(pass, a, s_cand, ncand, s_wcount, wave, lane);
        a0 += kSplatThreads;
      }

      for (int c0 = 0; c0 < ncand; c0 += kChunk) {
        const int m = min(kChunk, ncand - c0);
        if (tid < m) {
          const int a = s_cand[c0 + tid];
          const float ax = coords[3 * a], ay = coords[3 * a + 1], az = coords[3 * a + 2];
          float w = 0.f;
          if (!RTI) {
            const float radius = radii_b[a];
            float ar, ar2;
            {
#pragma clang fp contract(off)
              ar = radius * g.radius_scale;
              ar2 = ar * ar;
            }
            w = BINARY ? ar2 : 1.0f / ar2;
            if (EXACT) {
              const uint3 cl = pack_clip(g, s, ax, ay, az, radius);
              s_clip[tid] = make_uint4(cl.x, cl.y, cl.z, __float_as_uint(ar));
            }
          }
          s_rec[tid] = make_float4(ax, ay, az, w);
          s_recatom[tid] = a;
        }
        __syncthreads();

        int wcnt = 0;
        if (s.wave_live) {
          for (int r0 = 0; r0 < m; r0 += kWave) {
            const int i = r0 + lane;
            bool pass = false;
            if (i < m) {
              const float4 rec = s_rec[i];
              const float d2 = box_distance2(rec.x, rec.y, rec.z, s.wlo[0], s.wlo[1], s.wlo[2],
                                             s.whi[0], s.whi[1], s.whi[2]);
              if (RTI) pass = d2 <= group_reach * group_reach * kCullSlack;
              else pass = BINARY ? (d2 <= rec.w * kCullSlack) : (d2 * rec.w <= frm2 * kCullSlack);
            }
            const unsigned long long bm = __ballot(pass);
            if (pass) s_wlist[wave][wcnt + __popcll(bm & ((1ull << lane) - 1ull))] = (unsigned char)i;
            wcnt += __popcll(bm);
          }
        }
        __syncthreads();

        for (int it = 0; it < wcnt; ++it) {
          const int ri = s_wlist[wave][it];
          const float4 rec = s_rec[ri];
          // wave-uniform atom index -> the weights come in through scalar loads
          const int a = __builtin_amdgcn_readfirstlane(s_recatom[ri]);
          const float* __restrict__ tv = type_vector + (size_t)a * T + cbase;
          const float dx = s.vx - rec.x, dy = s.vy - rec.y, dz = s.vz - rec.z;
          if (!RTI) {
            bool inside = s.voxel_live;
            float ar = 0.f;
            if (EXACT) {
              const uint4 cl = s_clip[ri];
              inside = inside && inside_clip(s, make_uint3(cl.x, cl.y, cl.z));
              ar = __uint_as_float(cl.w);
            }
            float val = density<BINARY, EXACT>(g, dx, dy, dz, rec.w, ar, frm2, grm2);
            if (!inside) val = 0.f;
            if (BINARY) {
              if (val != 0.f) {
#pragma unroll
                for (int t = 0; t < TG; ++t)
                  if (t < nchan) acc[t] += tv[t];
              }
            } else {
#pragma unroll
              for (int t = 0; t < TG; ++t)
                if (t < nchan) acc[t] = fmaf(val, tv[t], acc[t]);
            }
          } else {
            // a different radius per channel: density (and index box) per type
#pragma unroll
            for (int t = 0; t < TG; ++t) {
              if (t < nchan) {
                const float tm = tv[t];
                if (tm != 0.f) {
                  const float ar = s_type_ar[t];
                  bool inside = s.voxel_live;
                  if (EXACT) {
                    float radius = radii_b[cbase + t];
                    inside = inside && inside_clip(s, pack_clip(g, s, rec.x, rec.y, rec.z, radius));
                  }
                  const float val = density<BINARY, EXACT>(g, dx, dy, dz, s_type_w[t], ar, frm2, grm2);
                  if (inside && val != 0.f) {
                    if (BINARY) acc[t] += tm;
                    else acc[t] = fmaf(val, tm, acc[t]);
                  }
                }
              }
            }
          }
        }
        __syncthreads();
      }
    } while (a0 < end);

    // ---- stage through LDS and stream out as float4 rows ----------------------
    __syncthreads();
#pragma unroll
    for (int t = 0; t < TG; ++t)
      if (t < nchan) s_stage[t * kTileVox + s.slot] = acc[t];
    __syncthreads();
    for (int item = tid; item < nchan * 128; item += kSplatThreads) {
      const int c = item >> 7;
      const int r = item & 127;
      const int x = r >> 4, y = (r >> 1) & 7, h = r & 1;
      const int gx = s.x0 + x, gy = s.y0 + y, gz = s.z0 + h * 4;
      if (gx < dim && gy < dim && gz < dim) {
        const v4f v = *reinterpret_cast<const v4f*>(s_stage + c * kTileVox + lds_voxel(x, y, h * 4));
        float* dst = out_b + (size_t)(cbase + c) * chan_stride + ((size_t)gx * dim + gy) * dim + gz;
        if (vec_store && gz + 3 < dim) {
          __builtin_nontemporal_store(v, reinterpret_cast<v4f*>(dst));
        } else {
          dst[0] = v.x;
          if (gz + 1 < dim) dst[1] = v.y;
          if (gz + 2 < dim) dst[2] = v.z;
          if (gz + 3 < dim) dst[3] = v.w;
        }
      }
    }
    __syncthreads();
  }
}

template <bool BINARY, bool EXACT, bool RTI, int TG>
hipError_t launch_one(const GridArg& g, const BatchArg& batch, int nbatch, const Vec3Arg& centers,
                      const float* coords, const float* type_vector, const float* radii,
                      float* out, hipStream_t stream) {
  const int tiles_per_side = (g.dim + kTile - 1) / kTile;
  const int tiles = tiles_per_side * tiles_per_side * tiles_per_side;
  const size_t dyn_lds = (size_t)TG * kTileVox * sizeof(float);
  const size_t chan_stride = (size_t)g.dim * g.dim * g.dim;
  const int vec_store = (g.dim % 4 == 0) && ((reinterpret_cast<uintptr_t>(out) & 15) == 0) &&
                        ((chan_stride * g.ntypes) % 4 == 0);
  auto kern = splat_vector_kernel<BINARY, EXACT, RTI, TG>;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)dyn_lds);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(kern, dim3(tiles, nbatch), dim3(kSplatThreads), dyn_lds, stream, g, batch,
                     centers, coords, type_vector, radii, out, tiles_per_side, vec_store);
  return hipGetLastError();
}

template <bool BINARY, bool RTI>
hipError_t launch_sized(const GridArg& g, const BatchArg& batch, int nbatch, const Vec3Arg& centers,
                        const float* coords, const float* type_vector, const float* radii,
                        float* out, bool exact, hipStream_t stream) {
  if (exact)
    return launch_one<BINARY, true, RTI, 32>(g, batch, nbatch, centers, coords, type_vector, radii, out, stream);
  if (g.ntypes <= 8)
    return launch_one<BINARY, false, RTI, 8>(g, batch, nbatch, centers, coords, type_vector, radii, out, stream);
  if (g.ntypes <= 16)
    return launch_one<BINARY, false, RTI, 16>(g, batch, nbatch, centers, coords, type_vector, radii, out, stream);
  if (g.ntypes <= 28)
    return launch_one<BINARY, false, RTI, 28>(g, batch, nbatch, centers, coords, type_vector, radii, out, stream);
  return launch_one<BINARY, false, RTI, 32>(g, batch, nbatch, centers, coords, type_vector, radii, out, stream);
}

}  // namespace

hipError_t launch_forward_vector(const GridArg& g, const BatchArg& batch, int nbatch,
                                 const Vec3Arg& centers, const float* coords,
                                 const float* type_vector, const float* radii, float* out,
                                 bool binary, bool radii_type_indexed, bool exact,
                                 void* workspace, size_t workspace_bytes, hipStream_t stream) {
  // per-atom radii take the matrix-core kernel; type-indexed radii and the exact-predicate modes
  // (truncated Gaussian) use the cubic-tile kernel below
  if (!radii_type_indexed && !exact)
    return launch_forward_vector_mfma(g, batch, nbatch, centers, coords, type_vector, radii, out,
                                      binary, workspace, workspace_bytes, stream);
  if (binary && radii_type_indexed)
    return launch_sized<true, true>(g, batch, nbatch, centers, coords, type_vector, radii, out, exact, stream);
  if (binary)
    return launch_sized<true, false>(g, batch, nbatch, centers, coords, type_vector, radii, out, exact, stream);
  if (radii_type_indexed)
    return launch_sized<false, true>(g, batch, nbatch, centers, coords, type_vector, radii, out, exact, stream);
  return launch_sized<false, false>(g, batch, nbatch, centers, coords, type_vector, radii, out, exact, stream);
}

}  // namespace mg
