// Forward density splat for index-typed atoms on gfx950.
//
// One workgroup (8 waves of 64 lanes) owns an 8x8x8 voxel tile of one example
// and produces every channel of it:
//   1. the tile's channel accumulators live in LDS and are cleared there (no
//      memset pass over HBM);
//   2. all atoms of the example are tested against the tile's bounding box; the
//      survivors are compacted, in ascending atom order, into an LDS list with a
//      wavefront ballot + prefix count;
//   3. each wave culls that list again against its own 4x4x4 sub-tile;
//   4. every lane owns one voxel and walks its wave's list in order, adding the
//      density to its own LDS accumulator (no two lanes share a voxel, so the
//      sum order per voxel is the ascending atom order of the CPU loop,
//      src/grid_maker.cpp:170-211);
//   5. the tile is streamed to HBM once, as float4 rows along z per channel.
#include "kernels.h"
#include "splat_common.h"

namespace mg {

namespace {

template <bool BINARY, bool EXACT>
__global__ __launch_bounds__(kSplatThreads) void splat_index_kernel(
    GridArg g, BatchArg batch, Vec3Arg centers, const float* __restrict__ coords,
    const float* __restrict__ type_index, const float* __restrict__ radii,
    float* __restrict__ out, int tiles_per_side, int chan_group, int vec_store) {
  extern __shared__ __align__(16) float s_acc[];  // [chan_group][512]
  __shared__ int s_cand[kCandCap];
  __shared__ float4 s_rec[kChunk];  // x, y, z, (ar^2 | 1/ar^2)
  __shared__ unsigned char s_rectype[kChunk];
  __shared__ uint4 s_clip[EXACT ? kChunk : 1];  // index box + ar, EXACT only
  __shared__ unsigned short s_wlist[kSplatWaves][kChunk];
  __shared__ int s_wcount[kSplatWaves];

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid >> 6;
  const int b = blockIdx.y;
  int begin, end;
  example_range(batch, b, begin, end);
  const SplatGeom s = make_geom(g, load3(centers, b), blockIdx.x, tiles_per_side, wave, lane);
  const int dim = g.dim;
  const float frm2 = g.frm * g.frm;
  const float grm2 = g.grm * g.grm;
  const float cull_mult = BINARY ? 1.0f : g.frm;  // support radius / ar

  const size_t chan_stride = (size_t)dim * dim * dim;
  float* out_b = out + (size_t)b * g.ntypes * chan_stride;

  for (int cbase = 0; cbase < g.ntypes; cbase += chan_group) {
    const int nchan = min(chan_group, g.ntypes - cbase);
    for (int i = tid; i < nchan * (kTileVox / 4); i += kSplatThreads)
      reinterpret_cast<float4*>(s_acc)[i] = make_float4(0.f, 0.f, 0.f, 0.f);

    int a0 = begin;
    do {
      // ---- scan atoms against the tile until the candidate list may overflow
      int ncand = 0;
      while (a0 < end && ncand <= kCandCap - kSplatThreads) {
        const int a = a0 + tid;
        bool pass = false;
        if (a < end) {
          const float tf = floorf(type_index[a]);
          if (tf >= (float)cbase && tf < (float)(cbase + nchan)) {
            const float reach = radii[a] * g.radius_scale * cull_mult;
            const float d2 = box_distance2(coords[3 * a], coords[3 * a + 1], coords[3 * a + 2],
                                           s.tlo[0], s.tlo[1], s.tlo[2], s.thi[0], s.thi[1],
                                           s.thi[2]);
            pass = d2 <= reach * reach * kCullSlack;
          }
        }
        ncand += append_candidates(pass, a, s_cand, ncand, s_wcount, wave, lane);
        a0 += kSplatThreads;
      }

      for (int c0 = 0; c0 < ncand; c0 += kChunk) {
        // ---- LDS records for up to 256 candidates ---------------------------
        const int m = min(kChunk, ncand - c0);
        if (tid < m) {
          const int a = s_cand[c0 + tid];
          const float ax = coords[3 * a], ay = coords[3 * a + 1], az = coords[3 * a + 2];
          const float radius = radii[a];
          float ar, ar2;
          {
#pragma clang fp contract(off)
            ar = radius * g.radius_scale;
            ar2 = ar * ar;
          }
          s_rec[tid] = make_float4(ax, ay, az, BINARY ? ar2 : 1.0f / ar2);
          s_rectype[tid] = (unsigned char)((int)floorf(type_index[a]) - cbase);
          if (EXACT) {
            const uint3 cl = pack_clip(g, s, ax, ay, az, radius);
            s_clip[tid] = make_uint4(cl.x, cl.y, cl.z, __float_as_uint(ar));
          }
        }
        __syncthreads();

        // ---- per-wave cull against the 4x4x4 sub-tile --------------------------
        int wcnt = 0;
        if (s.wave_live) {
          for (int r0 = 0; r0 < m; r0 += kWave) {
            const int i = r0 + lane;
            bool pass = false;
            if (i < m) {
              const float4 rec = s_rec[i];
              const float d2 = box_distance2(rec.x, rec.y, rec.z, s.wlo[0], s.wlo[1], s.wlo[2],
                                             s.whi[0], s.whi[1], s.whi[2]);
              pass = BINARY ? (d2 <= rec.w * kCullSlack) : (d2 * rec.w <= frm2 * kCullSlack);
            }
            const unsigned long long bm = __ballot(pass);
            if (pass)
              s_wlist[wave][wcnt + __popcll(bm & ((1ull << lane) - 1ull))] =
                  (unsigned short)(i | (s_rectype[i] << 8));
            wcnt += __popcll(bm);
          }
        }
        __syncthreads();

        // ---- accumulate: one voxel per lane, atoms in ascending order ----------
        for (int it = 0; it < wcnt; ++it) {
          const unsigned e = s_wlist[wave][it];
          const int ri = e & 0xff;
          const float4 rec = s_rec[ri];
          float* cell = s_acc + (e >> 8) * kTileVox + s.slot;
          bool inside = s.voxel_live;
          float ar = 0.f;
          if (EXACT) {
            const uint4 cl = s_clip[ri];
            inside = inside && inside_clip(s, make_uint3(cl.x, cl.y, cl.z));
            ar = __uint_as_float(cl.w);
          }
          const float val = density<BINARY, EXACT>(g, s.vx - rec.x, s.vy - rec.y, s.vz - rec.z,
                                                   rec.w, ar, frm2, grm2);
          if (inside && val != 0.f) {
            if (BINARY) *cell = 1.0f;
            else __hip_atomic_fetch_add(cell, val, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
          }
        }
        __syncthreads();
      }
    } while (a0 < end);

    // ---- stream the tile out: float4 rows along z, one channel plane at a time
    __syncthreads();
    for (int item = tid; item < nchan * 128; item += kSplatThreads) {
      const int c = item >> 7;
      const int r = item & 127;
      const int x = r >> 4, y = (r >> 1) & 7, h = r & 1;
      const int gx = s.x0 + x, gy = s.y0 + y, gz = s.z0 + h * 4;
      if (gx < dim && gy < dim && gz < dim) {
        const v4f v = *reinterpret_cast<const v4f*>(s_acc + c * kTileVox + lds_voxel(x, y, h * 4));
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

template <bool BINARY, bool EXACT>
hipError_t launch_one(const GridArg& g, const BatchArg& batch, int nbatch, const Vec3Arg& centers,
                      const float* coords, const float* type_index, const float* radii,
                      float* out, hipStream_t stream) {
  const int tiles_per_side = (g.dim + kTile - 1) / kTile;
  const int tiles = tiles_per_side * tiles_per_side * tiles_per_side;
  const int chan_group = g.ntypes < kMaxChannelGroup ? g.ntypes : kMaxChannelGroup;
  const size_t dyn_lds = (size_t)chan_group * kTileVox * sizeof(float);
  const size_t chan_stride = (size_t)g.dim * g.dim * g.dim;
  const int vec_store = (g.dim % 4 == 0) && ((reinterpret_cast<uintptr_t>(out) & 15) == 0) &&
                        ((chan_stride * g.ntypes) % 4 == 0);
  auto kern = splat_index_kernel<BINARY, EXACT>;
  // the workgroup needs more than the default 64 KiB of LDS
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                     hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)(kMaxChannelGroup * kTileVox * sizeof(float)));
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(kern, dim3(tiles, nbatch), dim3(kSplatThreads), dyn_lds, stream, g, batch,
                     centers, coords, type_index, radii, out, tiles_per_side, chan_group,
                     vec_store);
  return hipGetLastError();
}

}  // namespace

hipError_t launch_forward_index(const GridArg& g, const BatchArg& batch, int nbatch,
                                const Vec3Arg& centers, const float* coords,
                                const float* type_index, const float* radii, float* out,
                                bool binary, bool exact, hipStream_t stream) {
  if (binary && exact)
    return launch_one<true, true>(g, batch, nbatch, centers, coords, type_index, radii, out, stream);
  if (binary)
    return launch_one<true, false>(g, batch, nbatch, centers, coords, type_index, radii, out, stream);
  if (exact)
    return launch_one<false, true>(g, batch, nbatch, centers, coords, type_index, radii, out, stream);
  return launch_one<false, false>(g, batch, nbatch, centers, coords, type_index, radii, out, stream);
}

}  // namespace mg
