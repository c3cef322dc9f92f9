// Forward density splat for index-typed atoms on gfx950.
//
// One workgroup of four waves owns a column of the grid: 4 x 4 voxels in (x, y)
// and up to 48 voxels along z, for every channel.
//   scan    each wave walks a quarter of the example's atoms (loads batched four
//           deep), keeps those whose density support touches the column's box
//           and compacts their indices, in ascending order, into its own LDS
//           segment with a wavefront ballot + prefix count;
//   records the survivors become 16-byte LDS records (x, y, z, 1/ar^2);
//   cull    per 4x4x4 block (three blocks per wave) the records are culled again
//           and compacted into a wave-private list;
//   splat   every lane owns one voxel per block and walks the list in atom order.
//           The channel of an atom is uniform across the wave, so the 28 channel
//           sums of a voxel live in registers and are addressed through the
//           scalar register index (no LDS atomics, no read-modify-write of HBM);
//   store   the column is staged through LDS four channels at a time and written
//           out as full z rows (768 contiguous bytes per channel and x), which is
//           the pattern the HBM write path sustains best; nothing is memset.
// Per voxel the contributions are added in ascending atom order, as in the CPU
// loop (src/grid_maker.cpp:170-211).
#include "kernels.h"
#include "splat_common.h"

namespace mg {

namespace {

constexpr int kColXY = 4;                        // column is 4 x 4 voxels in x, y
constexpr int kBlocksPerWave = 3;                // 4x4x4 blocks per wave
constexpr int kColWaves = 4;
constexpr int kColThreads = kColWaves * kWave;   // 256
constexpr int kSlabZ = kColWaves * kBlocksPerWave * 4;  // 48 voxels of z per workgroup
constexpr int kRegChannels = 28;                 // channel sums kept in registers per voxel
constexpr int kRowPad = 52;                      // staged z row, padded against bank conflicts
constexpr int kPlane = 16 * kRowPad;             // one staged channel: 16 rows
constexpr int kStageCh = 4;                      // channels staged per round
constexpr int kSuper = 4096;                     // atoms scanned per pass
constexpr int kSeg = kSuper / kColWaves;         // per wave
constexpr int kRecChunk = 256;

// LDS-only barrier: outstanding global stores are not waited for.
__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

template <bool BINARY, bool EXACT>
__global__ __launch_bounds__(kColThreads) void splat_index_kernel(
    GridArg g, BatchArg batch, Vec3Arg centers, const float* __restrict__ coords,
    const float* __restrict__ type_index, const float* __restrict__ radii,
    float* __restrict__ out, int cols_per_side, int vec_store) {
  __shared__ unsigned short s_idx[kColWaves][kSeg];
  __shared__ int s_wcount[kColWaves];
  __shared__ float4 s_rec[kRecChunk];            // x, y, z, (ar^2 | 1/ar^2)
  __shared__ unsigned char s_rectype[kRecChunk];
  __shared__ uint4 s_clip[EXACT ? kRecChunk : 1];  // index box + ar, EXACT only
  __shared__ float4 s_mini[kColWaves][kWave];
  __shared__ uint4 s_miniclip[EXACT ? kColWaves : 1][EXACT ? kWave : 1];
  __shared__ unsigned char s_minitype[kColWaves][kWave + 4];
  __shared__ __align__(16) float s_stage[2 * kStageCh * kPlane];

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid >> 6;
  const int b = blockIdx.y;
  int begin, end;
  example_range(batch, b, begin, end);
  const float3 center = load3(centers, b);
  const float ox = center.x - g.half_dimension;
  const float oy = center.y - g.half_dimension;
  const float oz = center.z - g.half_dimension;
  const int dim = g.dim;

  // which column / z slab this workgroup owns
  const int ncols = cols_per_side * cols_per_side;
  const int slab = blockIdx.x / ncols;
  const int col = blockIdx.x - slab * ncols;
  const int x0 = (col / cols_per_side) * kColXY, y0 = (col % cols_per_side) * kColXY;
  const int z0 = slab * kSlabZ;
  const int zend = min(z0 + kSlabZ, dim);          // exclusive

  const int lx = lane >> 4, ly = (lane >> 2) & 3, lz = lane & 3;
  const int vxi = x0 + lx, vyi = y0 + ly;
  const bool xy_live = vxi < dim && vyi < dim;
  const float vx = grid_coord(ox, vxi, g.resolution), vy = grid_coord(oy, vyi, g.resolution);
  // box of the column (first/last voxel centre inside the grid)
  const float clx = grid_coord(ox, x0, g.resolution), cly = grid_coord(oy, y0, g.resolution);
  const float clz = grid_coord(oz, z0, g.resolution);
  const float chx = grid_coord(ox, min(x0 + kColXY, dim) - 1, g.resolution);
  const float chy = grid_coord(oy, min(y0 + kColXY, dim) - 1, g.resolution);
  const float chz = grid_coord(oz, zend - 1, g.resolution);

  const float frm2 = g.frm * g.frm;
  const float grm2 = g.grm * g.grm;
  const float cull_mult = BINARY ? 1.0f : g.frm;  // support radius / ar
  const size_t chan_stride = (size_t)dim * dim * dim;
  float* out_b = out + (size_t)b * g.ntypes * chan_stride;

  const int dump_off = lx * (4 * kRowPad) + ly * kRowPad + wave * kBlocksPerWave * 4 + lz;

  for (int cbase = 0; cbase < g.ntypes; cbase += kRegChannels) {
    const int nchan = min(kRegChannels, g.ntypes - cbase);
    float acc0[kRegChannels], acc1[kRegChannels], acc2[kRegChannels];
#pragma unroll
    for (int c = 0; c < kRegChannels; ++c) acc0[c] = acc1[c] = acc2[c] = 0.f;

    for (int s0 = begin; s0 < end; s0 += kSuper) {
      const int send = min(end, s0 + kSuper);
      // ---- scan --------------------------------------------------------------
      int wcnt = 0;
      {
        const int wb = s0 + wave * kSeg, we = min(send, wb + kSeg);
        constexpr int U = 2;
        for (int a0 = wb; a0 < we; a0 += kWave * U) {
          float rr[U], cx[U], cy[U], cz[U];
#pragma unroll
          for (int u = 0; u < U; ++u) {
            const int a = min(a0 + u * kWave + lane, we - 1);
            rr[u] = radii[a];
            cx[u] = coords[3 * a];
            cy[u] = coords[3 * a + 1];
            cz[u] = coords[3 * a + 2];
          }
#pragma unroll
          for (int u = 0; u < U; ++u) {
            const int a = a0 + u * kWave + lane;
            const float reach = rr[u] * g.radius_scale * cull_mult;
            const bool p = (a < we) && box_distance2(cx[u], cy[u], cz[u], clx, cly, clz, chx, chy,
                                                     chz) <= reach * reach * kCullSlack;
            const unsigned long long m = __ballot(p);
            if (p) s_idx[wave][wcnt + __popcll(m & ((1ull << lane) - 1ull))] = (unsigned short)(a - s0);
            wcnt += __popcll(m);
          }
        }
      }
      if (lane == 0) s_wcount[wave] = wcnt;
      __syncthreads();
      int segstart[kColWaves + 1];
      segstart[0] = 0;
#pragma unroll
      for (int w = 0; w < kColWaves; ++w) segstart[w + 1] = segstart[w] + s_wcount[w];
      const int ncand = segstart[kColWaves];

      for (int c0 = 0; c0 < ncand; c0 += kRecChunk) {
        // ---- records -----------------------------------------------------------
        const int m = min(kRecChunk, ncand - c0);
        if (tid < m) {
          const int gi = c0 + tid;
          int w = 0;
#pragma unroll
          for (int k = 1; k < kColWaves; ++k) w += (gi >= segstart[k]) ? 1 : 0;
          const int a = s0 + s_idx[w][gi - segstart[w]];
          const float ax = coords[3 * a], ay = coords[3 * a + 1], az = coords[3 * a + 2];
          const float radius = radii[a];
          const float tf = floorf(type_index[a]) - (float)cbase;
          const bool typed = tf >= 0.f && tf < (float)nchan;
          float ar, ar2;
          {
#pragma clang fp contract(off)
            ar = radius * g.radius_scale;
            ar2 = ar * ar;
          }
          // an atom of another channel group (or an ignored one) can never hit
          const float w4 = typed ? (BINARY ? ar2 : 1.0f / ar2) : (BINARY ? -1.0f : INFINITY);
          s_rec[tid] = make_float4(ax, ay, az, w4);
          s_rectype[tid] = typed ? (unsigned char)(int)tf : 0;
          if (EXACT) {
            const uint3 cl = pack_clip(g, ox, oy, oz, ax, ay, az, radius);
            s_clip[tid] = make_uint4(cl.x, cl.y, cl.z, __float_as_uint(ar));
          }
        }
        __syncthreads();

        // ---- cull per 4x4x4 block, then splat ------------------------------------
#pragma unroll
        for (int blk = 0; blk < kBlocksPerWave; ++blk) {
          const int zb = z0 + (wave * kBlocksPerWave + blk) * 4;
          if (zb >= zend) continue;
          const float blz = grid_coord(oz, zb, g.resolution);
          const float bhz = grid_coord(oz, min(zb + 4, zend) - 1, g.resolution);
          const int vzi = zb + lz;
          const bool live = xy_live && vzi < zend;
          const float vz = grid_coord(oz, vzi, g.resolution);
          for (int r0 = 0; r0 < m; r0 += kWave) {
            const int i = r0 + lane;
            bool pass = false;
            float4 rec = make_float4(0.f, 0.f, 0.f, 0.f);
            if (i < m) {
              rec = s_rec[i];
              const float d2 = box_distance2(rec.x, rec.y, rec.z, clx, cly, blz, chx, chy, bhz);
              pass = BINARY ? (d2 <= rec.w * kCullSlack) : (d2 * rec.w <= frm2 * kCullSlack);
            }
            const unsigned long long bm = __ballot(pass);
            const int n = __popcll(bm);
            if (n == 0) continue;
            if (pass) {
              const int p = __popcll(bm & ((1ull << lane) - 1ull));
              s_mini[wave][p] = rec;
              s_minitype[wave][p] = s_rectype[i];
              if (EXACT) s_miniclip[wave][p] = s_clip[i];
            }
            const float4* mp = s_mini[wave];
            const unsigned char* tp = s_minitype[wave];
            auto body = [&](const float4& r, int tt, int it) {
              const int t = __builtin_amdgcn_readfirstlane(tt);
              bool inside = live;
              float ar = 0.f;
              if (EXACT) {
                const uint4 cl = s_miniclip[wave][it];
                inside = inside && inside_clip(vxi, vyi, vzi, make_uint3(cl.x, cl.y, cl.z));
                ar = __uint_as_float(cl.w);
              }
              float val = density<BINARY, EXACT>(g, vx - r.x, vy - r.y, vz - r.z, r.w, ar, frm2, grm2);
              if (!inside) val = 0.f;
              // binary occupancy stores 1 where any atom covers the voxel
              if (blk == 0) acc0[t] = BINARY ? fmaxf(acc0[t], val) : acc0[t] + val;
              else if (blk == 1) acc1[t] = BINARY ? fmaxf(acc1[t], val) : acc1[t] + val;
              else acc2[t] = BINARY ? fmaxf(acc2[t], val) : acc2[t] + val;
            };
            // software pipelined: the next record is in flight while this one is evaluated
            float4 cur = mp[0];
            int ct = tp[0];
            int it = 0;
            for (; it + 2 <= n; it += 2) {
              const float4 r1 = mp[it + 1];
              const int t1 = tp[it + 1];
              body(cur, ct, it);
              cur = mp[min(it + 2, kWave - 1)];
              ct = tp[it + 2];
              body(r1, t1, it + 1);
            }
            if (it < n) body(cur, ct, it);
          }
        }
        lds_barrier();
      }
    }

    // ---- store: four channels per round through a double-buffered LDS stage ------
    // fixed positions of this thread in the staged write-out (float4 granules)
    constexpr int kItems = kStageCh * 16 * (kSlabZ / 4);               // 768 per round
    constexpr int kPer = (kItems + kColThreads - 1) / kColThreads;     // 3
    int st_lds[kPer], st_chan[kPer], st_sp[kPer];
#pragma unroll
    for (int k = 0; k < kPer; ++k) {
      const int item = tid + k * kColThreads;
      const int j = item / 192, q = item % 192, row = q / 12, f4 = q % 12;
      const int gx = x0 + (row >> 2), gy = y0 + (row & 3), gz = z0 + f4 * 4;
      st_lds[k] = j * kPlane + row * kRowPad + f4 * 4;
      st_chan[k] = (gx < dim && gy < dim && gz < dim) ? j : -1;
      st_sp[k] = (gx * dim + gy) * dim + gz;
    }
#pragma unroll
    for (int r = 0; r < (kRegChannels + kStageCh - 1) / kStageCh; ++r) {
      if (r * kStageCh >= nchan) break;
      float* stage = s_stage + (r & 1) * (kStageCh * kPlane);
#pragma unroll
      for (int j = 0; j < kStageCh; ++j) {
        const int c = r * kStageCh + j;
        if (c < kRegChannels) {
          stage[j * kPlane + dump_off] = acc0[c];
          stage[j * kPlane + dump_off + 4] = acc1[c];
          stage[j * kPlane + dump_off + 8] = acc2[c];
        }
      }
      lds_barrier();
      float* ob = out_b + (size_t)(cbase + r * kStageCh) * chan_stride;
      const int nch = min(kStageCh, nchan - r * kStageCh);
#pragma unroll
      for (int k = 0; k < kPer; ++k) {
        if (st_chan[k] >= 0 && st_chan[k] < nch) {
          const v4f v = *reinterpret_cast<const v4f*>(stage + st_lds[k]);
          float* dst = ob + (size_t)st_chan[k] * chan_stride + st_sp[k];
          const int gz = z0 + ((tid + k * kColThreads) % 12) * 4;
          if (vec_store && gz + 3 < dim) {
            *reinterpret_cast<v4f*>(dst) = v;
          } else {
            dst[0] = v.x;
            if (gz + 1 < dim) dst[1] = v.y;
            if (gz + 2 < dim) dst[2] = v.z;
            if (gz + 3 < dim) dst[3] = v.w;
          }
        }
      }
    }
    lds_barrier();
  }
}

template <bool BINARY, bool EXACT>
hipError_t launch_one(const GridArg& g, const BatchArg& batch, int nbatch, const Vec3Arg& centers,
                      const float* coords, const float* type_index, const float* radii,
                      float* out, hipStream_t stream) {
  const int cols_per_side = (g.dim + kColXY - 1) / kColXY;
  const int slabs = (g.dim + kSlabZ - 1) / kSlabZ;
  const size_t chan_stride = (size_t)g.dim * g.dim * g.dim;
  const int vec_store = (g.dim % 4 == 0) && ((reinterpret_cast<uintptr_t>(out) & 15) == 0) &&
                        ((chan_stride * g.ntypes) % 4 == 0);
  hipLaunchKernelGGL((splat_index_kernel<BINARY, EXACT>),
                     dim3(cols_per_side * cols_per_side * slabs, nbatch), dim3(kColThreads), 0,
                     stream, g, batch, centers, coords, type_index, radii, out, cols_per_side,
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
