// Forward density splat for vector-typed atoms with per-atom radii, density mode
// (GridMaker::forward with a type vector, src/grid_maker.cpp:226-270).
//
// Every atom feeds every channel: out[c][v] = sum_a W[a][c] * D[a][v] with W the type vector of
// atom a and D its density at voxel v.  That is a matrix product, and the only dense contraction of
// the gridding path, so it runs on the matrix cores: v_mfma_f32_16x16x4f32 multiplies a
// 16-channel x 4-atom slice of W with a 4-atom x 16-voxel slice of D into a 16 x 16 tile of sums
// (all float32).  The VALU evaluates each density once; the 28 multiply-adds per atom and voxel of
// a plain loop are gone.
//
// Geometry, culling and write-out follow the column kernel of forward_index.hip: a workgroup (four
// waves) owns a group of three columns of 4 x 4 voxels in (x, y) over a slab of up to 48 voxels in z
// and takes them one after the other; the atoms that can reach the group are found by one scan and
// kept as indices, records (x, y, z, 1/ar^2, atom) are built 256 at a time, each wave culls them
// again per 4x4x4 block into a private list, and the sums leave through a double-buffered LDS stage
// as float4 pieces of whole z rows.  A wave keeps the 32 x 64 sums of each of its three blocks in
// eight 4-register tiles: two halves of the channels by the four x planes of the 4x4x4 voxels.
//
// Binary occupancy adds the weights themselves (density 1 where the atom covers the voxel, by the
// reference's exact float comparison) and is compared bit for bit with the CPU loop, which adds
// them in atom order.  v_mfma_f32_16x16x4f32 adds the four products of a step to the running sum
// one after the other, each rounded to float32 -- measured: every binary comparison of the test
// suite (sums of tens of weights in tens of thousands of voxels) is identical -- so the order of
// the list, ascending atoms, is the order of the sum.  Densities differ from the column kernel in
// the last bits only because dy^2 + dz^2 is shared by the four x planes here.
#include <type_traits>

#include "kernels.h"
#include "splat_common.h"

namespace mg {
namespace {

constexpr int kColXY = 4;
constexpr int kColsPerGroup = 3;
constexpr int kColWaves = 4;
constexpr int kColThreads = kColWaves * kWave;
constexpr int kBlocksPerWave = 3;
constexpr int kSlabZ = kColWaves * kBlocksPerWave * 4;   // 48
constexpr int kRowPad = 52;                      // staged z row, padded against bank conflicts
constexpr int kPlane = 16 * kRowPad;             // one staged channel: 16 rows
constexpr int kStageCh = 4;                      // channels staged per round
constexpr int kSuper = 4096;                     // atoms scanned per pass
constexpr int kSeg = kSuper / kColWaves;
constexpr int kRecChunk = 256;
constexpr int kChannels = 32;                    // channels per pass: the rows of a tile
constexpr int kEntryBytes = 80;                  // four records (16 B each) and their four atoms


__device__ __forceinline__ float uniform(float v) {
  return __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(v)));
}
__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

template <bool BINARY>
__global__ __launch_bounds__(kColThreads) __attribute__((amdgpu_waves_per_eu(3, 3))) void
splat_vector_mfma_kernel(
    GridArg g, BatchArg batch, Vec3Arg centers, const float* __restrict__ coords,
    const float* __restrict__ type_vector, const float* __restrict__ radii,
    float* __restrict__ out, int cols_per_side, int vec_store) {
  __shared__ unsigned short s_idx[kColWaves][kSeg];
  __shared__ int s_wcount[kColWaves];
  __shared__ float4 s_rec[kRecChunk];            // x, y, z, 1/ar^2
  __shared__ int s_recatom[kRecChunk];
  // wave-private list of a block's atoms, four per entry; spare entries because the loop reads
  // ahead
  __shared__ __align__(16) unsigned char s_mini[kColWaves][(kWave / 4 + 3) * kEntryBytes];
  __shared__ __align__(16) float s_stage[2 * kStageCh * kPlane];

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid >> 6;
  const int b = example_for_slot(batch, blockIdx.y, gridDim.y, lane);
  int begin, end;
  example_range(batch, b, begin, end);
  const float3 center = load3(centers, b);
  const float ox = uniform(center.x - g.half_dimension);
  const float oy = uniform(center.y - g.half_dimension);
  const float oz = uniform(center.z - g.half_dimension);
  const int dim = g.dim;
  const int ntypes = g.ntypes;

  const int groups_per_row = (cols_per_side + kColsPerGroup - 1) / kColsPerGroup;
  const int ngroups = cols_per_side * groups_per_row;
  const int slab = blockIdx.x / ngroups;
  const int grp = blockIdx.x - slab * ngroups;
  const int x0 = (grp / groups_per_row) * kColXY;
  const int gy0 = (grp % groups_per_row) * (kColXY * kColsPerGroup);
  const int z0 = slab * kSlabZ;
  const int zend = min(z0 + kSlabZ, dim);          // exclusive

  // a lane's place in the matrix tiles: voxel j (y, z) of a 16-voxel tile, atom `quad` of the four
  // of a step; tile t holds the voxels with x = t
  const int j = lane & 15, quad = lane >> 4;
  const int jy = j >> 2, jz = j & 3;
  float vx[4];
#pragma unroll
  for (int t = 0; t < 4; ++t)
    vx[t] = x0 + t < dim ? grid_coord(ox, x0 + t, g.resolution) : INFINITY;   // outside: unreachable

  const float clx = uniform(grid_coord(ox, x0, g.resolution));
  const float clz = uniform(grid_coord(oz, z0, g.resolution));
  const float chx = uniform(grid_coord(ox, min(x0 + kColXY, dim) - 1, g.resolution));
  const float chz = uniform(grid_coord(oz, zend - 1, g.resolution));
  const float gly = uniform(grid_coord(oy, gy0, g.resolution));
  const float ghy = uniform(grid_coord(oy, min(gy0 + kColXY * kColsPerGroup, dim) - 1, g.resolution));

  const float frm2 = uniform(g.frm * g.frm);
  const float grm2 = uniform(g.grm * g.grm);
  const size_t chan_stride = (size_t)dim * dim * dim;
  float* out_b = out + (size_t)b * ntypes * chan_stride;

  int segstart[kColWaves + 1];
  int ncand = 0;

  // ---- scan: atoms [s0, s1) against the group's box -> per-wave index segments --------------
  auto scan = [&](int s0, int s1) -> bool {
    const int quarter = (s1 - s0 + kColWaves - 1) / kColWaves;
    int wcnt = 0;
    const int wb = s0 + wave * quarter, we = min(s1, wb + quarter);
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
        const float reach = rr[u] * g.radius_scale * (BINARY ? 1.0f : g.frm);
        const bool p = (a < we) && box_distance2(cx[u], cy[u], cz[u], clx, gly, clz, chx, ghy,
                                                 chz) <= reach * reach * kCullSlack;
        const unsigned long long m = __ballot(p);
        const int pos = wcnt + __popcll(m & ((1ull << lane) - 1ull));
        if (p && pos < kSeg) s_idx[wave][pos] = (unsigned short)(a - s0);
        wcnt += __popcll(m);
      }
    }
    if (lane == 0) s_wcount[wave] = wcnt;
    __syncthreads();
    segstart[0] = 0;
    bool fits = true;
#pragma unroll
    for (int w = 0; w < kColWaves; ++w) {
      const int c = __builtin_amdgcn_readfirstlane(s_wcount[w]);
      fits = fits && c <= kSeg;
      segstart[w + 1] = segstart[w] + min(c, kSeg);
    }
    ncand = segstart[kColWaves];
    lds_barrier();   // every wave has read the counts before any of them scans again
    return fits;
  };

  // ---- records: candidates [c0, c0 + m) of the current scan -----------------------------------
  auto build_records = [&](int s0, int c0, int m) {
    if (tid < m) {
      const int gi = c0 + tid;
      int w = 0;
#pragma unroll
      for (int k = 1; k < kColWaves; ++k) w += (gi >= segstart[k]) ? 1 : 0;
      const int a = s0 + s_idx[w][min(gi - segstart[w], kSeg - 1)];
      float ar, ar2;
      {
#pragma clang fp contract(off)
        ar = radii[a] * g.radius_scale;
        ar2 = ar * ar;
      }
      s_rec[tid] = make_float4(coords[3 * a], coords[3 * a + 1], coords[3 * a + 2],
                               BINARY ? ar2 : 1.0f / ar2);
      s_recatom[tid] = a;
    }
    __syncthreads();
  };

  // whole example in one scan when its survivors fit; else passes of kSuper atoms per column
  bool one_pass = false;
  if (end - begin <= 65536) one_pass = scan(begin, end);
  const int pass_len = one_pass ? max(end - begin, 1) : kSuper;

  // fixed positions of this thread in the staged write-out (float4 granules)
  constexpr int kItems = kStageCh * 16 * (kSlabZ / 4);               // 768 per round
  constexpr int kPer = (kItems + kColThreads - 1) / kColThreads;     // 3

  for (int cbase = 0; cbase < ntypes; cbase += kChannels) {
    const int nchan = min(kChannels, ntypes - cbase);
    // this lane's two rows of the weight matrix: channels cbase + j and cbase + 16 + j of every
    // atom (a row past the last channel reads the last channel and is zeroed afterwards)
    const bool chan_live[2] = {j < nchan, 16 + j < nchan};
    const float* __restrict__ weights0 = type_vector + cbase + min(j, nchan - 1);
    const float* __restrict__ weights1 = type_vector + cbase + min(16 + j, nchan - 1);
    for (int col = 0; col < kColsPerGroup; ++col) {
      const int y0 = gy0 + col * kColXY;
      if (y0 >= dim) break;
      const float vy = grid_coord(oy, y0 + jy, g.resolution);
      const bool y_live = y0 + jy < dim;
      const float cly = uniform(grid_coord(oy, y0, g.resolution));
      const float chy = uniform(grid_coord(oy, min(y0 + kColXY, dim) - 1, g.resolution));

      v4f sums[kBlocksPerWave][4][2];            // [block][x plane][channel half]
#pragma unroll
      for (int blk = 0; blk < kBlocksPerWave; ++blk)
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
          for (int h = 0; h < 2; ++h) sums[blk][t][h] = v4f{0.f, 0.f, 0.f, 0.f};

      for (int s0 = begin; s0 < end; s0 += pass_len) {
        if (!one_pass) scan(s0, min(end, s0 + kSuper));
        for (int c0 = 0; c0 < ncand; c0 += kRecChunk) {
          const int m = min(kRecChunk, ncand - c0);
          build_records(s0, c0, m);
#pragma unroll
          for (int blk = 0; blk < kBlocksPerWave; ++blk) {
            const int zb = z0 + (wave * kBlocksPerWave + blk) * 4;
            if (zb >= zend) continue;
            const float blz = uniform(grid_coord(oz, zb, g.resolution));
            const float bhz = uniform(grid_coord(oz, min(zb + 4, zend) - 1, g.resolution));
            // a voxel outside the grid sits at infinity: no atom reaches it
            const float vz = (y_live && zb + jz < zend) ? grid_coord(oz, zb + jz, g.resolution)
                                                        : INFINITY;
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
              unsigned char* mine = s_mini[wave];
              if (pass) {
                const int p = __popcll(bm & ((1ull << lane) - 1ull));
                unsigned char* e = mine + (p >> 2) * kEntryBytes;
                *reinterpret_cast<float4*>(e + (p & 3) * 16) = rec;
                *reinterpret_cast<int*>(e + 64 + (p & 3) * 4) = s_recatom[i];
              }
              // one entry = four atoms = one step of the matrix product; the quarter wave that
              // holds atom `quad` reads its record and its two weights, every lane evaluates four
              // densities (its (y, z) in each of the four x planes)
              struct Step { float4 r; float w0, w1; bool have; };
              auto fetch = [&](int k) -> Step {
                const unsigned char* e = mine + k * kEntryBytes;
                Step s;
                s.r = *reinterpret_cast<const float4*>(e + quad * 16);
                const int atom = *reinterpret_cast<const int*>(e + 64 + quad * 4);
                s.have = 4 * k + quad < n;   // (past the list: an older atom or none)
                // Both weights are always loaded (from the example's first atom where there is
                // none) and masked only when they are used, an iteration later: the loads of
                // the next entry then stay in flight while this entry is evaluated.
                const size_t row = (size_t)(s.have ? atom : begin) * ntypes;
                s.w0 = weights0[row];
                s.w1 = weights1[row];
                return s;
              };
              const int steps = (n + 3) >> 2;
              Step cur = fetch(0);
              for (int k = 0; k < steps; ++k) {
                const Step nxt = fetch(k + 1);   // in flight while this entry is evaluated
                __builtin_amdgcn_sched_barrier(0);  // (keeps the loads up here)
                // a slot past the list has no reach at all, so its density is exactly zero (zero
                // weight alone would not do: a stale record can give an infinite density, and
                // 0 * inf is not a number)
                const float rw = cur.have ? cur.r.w : (BINARY ? -1.0f : INFINITY);
                const float w0 = (cur.have && chan_live[0]) ? cur.w0 : 0.f;
                const float w1 = (cur.have && chan_live[1]) ? cur.w1 : 0.f;
                const float dy = vy - cur.r.y, dz = vz - cur.r.z;
                const float dyz2 = dy * dy + dz * dz;
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                  const float dx = vx[t] - cur.r.x;
                  float d;
                  if (BINARY) {
                    // the reference's own float sequence ((dx^2 + dy^2) + dz^2) < ar^2
                    d = sq_distance_exact(dx, dy, dz) < rw ? 1.0f : 0.0f;
                  } else {
                    const float u = (dx * dx + dyz2) * rw;
                    const float gauss = __builtin_amdgcn_exp2f(u * kNeg2Log2e);
                    const float su = __builtin_amdgcn_sqrtf(u);
                    const float quadr = fmaxf(fmaf(g.A, u, fmaf(g.B, su, g.C)), 0.f);
                    d = (u <= grm2) ? gauss : quadr;
                    d = (u <= frm2) ? d : 0.f;
                  }
                  sums[blk][t][0] = __builtin_amdgcn_mfma_f32_16x16x4f32(w0, d, sums[blk][t][0], 0, 0, 0);
                  sums[blk][t][1] = __builtin_amdgcn_mfma_f32_16x16x4f32(w1, d, sums[blk][t][1], 0, 0, 0);
                }
                cur = nxt;
              }
            }
          }
          lds_barrier();   // records are rebuilt next round
        }
      }

      // ---- store: four channels per round through a double-buffered LDS stage ----
      int st_lds[kPer], st_chan[kPer], st_sp[kPer];
#pragma unroll
      for (int k = 0; k < kPer; ++k) {
        const int item = tid + k * kColThreads;
        const int jj = item / 192, q = item % 192, row = q / 12, f4 = q % 12;
        const int gx = x0 + (row >> 2), gy = y0 + (row & 3), gz = z0 + f4 * 4;
        st_lds[k] = jj * kPlane + row * kRowPad + f4 * 4;
        st_chan[k] = (gx < dim && gy < dim && gz < dim) ? jj : -1;
        st_sp[k] = (gx * dim + gy) * dim + gz;
      }
      auto store_round = [&](int r) {
        const float* stage = s_stage + (r & 1) * (kStageCh * kPlane);
        lds_barrier();
        float* ob = out_b + (size_t)(cbase + r * kStageCh) * chan_stride;
        const int nch = min(kStageCh, nchan - r * kStageCh);
#pragma unroll
        for (int k = 0; k < kPer; ++k) {
          if (st_chan[k] >= 0 && st_chan[k] < nch) {
            const v4f v = *reinterpret_cast<const v4f*>(stage + st_lds[k]);
            float* dst = ob + (size_t)st_chan[k] * chan_stride + st_sp[k];
            const int gz = z0 + ((tid + k * kColThreads) % 12) * 4;
            if ((vec_store & 1) && gz + 3 < dim) {
              // non-temporal: the grids are not read back soon, and the write-back of plain
              // stores runs on into the next launch (binary occupancy: 0.65 ms against 0.85 ms)
              __builtin_nontemporal_store(v, reinterpret_cast<v4f*>(dst));
            } else {
              dst[0] = v.x;
              if (gz + 1 < dim) dst[1] = v.y;
              if (gz + 2 < dim) dst[2] = v.z;
              if (gz + 3 < dim) dst[3] = v.w;
            }
          }
        }
      };
      // Register e of a tile holds channel 16 * h + 4 * quad + e of the lane's voxel, so channels
      // 4r .. 4r+3 are the four registers of the tiles with h = r / 4 in the lanes with
      // quad == r % 4.
      auto dump_round = [&](auto rc) {
        constexpr int r = decltype(rc)::value;
        if (quad == (r & 3)) {
          float* stage = s_stage + (r & 1) * (kStageCh * kPlane);
#pragma unroll
          for (int blk = 0; blk < kBlocksPerWave; ++blk)
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
              for (int e = 0; e < 4; ++e)
                stage[e * kPlane + (t * 4 + jy) * kRowPad + (wave * kBlocksPerWave + blk) * 4 + jz] =
                    sums[blk][t][r >> 2][e];
        }
      };
      auto round = [&](auto rc) {
        constexpr int r = decltype(rc)::value;
        if (nchan > r * kStageCh) {
          dump_round(rc);
          store_round(r);
        }
      };
      round(std::integral_constant<int, 0>{});
      round(std::integral_constant<int, 1>{});
      round(std::integral_constant<int, 2>{});
      round(std::integral_constant<int, 3>{});
      round(std::integral_constant<int, 4>{});
      round(std::integral_constant<int, 5>{});
      round(std::integral_constant<int, 6>{});
      round(std::integral_constant<int, 7>{});
      lds_barrier();
    }
  }
}

}  // namespace

hipError_t launch_forward_vector_mfma(const GridArg& g, const BatchArg& batch, int nbatch,
                                      const Vec3Arg& centers, const float* coords,
                                      const float* type_vector, const float* radii, float* out,
                                      bool binary, hipStream_t stream) {
  const int cols_per_side = (g.dim + kColXY - 1) / kColXY;
  const int slabs = (g.dim + kSlabZ - 1) / kSlabZ;
  const size_t chan_stride = (size_t)g.dim * g.dim * g.dim;
  const int vec_store = ((g.dim % 4 == 0) && ((reinterpret_cast<uintptr_t>(out) & 15) == 0) &&
                         ((chan_stride * g.ntypes) % 4 == 0)) ? 1 : 0;
  const int groups = cols_per_side * ((cols_per_side + kColsPerGroup - 1) / kColsPerGroup);
  if (binary)
    hipLaunchKernelGGL(splat_vector_mfma_kernel<true>, dim3(groups * slabs, nbatch),
                       dim3(kColThreads), 0, stream, g, batch, centers, coords, type_vector, radii,
                       out, cols_per_side, vec_store);
  else
    hipLaunchKernelGGL(splat_vector_mfma_kernel<false>, dim3(groups * slabs, nbatch),
                       dim3(kColThreads), 0, stream, g, batch, centers, coords, type_vector, radii,
                       out, cols_per_side, vec_store);
  return hipGetLastError();
}

}  // namespace mg
