// Forward density splat for vector-typed atoms with per-atom radii, density mode
// (GridMaker::forward with a type vector, src/grid_maker.cpp:226-270).
//
// Every atom feeds every channel: out[c][v] = sum_a W[a][c] * D[a][v] with W the type vector of
// atom a and D its density at voxel v.  That is a matrix product, and the only dense contraction of
// the gridding path: v_mfma_f32_16x16x4f32 multiplies a 16-channel x 4-atom slice of W with a
// 4-atom x 16-voxel slice of D into a 16 x 16 tile of sums (all float32).  The VALU evaluates
// each density once; the 28 multiply-adds per atom and voxel of a plain loop become two matrix
// instructions per four atoms and 64 voxels.  On this chip a float32 matrix instruction and VALU
// work do not overlap on a SIMD (a loop of eight such instructions and 64 independent v_fma_f32
// takes the sum of the two loops' times, with one, two or three waves on the SIMD), so the kernel
// is bound by the sum of the two, not by the larger.
//
// A workgroup (four waves) owns a group of three columns of 4 x 4 voxels in (x, y) over a slab of
// up to 48 voxels in z and takes the columns one after the other; a wave owns three 4x4x4 blocks
// of the column.  The atoms that can reach the group are found by one scan and kept as indices.
// For a column they are taken 256 at a time: the workgroup builds a row per atom in LDS -- its 32
// weights of the pass (zero past the last channel) and its record (x, y, z, 1/ar^2) -- each wave
// culls the rows against its three blocks in one pass (the x and y terms of the box distance are
// shared) into three lists of row offsets, and then walks each list four atoms a step.  The walk
// is software-pipelined two steps a trip: rows and list entries are read ahead, the densities of
// the next step are evaluated between the matrix instructions of this one.  A list ends in
// entries that point at a row of no atom (zero weights, unreachable record), so a short last
// step and the read-ahead need no masks.  A wave keeps the 32 x 64 sums of each of its three
// blocks in eight 4-register tiles: two halves of the channels by the four x planes of the block.
// The sums leave through an LDS stage, eight channels a round with every lane writing, as float4
// pieces of whole z rows.
//
// Binary occupancy adds the weights themselves (density 1 where the atom covers the voxel, by the
// reference's exact float comparison) and is compared bit for bit with the CPU loop, which adds
// them in atom order.  v_mfma_f32_16x16x4f32 adds the four products of a step to the running sum
// one after the other, each rounded to float32 -- measured: every binary comparison of the test
// suite (sums of tens of weights in up to 25 million voxels, full size included) is identical --
// so the order of the list, ascending atoms, is the order of the sum.  Gaussian densities share
// dy^2 + dz^2 between the four x planes and agree with the CPU loop to rounding.
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
constexpr int kStageCh = 4;                      // channel planes a pass of the write-out covers
constexpr int kPlaneS = kPlane + 4;              // stage plane stride: the four quads of a wave, which
                                                 // write planes 2 apart, then meet no bank twice over
constexpr int kSuper = 4096;                     // atoms scanned per pass
constexpr int kSeg = kSuper / kColWaves;
constexpr int kRecChunk = 256;
constexpr int kChannels = 32;                    // channels per pass: the rows of a tile
constexpr int kRowBytes = 144;                   // a chunk row: 32 weights, then x, y, z, 1/ar^2
constexpr int kStageBytes = 2 * kStageCh * kPlaneS * 4;
constexpr int kRowsBytes = (kRecChunk + 1) * kRowBytes;   // the last row belongs to no atom


__device__ __forceinline__ float uniform(float v) {
  return __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(v)));
}

template <bool BINARY>
__global__ __launch_bounds__(kColThreads) __attribute__((amdgpu_waves_per_eu(3, 3))) void
splat_vector_mfma_kernel(
    GridArg g, BatchArg batch, Vec3Arg centers, const float* __restrict__ coords,
    const float* __restrict__ type_vector, const float* __restrict__ radii,
    float* __restrict__ out, int cols_per_side, int vec_store, int vec_weights,
    const unsigned* __restrict__ slab_lists, const int* __restrict__ slab_counts, int list_stride) {
  __shared__ unsigned short s_idx[kColWaves][kSeg];
  __shared__ int s_wcount[kColWaves];
  // The rows of the current chunk of records while sums are formed, the stage of the write-out
  // afterwards.  A row holds the atom's weights for the 32 channels of the pass (zero past the
  // last channel) and its record; the row after the chunk has zero weights and a record at an
  // unreachable distance, and lies past the stage, which never overwrites it.
  __shared__ __align__(16) unsigned char s_rows[kRowsBytes > kStageBytes ? kRowsBytes : kStageBytes];
  // wave-private lists of the atoms of each block (byte offsets of their rows); spare entries
  // because the loop reads ahead
  __shared__ unsigned short s_mini[kColWaves][kBlocksPerWave][kRecChunk + 24];
  float* const s_stage = reinterpret_cast<float*>(s_rows);

  // Waves that scan, build rows, cull or write out issue ahead of waves that are in their steps:
  // those phases are short in instructions but long in waiting when they have to share a SIMD's
  // issue slots with streams of matrix instructions (measured: 1.31 -> 1.29 ms, binary 0.58 ->
  // 0.555 ms).
  __builtin_amdgcn_s_setprio(3);
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
    vx[t] = uniform(x0 + t < dim ? grid_coord(ox, x0 + t, g.resolution) : INFINITY);   // outside: unreachable

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

  // ---- scan: units [u0, u1) against the group's box -> per-wave index segments -----------------
  // A unit is an atom of the example (its index), or -- with lists: a launch before this one has
  // left, for every example and slab of four x planes, the atoms that can reach the slab's planes,
  // in atom order -- a position of this slab's list, about a fifth of the example.  A segment
  // entry is the atom's index relative to `base`, in 16 bits: the first atom of the window for
  // windows of atoms, the first atom of the example for lists (which the launcher therefore
  // builds for examples of up to 65,536 atoms only).  A window of kSuper units gives a wave at
  // most kSeg of them, so its segment cannot overflow.
  const unsigned* const my_list =
      slab_lists != nullptr ? slab_lists + ((size_t)b * cols_per_side + x0 / kColXY) * list_stride : nullptr;
  const int my_listed = slab_lists != nullptr ? slab_counts[b * cols_per_side + x0 / kColXY] : 0;
  const int unit_begin = my_list != nullptr ? 0 : begin, unit_end = my_list != nullptr ? my_listed : end;
  auto scan = [&](int u0, int u1, int base) -> bool {
    const int quarter = (u1 - u0 + kColWaves - 1) / kColWaves;
    int wcnt = 0;
    const int wb = u0 + wave * quarter, we = min(u1, wb + quarter);
    constexpr int U = 2;
    for (int i0 = wb; i0 < we; i0 += kWave * U) {
      float rr[U], cx[U], cy[U], cz[U];
      int at[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int i = min(i0 + u * kWave + lane, we - 1);
        at[u] = my_list != nullptr ? begin + (int)my_list[i] : i;
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int a = at[u];
        rr[u] = radii[a];
        cx[u] = coords[3 * a];
        cy[u] = coords[3 * a + 1];
        cz[u] = coords[3 * a + 2];
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int a = at[u];
        const float reach = rr[u] * g.radius_scale * (BINARY ? 1.0f : g.frm);
        const bool p = (i0 + u * kWave + lane < we) &&
                       box_distance2(cx[u], cy[u], cz[u], clx, gly, clz, chx, ghy, chz) <=
                           reach * reach * kCullSlack;
        const unsigned long long m = __ballot(p);
        const int pos = wcnt + __popcll(m & ((1ull << lane) - 1ull));
        if (p && pos < kSeg) s_idx[wave][pos] = (unsigned short)(a - base);
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
  auto build_records = [&](int s0, int c0, int m, int cbase, int nchan) {
    if (tid < m) {
      const int gi = c0 + tid;
      int w = 0;
#pragma unroll
      for (int k = 1; k < kColWaves; ++k) w += (gi >= segstart[k]) ? 1 : 0;
      const int a = s0 + s_idx[w][min(gi - segstart[w], kSeg - 1)];
      const float* __restrict__ wrow = type_vector + (size_t)a * ntypes + cbase;
      unsigned char* row = s_rows + tid * kRowBytes;
      // the weights, four quads in flight at a time (the sums of the column stay in registers)
#pragma unroll
      for (int q0 = 0; q0 < kChannels / 4; q0 += 4) {
        v4f wq[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int c = 4 * (q0 + u);
          if (vec_weights) {
            wq[u] = *reinterpret_cast<const v4f*>(wrow + min(c, nchan - 4));
          } else {
            wq[u].x = wrow[min(c, nchan - 1)];
            wq[u].y = wrow[min(c + 1, nchan - 1)];
            wq[u].z = wrow[min(c + 2, nchan - 1)];
            wq[u].w = wrow[min(c + 3, nchan - 1)];
          }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int c = 4 * (q0 + u);
          v4f v = wq[u];
          if (c >= nchan) v.x = 0.f;
          if (c + 1 >= nchan) v.y = 0.f;
          if (c + 2 >= nchan) v.z = 0.f;
          if (c + 3 >= nchan) v.w = 0.f;
          *reinterpret_cast<v4f*>(row + 4 * c) = v;
        }
      }
      float ar, ar2;
      {
#pragma clang fp contract(off)
        ar = radii[a] * g.radius_scale;
        ar2 = ar * ar;
      }
      const v4f rec = {coords[3 * a], coords[3 * a + 1], coords[3 * a + 2], BINARY ? ar2 : 1.0f / ar2};
      *reinterpret_cast<v4f*>(row + 4 * kChannels) = rec;
    }
    __syncthreads();
  };

  // the row of no atom: zero weights, and a record no voxel is within reach of (its squared
  // distance overflows to infinity, which passes neither comparison)
  if (tid < kRowBytes / 4) {
    float v = 0.f;
    if (tid >= kChannels) v = tid < kChannels + 3 ? 1e30f : (BINARY ? -1.0f : 1.0f);
    reinterpret_cast<float*>(s_rows + kRecChunk * kRowBytes)[tid] = v;
  }
  // whole example in one scan when its survivors fit; else passes of kSuper atoms per column
  bool one_pass = false;
  if (end - begin <= 65536) one_pass = scan(unit_begin, unit_end, begin);
  const int pass_len = one_pass ? max(unit_end - unit_begin, 1) : kSuper;

  // fixed positions of this thread in the staged write-out (float4 granules)
  constexpr int kItems = kStageCh * 16 * (kSlabZ / 4);               // 768 per round
  constexpr int kPer = (kItems + kColThreads - 1) / kColThreads;     // 3

  for (int cbase = 0; cbase < ntypes; cbase += kChannels) {
    const int nchan = min(kChannels, ntypes - cbase);
    // (a lane's two rows of the weight matrix are channels cbase + j and cbase + 16 + j)
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

      for (int u0 = unit_begin; u0 < unit_end; u0 += pass_len) {
        const int s0 = my_list != nullptr || one_pass ? begin : u0;   // what segment entries count from
        if (!one_pass) scan(u0, min(unit_end, u0 + kSuper), s0);
        for (int c0 = 0; c0 < ncand; c0 += kRecChunk) {
          const int m = min(kRecChunk, ncand - c0);
          build_records(s0, c0, m, cbase, nchan);
          // one pass over the chunk's records finds, for each of the wave's blocks, the atoms
          // that can reach it (the x and y terms of the box distance are shared); each list
          // ends in rows of no atom, because the last step may be short and the loop reads one
          // step ahead
          int nlist[kBlocksPerWave];
#pragma unroll
          for (int blk = 0; blk < kBlocksPerWave; ++blk) nlist[blk] = 0;
          for (int r0 = 0; r0 < m; r0 += kWave) {
            const int i = min(r0 + lane, m - 1);
            const float4 rec = *reinterpret_cast<const float4*>(s_rows + i * kRowBytes + 4 * kChannels);
            const float ex = fmaxf(fmaxf(clx - rec.x, rec.x - chx), 0.f);
            const float ey = fmaxf(fmaxf(cly - rec.y, rec.y - chy), 0.f);
            const float exy = ex * ex + ey * ey;
#pragma unroll
            for (int blk = 0; blk < kBlocksPerWave; ++blk) {
              const int zb = z0 + (wave * kBlocksPerWave + blk) * 4;
              const float blz = uniform(grid_coord(oz, zb, g.resolution));
              const float bhz = uniform(grid_coord(oz, min(zb + 4, zend) - 1, g.resolution));
              const float ez = fmaxf(fmaxf(blz - rec.z, rec.z - bhz), 0.f);
              const float d2 = exy + ez * ez;
              const bool pass = (r0 + lane < m) && (zb < zend) &&
                                (BINARY ? (d2 <= rec.w * kCullSlack) : (d2 * rec.w <= frm2 * kCullSlack));
              const unsigned long long bm = __ballot(pass);
              if (pass)
                s_mini[wave][blk][nlist[blk] + __popcll(bm & ((1ull << lane) - 1ull))] =
                    (unsigned short)(i * kRowBytes);
              nlist[blk] += __popcll(bm);
            }
          }
#pragma unroll
          for (int blk = 0; blk < kBlocksPerWave; ++blk)
            if (lane < 24) s_mini[wave][blk][nlist[blk] + lane] = (unsigned short)(kRecChunk * kRowBytes);

          wave_lds_fence();                    // the wave's lists are complete
          __builtin_amdgcn_s_setprio(0);
#pragma unroll
          for (int blk = 0; blk < kBlocksPerWave; ++blk) {
            const int n = nlist[blk];
            if (n == 0) continue;
            const int zb = z0 + (wave * kBlocksPerWave + blk) * 4;
            // a voxel outside the grid sits at infinity: no atom reaches it
            const float vz = (y_live && zb + jz < zend) ? grid_coord(oz, zb + jz, g.resolution)
                                                        : INFINITY;
            const unsigned short* mine = s_mini[wave][blk];
            // four atoms = one step of the matrix product; the quarter wave that holds atom
            // `quad` reads its record and its two weights, every lane evaluates four densities
            // (its (y, z) in each of the four x planes)
            struct Step { float4 r; float w0, w1; };
            auto fetch_row = [&](unsigned off) -> Step {
              const unsigned char* row = s_rows + off;
              Step s;
              s.r = *reinterpret_cast<const float4*>(row + 4 * kChannels);
              s.w0 = *reinterpret_cast<const float*>(row + 4 * j);
              s.w1 = *reinterpret_cast<const float*>(row + 4 * (16 + j));
              return s;
            };
            // the four densities of a lane for one atom: its (y, z) in each of the four x planes
            auto densities = [&](const float4& r, float (&d)[4]) {
              const float dy = vy - r.y, dz = vz - r.z;
              const float dyz2 = dy * dy + dz * dz;
#pragma unroll
              for (int t = 0; t < 4; ++t) {
                const float dx = vx[t] - r.x;
                if (BINARY) {
                  // the reference's own float sequence ((dx^2 + dy^2) + dz^2) < ar^2
                  d[t] = sq_distance_exact(dx, dy, dz) < r.w ? 1.0f : 0.0f;
                } else {
                  const float u = (dx * dx + dyz2) * r.w;
                  const float gauss = __builtin_amdgcn_exp2f(u * kNeg2Log2e);
                  const float su = __builtin_amdgcn_sqrtf(u);
                  const float quadr = fmaxf(fmaf(g.A, u, fmaf(g.B, su, g.C)), 0.f);
                  const float core = (u <= grm2) ? gauss : quadr;
                  d[t] = (u <= frm2) ? core : 0.f;
                }
              }
            };
            auto multiply = [&](const Step& s, const float (&d)[4]) {
#pragma unroll
              for (int t = 0; t < 4; ++t) {
                sums[blk][t][0] = __builtin_amdgcn_mfma_f32_16x16x4f32(s.w0, d[t], sums[blk][t][0], 0, 0, 0);
                sums[blk][t][1] = __builtin_amdgcn_mfma_f32_16x16x4f32(s.w1, d[t], sums[blk][t][1], 0, 0, 0);
              }
            };
            // Two steps per trip, software-pipelined: while the matrix cores multiply the
            // densities of one step, the VALU evaluates those of the next and the rows of the
            // step after that are on their way from LDS.  The rows of no atom at the end of the
            // list make a step past the last atom add nothing.
            const int trips = (n + 7) >> 3;
            Step a = fetch_row(mine[quad]);
            Step b = fetch_row(mine[4 + quad]);
            unsigned oc = mine[8 + quad], oe = mine[12 + quad];   // list entries, a trip ahead
            float da[4], db[4];
            densities(a.r, da);
            for (int k = 0; k < 2 * trips; k += 2) {
              const Step c = fetch_row(oc);
              const Step e = fetch_row(oe);
              oc = mine[4 * (k + 4) + quad];
              oe = mine[4 * (k + 5) + quad];
              multiply(a, da);
              densities(b.r, db);
              multiply(b, db);
              densities(c.r, da);
              a = c;
              b = e;
            }
          }
          __builtin_amdgcn_s_setprio(3);
          lds_barrier();   // records are rebuilt next round
        }
      }

      // ---- store: eight channels per round through the LDS stage ----
      // Register e of a tile holds channel 16 * h + 4 * quad + e of the lane's voxel.  A round
      // takes the registers e = 2p and 2p + 1 of the tiles of one h: every lane writes two
      // channels, plane 2 * quad + (e & 1) of the stage holds channel
      // 16 * h + 4 * quad + 2 * p + (e & 1).
      // (worked out here, after the steps, and not once before them, where these nine values
      // would sit in scratch memory for the whole column)
      int st_lds[kPer], st_slot[kPer], st_sp[kPer];
      int tid_now = tid;
      compute_here(tid_now);
#pragma unroll
      for (int k = 0; k < kPer; ++k) {
        const int item = tid_now + k * kColThreads;
        const int jj = item / 192, q = item % 192, row = q / 12, f4 = q % 12;
        const int gx = x0 + (row >> 2), gy = y0 + (row & 3), gz = z0 + f4 * 4;
        st_lds[k] = jj * kPlaneS + row * kRowPad + f4 * 4;
        st_slot[k] = (gx < dim && gy < dim && gz < dim) ? jj : -1;
        st_sp[k] = (gx * dim + gy) * dim + gz;
      }
      auto store_round = [&](int h, int p) {
        lds_barrier();
        float* ob = out_b + (size_t)cbase * chan_stride;
#pragma unroll
        for (int half = 0; half < 2; ++half) {
#pragma unroll
          for (int k = 0; k < kPer; ++k) {
            const int slot = st_slot[k] + 4 * half;
            const int ch = 16 * h + 4 * (slot >> 1) + 2 * p + (slot & 1);
            if (st_slot[k] >= 0 && ch < nchan) {
              const v4f v = *reinterpret_cast<const v4f*>(s_stage + st_lds[k] + 4 * half * kPlaneS);
              float* dst = ob + (size_t)ch * chan_stride + st_sp[k];
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
        }
      };
      auto dump_round = [&](auto hc, auto pc) {
        constexpr int h = decltype(hc)::value, p = decltype(pc)::value;
        lds_barrier();   // the stage (or the chunk's rows) has been read
#pragma unroll
        for (int blk = 0; blk < kBlocksPerWave; ++blk)
#pragma unroll
          for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int ee = 0; ee < 2; ++ee)
              s_stage[(2 * quad + ee) * kPlaneS + (t * 4 + jy) * kRowPad +
                      (wave * kBlocksPerWave + blk) * 4 + jz] = sums[blk][t][h][2 * p + ee];
      };
      auto round = [&](auto hc, auto pc) {
        constexpr int h = decltype(hc)::value, p = decltype(pc)::value;
        if (nchan > 16 * h) {
          dump_round(hc, pc);
          store_round(h, p);
        }
      };
      round(std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{});
      round(std::integral_constant<int, 0>{}, std::integral_constant<int, 1>{});
      round(std::integral_constant<int, 1>{}, std::integral_constant<int, 0>{});
      round(std::integral_constant<int, 1>{}, std::integral_constant<int, 1>{});
      lds_barrier();
    }
  }
}

// The launch before the splat: for every example and slab of four x planes, the atoms whose reach
// (their final radius; binary: their radius) comes to the slab's planes, as indices relative to the
// example's first atom, in ascending order.  The test is the x term of the splat kernel's own box
// test with the same floats, so the list holds every atom that kernel would have found.
constexpr int kListThreads = 512;
constexpr int kListWaves = kListThreads / kWave;
template <bool BINARY>
__global__ __launch_bounds__(kListThreads) void slab_list_kernel(
    GridArg g, BatchArg batch, Vec3Arg centers, const float* __restrict__ coords,
    const float* __restrict__ radii, unsigned* __restrict__ slab_lists,
    int* __restrict__ slab_counts, int list_stride) {
  __shared__ int s_wave_count[kListWaves];
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
  const int xs = blockIdx.x, b = blockIdx.y, nxs = gridDim.x;
  int begin, end;
  example_range(batch, b, begin, end);
  const float ox = load3(centers, b).x - g.half_dimension;
  const float clx = grid_coord(ox, xs * kColXY, g.resolution);
  const float chx = grid_coord(ox, min(xs * kColXY + kColXY, g.dim) - 1, g.resolution);
  unsigned* const list = slab_lists + ((size_t)b * nxs + xs) * list_stride;
  int listed = 0;
  for (int a0 = begin; a0 < end; a0 += kListThreads) {
    const int a = a0 + tid;
    bool p = false;
    if (a < end) {
      const float x = coords[3 * a];
      const float reach = radii[a] * g.radius_scale * (BINARY ? 1.0f : g.frm);
      const float ex = fmaxf(fmaxf(clx - x, x - chx), 0.f);
      p = sq_distance_exact(ex, 0.f, 0.f) <= reach * reach * kCullSlack;
    }
    const unsigned long long m = __ballot(p);
    if (lane == 0) s_wave_count[wave] = __popcll(m);
    __syncthreads();
    int before = 0, all = 0;
#pragma unroll
    for (int w = 0; w < kListWaves; ++w) {
      const int c = s_wave_count[w];
      before += w < wave ? c : 0;
      all += c;
    }
    const int pos = listed + before + __popcll(m & ((1ull << lane) - 1ull));
    if (p && pos < list_stride) list[pos] = (unsigned)(a - begin);
    listed += all;
    __syncthreads();
  }
  if (tid == 0) slab_counts[b * nxs + xs] = min(listed, list_stride);
}

}  // namespace

size_t forward_vector_workspace_bytes(int nbatch, int atoms_per_example, int dim) {
  const size_t nxs = (size_t)((dim + kColXY - 1) / kColXY);
  return ((nbatch * nxs * sizeof(int) + 255) & ~(size_t)255) +
         (size_t)nbatch * nxs * (size_t)atoms_per_example * sizeof(unsigned);
}

hipError_t launch_forward_vector_mfma(const GridArg& g, const BatchArg& batch, int nbatch,
                                      const Vec3Arg& centers, const float* coords,
                                      const float* type_vector, const float* radii, float* out,
                                      bool binary, void* workspace, size_t workspace_bytes,
                                      hipStream_t stream) {
  const int cols_per_side = (g.dim + kColXY - 1) / kColXY;
  // per-slab atom lists, when the caller has brought the memory for them and the example has atoms
  unsigned* lists = nullptr;
  int* counts = nullptr;
  const int list_stride = batch.per_example;
  if (workspace != nullptr && list_stride > 0 && list_stride <= 65536 &&
      workspace_bytes >= forward_vector_workspace_bytes(nbatch, list_stride, g.dim)) {
    counts = static_cast<int*>(workspace);
    lists = reinterpret_cast<unsigned*>(static_cast<unsigned char*>(workspace) +
                                        (((size_t)nbatch * cols_per_side * sizeof(int) + 255) & ~(size_t)255));
    if (binary)
      hipLaunchKernelGGL(slab_list_kernel<true>, dim3(cols_per_side, nbatch), dim3(kListThreads), 0,
                         stream, g, batch, centers, coords, radii, lists, counts, list_stride);
    else
      hipLaunchKernelGGL(slab_list_kernel<false>, dim3(cols_per_side, nbatch), dim3(kListThreads), 0,
                         stream, g, batch, centers, coords, radii, lists, counts, list_stride);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
  }
  const int slabs = (g.dim + kSlabZ - 1) / kSlabZ;
  const size_t chan_stride = (size_t)g.dim * g.dim * g.dim;
  const int vec_store = ((g.dim % 4 == 0) && ((reinterpret_cast<uintptr_t>(out) & 15) == 0) &&
                         ((chan_stride * g.ntypes) % 4 == 0)) ? 1 : 0;
  const int groups = cols_per_side * ((cols_per_side + kColsPerGroup - 1) / kColsPerGroup);
  // weight rows can be read four channels at a time
  const int vec_weights = ((g.ntypes % 4 == 0) && ((reinterpret_cast<uintptr_t>(type_vector) & 15) == 0)) ? 1 : 0;
  if (binary)
    hipLaunchKernelGGL(splat_vector_mfma_kernel<true>, dim3(groups * slabs, nbatch),
                       dim3(kColThreads), 0, stream, g, batch, centers, coords, type_vector, radii,
                       out, cols_per_side, vec_store, vec_weights, lists, counts, list_stride);
  else
    hipLaunchKernelGGL(splat_vector_mfma_kernel<false>, dim3(groups * slabs, nbatch),
                       dim3(kColThreads), 0, stream, g, batch, centers, coords, type_vector, radii,
                       out, cols_per_side, vec_store, vec_weights, lists, counts, list_stride);
  return hipGetLastError();
}

}  // namespace mg
