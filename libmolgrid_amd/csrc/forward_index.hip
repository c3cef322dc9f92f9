// Forward density splat on gfx950: index-typed atoms, and vector-typed atoms with per-atom radii.
//
// One workgroup of four waves works through three neighbouring columns of the grid, one after the
// other; a column is 4 x 4 voxels in (x, y) and up to 48 voxels along z, for every channel.  The
// atom scan (and, in the common case, the record building) is done once for the three columns.
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
// loops (src/grid_maker.cpp:170-211, 226-270).
//
// Vector types (VEC): every atom feeds all channels, so the splat step multiplies the atom's
// density into all 28 register sums with the atom's weights, which are read through
// wave-uniform (scalar) loads; binary mode adds the bare weight, in atom order -> bit exact.
#include <cstdlib>

#include "kernels.h"
#include "splat_common.h"

namespace mg {

namespace {

constexpr int kColXY = 4;                        // column is 4 x 4 voxels in x, y
constexpr int kBlocksPerWave = 3;                // 4x4x4 blocks per wave
constexpr int kColWaves = 4;
constexpr int kColsPerGroup = 3;                // columns (consecutive in y) sharing one atom scan
constexpr int kColThreads = kColWaves * kWave;   // 256
constexpr int kSlabZ = kColWaves * kBlocksPerWave * 4;  // 48 voxels of z per workgroup
constexpr int kRegChannels = 28;                 // channel sums kept in registers per voxel
constexpr int kRowPad = 52;                      // staged z row, padded against bank conflicts
constexpr int kPlane = 16 * kRowPad;             // one staged channel: 16 rows
constexpr int kStageCh = 4;                      // channels staged per round
constexpr int kSuper = 4096;                     // atoms scanned per pass
constexpr int kSeg = kSuper / kColWaves;         // per wave
constexpr int kRecChunk = 256;
constexpr int kPairBytes = 48;                   // two records and their tags in a block's list

// A float that is the same in every lane, moved to a scalar register so that it does not occupy
// a vector register for the whole kernel.
__device__ __forceinline__ float uniform(float v) {
  return __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(v)));
}

// The channel sums -- 28 per voxel, three voxels (blocks) per lane -- are kept in registers that
// the compiler does not know about: it is limited to v0 .. v(MG_ACC_BASE-1) by the kernel's
// amdgpu_num_vgpr attribute, and the 84 registers from v(MG_ACC_BASE) on are touched only by the
// asm statements below, through the scalar register index (s_set_gpr_idx).  One indexed VALU
// instruction adds a density to the sum of (block, channel); with a C array the compiler spends
// three moves and, for arrays that are not a register-tuple size, copies of the whole array.
// The build checks the generated code: no compiler-allocated register may reach the reserved range.
#define MG_ACC_BASE 84
#define MG_ACC_TOP "v167"
constexpr int kAccRegs = kBlocksPerWave * kRegChannels;
static_assert(MG_ACC_BASE + kAccRegs - 1 == 167, "MG_ACC_TOP names the last reserved register");

// sum[idx] (+)= val; idx is wave-uniform
template <bool BINARY>
__device__ __forceinline__ void acc_add(int idx, float val) {
  if (BINARY)
    asm volatile("s_set_gpr_idx_on %1, gpr_idx(SRC0,DST)\n\tv_max_f32 v[%2], v[%2], %0\n\ts_set_gpr_idx_off"
                 :: "v"(val), "s"(idx), "n"(MG_ACC_BASE) : MG_ACC_TOP);
  else
    asm volatile("s_set_gpr_idx_on %1, gpr_idx(SRC0,DST)\n\tv_add_f32 v[%2], v[%2], %0\n\ts_set_gpr_idx_off"
                 :: "v"(val), "s"(idx), "n"(MG_ACC_BASE) : MG_ACC_TOP);
}
// all sums = 0
#define MG_XSTR2(x) #x
#define MG_XSTR(x) MG_XSTR2(x)
#define MG_Z1(e) "v_mov_b32 v[" MG_XSTR(MG_ACC_BASE) "+" #e "], 0\n\t"
#define MG_Z4(e) MG_Z1(e+0) MG_Z1(e+1) MG_Z1(e+2) MG_Z1(e+3)
#define MG_Z28(e) MG_Z4(e+0) MG_Z4(e+4) MG_Z4(e+8) MG_Z4(e+12) MG_Z4(e+16) MG_Z4(e+20) MG_Z4(e+24)
__device__ __forceinline__ void acc_zero_all() {
  static_assert(kAccRegs == 84, "the list below clears 3 x 28 registers");
  asm volatile(MG_Z28(0) MG_Z28(28) MG_Z28(56) "s_nop 0" ::: MG_ACC_TOP);
}
// Channels 4R .. 4R+3 of the lane's three voxels -> the LDS stage.  `a0`, `a1`, `a2` are the LDS
// byte addresses of the three voxels in plane 0 of stage buffer 0; planes are 13 x 256 bytes
// apart and the two stage buffers 52 x 256 bytes, which the 256-byte-granular offsets of
// ds_write2st64_b32 reach, so one instruction writes two channels.
template <int R>
__device__ __forceinline__ void acc_dump_round(unsigned a0, unsigned a1, unsigned a2) {
  static_assert(kPlane * 4 == 13 * 256 && kStageCh == 4, "offsets below");
  constexpr int buf = (R & 1) * 52;
  asm volatile("ds_write2st64_b32 %0, v[%3], v[%3+1] offset0:%4 offset1:%5\n\t"
               "ds_write2st64_b32 %0, v[%3+2], v[%3+3] offset0:%6 offset1:%7\n\t"
               "ds_write2st64_b32 %1, v[%3+28], v[%3+29] offset0:%4 offset1:%5\n\t"
               "ds_write2st64_b32 %1, v[%3+30], v[%3+31] offset0:%6 offset1:%7\n\t"
               "ds_write2st64_b32 %2, v[%3+56], v[%3+57] offset0:%4 offset1:%5\n\t"
               "ds_write2st64_b32 %2, v[%3+58], v[%3+59] offset0:%6 offset1:%7"
               :: "v"(a0), "v"(a1), "v"(a2), "n"(MG_ACC_BASE + 4 * R), "n"(buf), "n"(buf + 13),
                  "n"(buf + 26), "n"(buf + 39)
               : "memory", MG_ACC_TOP);
}

// sums[first + c] += val * w[c] for seven channels starting at the compile-time channel C0;
// first (= block * 28) is wave-uniform, the weights are scalars
template <int C0>
__device__ __forceinline__ void acc_fma7(int first, float val, float w0, float w1, float w2, float w3,
                                         float w4, float w5, float w6) {
  asm volatile("s_set_gpr_idx_on %1, gpr_idx(SRC2,DST)\n\t"
               "v_fma_f32 v[%9], %2, %0, v[%9]\n\t"
               "v_fma_f32 v[%10], %3, %0, v[%10]\n\t"
               "v_fma_f32 v[%11], %4, %0, v[%11]\n\t"
               "v_fma_f32 v[%12], %5, %0, v[%12]\n\t"
               "v_fma_f32 v[%13], %6, %0, v[%13]\n\t"
               "v_fma_f32 v[%14], %7, %0, v[%14]\n\t"
               "v_fma_f32 v[%15], %8, %0, v[%15]\n\t"
               "s_set_gpr_idx_off"
               :: "v"(val), "s"(first), "s"(w0), "s"(w1), "s"(w2), "s"(w3), "s"(w4), "s"(w5), "s"(w6),
                  "n"(MG_ACC_BASE + C0), "n"(MG_ACC_BASE + C0 + 1), "n"(MG_ACC_BASE + C0 + 2),
                  "n"(MG_ACC_BASE + C0 + 3), "n"(MG_ACC_BASE + C0 + 4), "n"(MG_ACC_BASE + C0 + 5),
                  "n"(MG_ACC_BASE + C0 + 6)
               : MG_ACC_TOP);
}

// byte address of a __shared__ object inside the workgroup's LDS
__device__ __forceinline__ unsigned lds_address(const void* p) {
  return (unsigned)(unsigned long)(const __attribute__((address_space(3))) void*)p;
}

// LDS-only barrier: outstanding global stores are not waited for.
__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// `types` is type_index [n] (VEC = false) or type_vector [n, ntypes] (VEC = true)
template <bool BINARY, bool EXACT, bool VEC>
__global__ __launch_bounds__(kColThreads) void splat_column_kernel(
    GridArg g, BatchArg batch, Vec3Arg centers, const float* __restrict__ coords,
    const float* __restrict__ types, const float* __restrict__ radii,
    float* __restrict__ out, int cols_per_side, int vec_store) {
  __shared__ unsigned short s_idx[kColWaves][kSeg];
  __shared__ int s_wcount[kColWaves];
  __shared__ float4 s_rec[kRecChunk];            // x, y, z, (ar^2 | 1/ar^2)
  __shared__ unsigned char s_rectype[VEC ? 1 : kRecChunk];   // channel of the record (index types)
  __shared__ int s_recatom[VEC ? kRecChunk : 1];             // atom of the record (vector types)
  __shared__ uint4 s_clip[EXACT ? kRecChunk : 1];  // index box + ar, EXACT only
  // wave-private list of a block's atoms, two per 48-byte entry: records at +0 and +16, then
  // their channels (two bytes at +32) or atom numbers (two ints at +32, VEC); two spare entries
  // because the splat loop reads ahead
  __shared__ __align__(16) unsigned char s_mini[kColWaves][(kWave / 2 + 2) * kPairBytes];
  __shared__ uint4 s_miniclip[EXACT ? kColWaves : 1][EXACT ? kWave : 1];
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

  // which row of columns / z slab this workgroup owns: kColsPerGroup columns, consecutive in y
  const int groups_per_row = (cols_per_side + kColsPerGroup - 1) / kColsPerGroup;
  const int ngroups = cols_per_side * groups_per_row;
  const int slab = blockIdx.x / ngroups;
  const int grp = blockIdx.x - slab * ngroups;
  const int x0 = (grp / groups_per_row) * kColXY;
  const int gy0 = (grp % groups_per_row) * (kColXY * kColsPerGroup);
  const int z0 = slab * kSlabZ;
  const int zend = min(z0 + kSlabZ, dim);          // exclusive

  const int lx = lane >> 4, ly = (lane >> 2) & 3, lz = lane & 3;
  const int vxi = x0 + lx;
  const float vx = grid_coord(ox, vxi, g.resolution);
  // box of the whole group (first/last voxel centre inside the grid)
  const float clx = uniform(grid_coord(ox, x0, g.resolution));
  const float clz = uniform(grid_coord(oz, z0, g.resolution));
  const float chx = uniform(grid_coord(ox, min(x0 + kColXY, dim) - 1, g.resolution));
  const float chz = uniform(grid_coord(oz, zend - 1, g.resolution));
  const float gly = uniform(grid_coord(oy, gy0, g.resolution));
  const float ghy = uniform(grid_coord(oy, min(gy0 + kColXY * kColsPerGroup, dim) - 1, g.resolution));

  float quad_c = g.C;                       // constant term of the quadratic tail, kept in a
  asm volatile("" : "+v"(quad_c));          // vector register (an fma takes one scalar operand)
  const float frm2 = uniform(g.frm * g.frm);
  const float grm2 = uniform(g.grm * g.grm);
  const float cull_mult = BINARY ? 1.0f : g.frm;  // support radius / ar
  const size_t chan_stride = (size_t)dim * dim * dim;
  float* out_b = out + (size_t)b * g.ntypes * chan_stride;

  const int dump_off = lx * (4 * kRowPad) + ly * kRowPad + wave * kBlocksPerWave * 4 + lz;

  int segstart[kColWaves + 1];
  int ncand = 0;

  // ---- scan: atoms [s0, s1) against the group's box -> per-wave index segments --------------
  // Each wave takes a contiguous quarter of the range and keeps up to kSeg survivors (offsets
  // from s0 as 16-bit values, so s1 - s0 <= 65536).  Returns false if a segment overflowed.
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
        const float reach = rr[u] * g.radius_scale * cull_mult;
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
      const int c = __builtin_amdgcn_readfirstlane(s_wcount[w]);  // keep in SGPRs
      fits = fits && c <= kSeg;
      segstart[w + 1] = segstart[w] + c;
    }
    ncand = segstart[kColWaves];
    lds_barrier();   // every wave has read the counts before any of them scans again
    return fits;
  };

  // ---- records: candidates [c0, c0 + m) of the current scan -> 16-byte LDS records -----------
  auto build_records = [&](int s0, int c0, int m, int cbase, int nchan) {
    if (tid < m) {
      const int gi = c0 + tid;
      int w = 0;
#pragma unroll
      for (int k = 1; k < kColWaves; ++k) w += (gi >= segstart[k]) ? 1 : 0;
      const int a = s0 + s_idx[w][gi - segstart[w]];
      const float ax = coords[3 * a], ay = coords[3 * a + 1], az = coords[3 * a + 2];
      const float radius = radii[a];
      const float tf = VEC ? 0.f : floorf(types[a]) - (float)cbase;
      const bool typed = VEC || (tf >= 0.f && tf < (float)nchan);
      float ar, ar2;
      {
#pragma clang fp contract(off)
        ar = radius * g.radius_scale;
        ar2 = ar * ar;
      }
      // an atom of another channel group (or an ignored one) can never hit
      const float w4 = typed ? (BINARY ? ar2 : 1.0f / ar2) : (BINARY ? -1.0f : INFINITY);
      s_rec[tid] = make_float4(ax, ay, az, w4);
      if (VEC) s_recatom[tid] = a;
      else s_rectype[tid] = typed ? (unsigned char)(int)tf : 0;
      if (EXACT) {
        const uint3 cl = pack_clip(g, ox, oy, oz, ax, ay, az, radius);
        s_clip[tid] = make_uint4(cl.x, cl.y, cl.z, __float_as_uint(ar));
      }
    }
    __syncthreads();
  };

  // Common case: the survivors of the whole example fit the per-wave segments -> one scan shared
  // by all columns of the group; if they also fit one record chunk and the channels one register
  // group, the records are shared as well.  Otherwise atoms are taken in passes of kSuper (whose
  // survivors always fit) and every column scans again.
  bool one_pass = false;
  bool records_cached = false;
  if (end - begin <= 65536) {
    one_pass = scan(begin, end);
    if (one_pass && ncand <= kRecChunk && g.ntypes <= kRegChannels) {
      build_records(begin, 0, ncand, 0, g.ntypes);
      records_cached = true;
    }
  }
  const int pass_len = one_pass ? max(end - begin, 1) : kSuper;

  for (int cbase = 0; cbase < g.ntypes; cbase += kRegChannels) {
    const int nchan = min(kRegChannels, g.ntypes - cbase);
    const bool full_group = nchan == kRegChannels;
    for (int col = 0; col < kColsPerGroup; ++col) {
      const int y0 = gy0 + col * kColXY;
      if (y0 >= dim) break;
      const int vyi = y0 + ly;
      const bool xy_live = vxi < dim && vyi < dim;
      const float vy = grid_coord(oy, vyi, g.resolution);
      const float cly = uniform(grid_coord(oy, y0, g.resolution));
      const float chy = uniform(grid_coord(oy, min(y0 + kColXY, dim) - 1, g.resolution));

      acc_zero_all();

      for (int s0 = begin; s0 < end; s0 += pass_len) {
        if (!one_pass) scan(s0, min(end, s0 + kSuper));
        for (int c0 = 0; c0 < ncand; c0 += kRecChunk) {
          const int m = min(kRecChunk, ncand - c0);
          if (!records_cached) build_records(s0, c0, m, cbase, nchan);

          // ---- cull per 4x4x4 block, then splat ----------------------------------
#pragma unroll 1
          for (int blk = 0; blk < kBlocksPerWave; ++blk) {
            const int zb = z0 + (wave * kBlocksPerWave + blk) * 4;
            if (zb >= zend) continue;
            const float blz = uniform(grid_coord(oz, zb, g.resolution));
            const float bhz = uniform(grid_coord(oz, min(zb + 4, zend) - 1, g.resolution));
            const int vzi = zb + lz;
            const bool live = xy_live && vzi < zend;
            // a voxel outside the grid sits at infinity: no atom reaches it
            const float vz = live ? grid_coord(oz, vzi, g.resolution) : INFINITY;
            const int acc0 = blk * kRegChannels;
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
                unsigned char* e = mine + (p >> 1) * kPairBytes;
                *reinterpret_cast<float4*>(e + (p & 1) * 16) = rec;
                if (VEC) *reinterpret_cast<int*>(e + 32 + (p & 1) * 4) = s_recatom[i];
                else e[32 + (p & 1)] = s_rectype[i];
                if (EXACT) s_miniclip[wave][p] = s_clip[i];
              }
              // one atom of the list against this lane's voxel; the sum is touched only where
              // the atom reaches the voxel
              auto splat = [&](const float4& r, int tag, int it) {
                float ar = 0.f;
                bool inside = true;
                if (EXACT) {
                  const uint4 cl = s_miniclip[wave][it];
                  inside = inside_clip(vxi, vyi, vzi, make_uint3(cl.x, cl.y, cl.z));
                  ar = __uint_as_float(cl.w);
                }
                float val;
                const bool hit = density_hit<BINARY, EXACT>(g, vx - r.x, vy - r.y, vz - r.z, r.w, ar,
                                                            frm2, grm2, quad_c, val);
                if (!VEC) {
                  if (hit && inside) acc_add<BINARY>(acc0 + tag, val);
                } else {
                  const float* __restrict__ tv = types + (size_t)tag * g.ntypes + cbase;
                  // the atom's weights, through wave-uniform loads issued together
                  float wgt[kRegChannels];
                  if (full_group && (vec_store & 2)) {   // 16-byte aligned rows: seven 4-wide loads
                    const float4* __restrict__ tv4 = reinterpret_cast<const float4*>(tv);
#pragma unroll
                    for (int q = 0; q < kRegChannels / 4; ++q) {
                      const float4 w4 = tv4[q];
                      wgt[4 * q] = w4.x; wgt[4 * q + 1] = w4.y; wgt[4 * q + 2] = w4.z; wgt[4 * q + 3] = w4.w;
                    }
                  } else if (full_group) {
#pragma unroll
                    for (int c = 0; c < kRegChannels; ++c) wgt[c] = tv[c];
                  } else {
#pragma unroll
                    for (int c = 0; c < kRegChannels; ++c) wgt[c] = c < nchan ? tv[c] : 0.f;
                  }
                  if (hit && inside) {
                    // binary occupancy (val is 1) adds the weight itself: fma(w, 1, sum) = sum + w
                    acc_fma7<0>(acc0, val, wgt[0], wgt[1], wgt[2], wgt[3], wgt[4], wgt[5], wgt[6]);
                    acc_fma7<7>(acc0, val, wgt[7], wgt[8], wgt[9], wgt[10], wgt[11], wgt[12], wgt[13]);
                    acc_fma7<14>(acc0, val, wgt[14], wgt[15], wgt[16], wgt[17], wgt[18], wgt[19], wgt[20]);
                    acc_fma7<21>(acc0, val, wgt[21], wgt[22], wgt[23], wgt[24], wgt[25], wgt[26], wgt[27]);
                  }
                }
              };
              struct Pair { float4 r0, r1; int t0, t1; };
              auto fetch = [&](int k) -> Pair {
                const unsigned char* e = mine + k * kPairBytes;
                Pair q;
                q.r0 = *reinterpret_cast<const float4*>(e);
                q.r1 = *reinterpret_cast<const float4*>(e + 16);
                if (VEC) {
                  q.t0 = *reinterpret_cast<const int*>(e + 32);
                  q.t1 = *reinterpret_cast<const int*>(e + 36);
                } else {
                  q.t0 = *reinterpret_cast<const unsigned short*>(e + 32);
                  q.t1 = 0;
                }
                return q;
              };
              auto splat_pair = [&](const Pair& q, int it) {
                int t0 = __builtin_amdgcn_readfirstlane(q.t0), t1;
                if (VEC) t1 = __builtin_amdgcn_readfirstlane(q.t1);
                else { t1 = t0 >> 8; t0 &= 0xff; }
                splat(q.r0, t0, it);
                if (it + 1 < n) splat(q.r1, t1, it + 1);
              };
              // four atoms per trip; entry k+1 is in flight while entry k is evaluated
              Pair pa = fetch(0);
              for (int it = 0; it < n; it += 4) {
                const Pair pb = fetch((it >> 1) + 1);
                splat_pair(pa, it);
                if (it + 2 >= n) break;
                pa = fetch((it >> 1) + 2);
                splat_pair(pb, it + 2);
              }
            }
          }
          if (!records_cached) lds_barrier();   // records are rebuilt next round
        }
      }

      // ---- store: four channels per round through a double-buffered LDS stage ----
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
      const unsigned dump0 = lds_address(s_stage + dump_off);
      const unsigned dump1 = dump0 + 16, dump2 = dump0 + 32;
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
              *reinterpret_cast<v4f*>(dst) = v;
            } else {
              dst[0] = v.x;
              if (gz + 1 < dim) dst[1] = v.y;
              if (gz + 2 < dim) dst[2] = v.z;
              if (gz + 3 < dim) dst[3] = v.w;
            }
          }
        }
      };
      static_assert(kRegChannels == 7 * kStageCh, "seven rounds below");
      acc_dump_round<0>(dump0, dump1, dump2); store_round(0);
      if (nchan > 4) { acc_dump_round<1>(dump0, dump1, dump2); store_round(1); }
      if (nchan > 8) { acc_dump_round<2>(dump0, dump1, dump2); store_round(2); }
      if (nchan > 12) { acc_dump_round<3>(dump0, dump1, dump2); store_round(3); }
      if (nchan > 16) { acc_dump_round<4>(dump0, dump1, dump2); store_round(4); }
      if (nchan > 20) { acc_dump_round<5>(dump0, dump1, dump2); store_round(5); }
      if (nchan > 24) { acc_dump_round<6>(dump0, dump1, dump2); store_round(6); }
      lds_barrier();
    }
  }
}

template <bool BINARY, bool EXACT, bool VEC>
hipError_t launch_one(const GridArg& g, const BatchArg& batch, int nbatch, const Vec3Arg& centers,
                      const float* coords, const float* types, const float* radii, float* out,
                      hipStream_t stream) {
  const int cols_per_side = (g.dim + kColXY - 1) / kColXY;
  const int slabs = (g.dim + kSlabZ - 1) / kSlabZ;
  const size_t chan_stride = (size_t)g.dim * g.dim * g.dim;
  // bit 0: float4 stores of the grid are aligned; bit 1: rows of the weight matrix are
  int vec_store = ((g.dim % 4 == 0) && ((reinterpret_cast<uintptr_t>(out) & 15) == 0) &&
                   ((chan_stride * g.ntypes) % 4 == 0)) ? 1 : 0;
  if (VEC && g.ntypes % 4 == 0 && (reinterpret_cast<uintptr_t>(types) & 15) == 0) vec_store |= 2;
  const int groups = cols_per_side * ((cols_per_side + kColsPerGroup - 1) / kColsPerGroup);
  hipLaunchKernelGGL((splat_column_kernel<BINARY, EXACT, VEC>),
                     dim3(groups * slabs, nbatch), dim3(kColThreads), 0,
                     stream, g, batch, centers, coords, types, radii, out, cols_per_side, vec_store);
  return hipGetLastError();
}

template <bool VEC>
hipError_t launch_mode(const GridArg& g, const BatchArg& batch, int nbatch, const Vec3Arg& centers,
                       const float* coords, const float* types, const float* radii, float* out,
                       bool binary, bool exact, hipStream_t stream) {
  if constexpr (!VEC) {
    if (binary && exact)
      return launch_one<true, true, VEC>(g, batch, nbatch, centers, coords, types, radii, out, stream);
    if (exact)
      return launch_one<false, true, VEC>(g, batch, nbatch, centers, coords, types, radii, out, stream);
  } else {
    // vector types with the exact predicates are not instantiated here (register budget)
    if (exact) return hipErrorInvalidValue;
  }
  if (binary)
    return launch_one<true, false, VEC>(g, batch, nbatch, centers, coords, types, radii, out, stream);
  return launch_one<false, false, VEC>(g, batch, nbatch, centers, coords, types, radii, out, stream);
}

}  // namespace

hipError_t launch_forward_index(const GridArg& g, const BatchArg& batch, int nbatch,
                                const Vec3Arg& centers, const float* coords,
                                const float* type_index, const float* radii, float* out,
                                bool binary, bool exact, hipStream_t stream) {
  // The channel-by-channel kernel takes every case it covers (anything but the exact cut-off
  // predicates and grids of 4 GB or more per example); MOLGRID_HIP_FORWARD_COLUMN_KERNEL=1 keeps
  // the column kernel below for all of them (a tested second implementation).
  const char* column_only = getenv("MOLGRID_HIP_FORWARD_COLUMN_KERNEL");
  if (!exact && !(column_only != nullptr && column_only[0] == '1')) {
    const hipError_t e = launch_forward_channel(g, batch, nbatch, centers, coords, type_index,
                                                radii, out, binary, stream);
    if (e != hipErrorInvalidValue) return e;
  }
  return launch_mode<false>(g, batch, nbatch, centers, coords, type_index, radii, out, binary, exact,
                            stream);
}

hipError_t launch_forward_vector_column(const GridArg& g, const BatchArg& batch, int nbatch,
                                        const Vec3Arg& centers, const float* coords,
                                        const float* type_vector, const float* radii, float* out,
                                        bool binary, bool exact, hipStream_t stream) {
  return launch_mode<true>(g, batch, nbatch, centers, coords, type_vector, radii, out, binary, exact,
                           stream);
}

}  // namespace mg
