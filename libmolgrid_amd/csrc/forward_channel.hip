// Forward splat for index types, one channel at a time (GridMaker::forward,
// src/grid_maker.cpp:160-211, src/grid_maker.cu:95-211).
//
// A workgroup owns four columns of 4 x 4 voxels in (x, y), consecutive in y, over a slab of up to
// 48 voxels in z, one column per wave.  The atoms that can reach the four columns are found by one
// scan of the example and sorted by channel (stably, so each channel keeps ascending atom order).
// Each wave then walks the channels on its own: the densities of one channel are summed in twelve
// registers per lane (one voxel in each of the column's twelve 4x4x4 blocks, in atom order), put
// into the wave's own LDS stage and written out as whole z rows.  Only the sums of the current
// channel live in registers, so the kernel needs few of them; after the sort the waves share
// read-only data only and never wait for each other.
//
// Every global access goes through buffer instructions with the extent of the array they address,
// so an index outside it reads zero or is dropped.
#include "kernels.h"
#include "splat_common.h"

namespace mg {
namespace {

constexpr int kColXY = 4;                        // column footprint in x and y
constexpr int kWaves = 4;                        // = columns per workgroup
constexpr int kThreads = kWaves * kWave;
constexpr int kBlocks = 12;                      // 4x4x4 blocks of a column
constexpr int kSlabZ = kBlocks * 4;              // 48
constexpr int kRowPad = 52;                      // staged z row, padded against bank conflicts
constexpr int kPlane = 16 * kRowPad;             // one staged column (floats)
constexpr int kSuper = 2048;                     // atoms scanned per pass
constexpr int kSeg = kSuper / kWaves;            // survivors kept per wave
constexpr int kRecMax = 512;                     // records resident at a time
constexpr int kSegs = kRecMax / kWave;           // 64-record pieces of the record array
constexpr int kSortChannels = 64;                // channels the one-pass sort handles
constexpr int kBufferFlags = 0x00020000;         // untyped 32-bit elements, no swizzle


typedef unsigned int v4u __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float uniform(float v) {
  return __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(v)));
}

__device__ __forceinline__ __amdgpu_buffer_rsrc_t buffer_of(const void* p, size_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0,
                                           (int)(bytes < 0xffffffffull ? bytes : 0xffffffffull),
                                           kBufferFlags);
}
__device__ __forceinline__ float buffer_float(__amdgpu_buffer_rsrc_t r, int index) {
  return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, index * 4, 0, 0));
}

// x, y, z of atom `index` with one 12-byte load (4-byte aligned, which multi-dword buffer loads
// accept): a third of the address cycles of three single loads.
typedef unsigned int v3u __attribute__((ext_vector_type(3)));
__device__ __forceinline__ float3 buffer_float3(__amdgpu_buffer_rsrc_t r, int index) {
  const v3u v = __builtin_amdgcn_raw_buffer_load_b96(r, index * 12, 0, 0);
  return make_float3(__uint_as_float(v.x), __uint_as_float(v.y), __uint_as_float(v.z));
}

// LDS-only barrier: outstanding global stores are not waited for.
__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// Seven workgroups per CU (72 registers): the launch of configuration 1 (1,800 workgroups) then
// fits the 1,792 slots of the chip in one go.
template <bool BINARY>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(7, 7))) void
splat_channel_kernel(
    GridArg g, BatchArg batch, Vec3Arg centers, const float* __restrict__ coords,
    const float* __restrict__ types, const float* __restrict__ radii, float* __restrict__ out,
    int cols_per_side, int aligned_rows) {
  constexpr int kStage = kWaves * kPlane;
  __shared__ __align__(16) float s_stage[kStage];  // one column per wave
  __shared__ float4 s_rec[kRecMax];                // x, y, z, (ar^2 | 1/ar^2), sorted by channel
  __shared__ int s_wcount[kWaves];
  __shared__ int s_start[kSortChannels + 1];       // first record of each channel

  // The stage is not in use while atoms are scanned and sorted; it then holds the survivors of
  // the scan (atom numbers) and the records per (64-record piece, channel).
  unsigned short (*s_idx)[kSeg] = reinterpret_cast<unsigned short (*)[kSeg]>(s_stage);
  int (*s_cnt)[kSortChannels] =
      reinterpret_cast<int (*)[kSortChannels]>(s_stage + kWaves * kSeg / 2);
  static_assert(kWaves * kSeg / 2 + kSegs * kSortChannels <= kStage, "both fit the stage");

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid >> 6;
  const int b = example_for_slot(batch, blockIdx.y, gridDim.y, lane);
  int begin, end;
  example_range(batch, b, begin, end);
  const int natoms = max(end - begin, 0);          // atoms are numbered from the example's first
  const float3 center = load3(centers, b);
  const float ox = uniform(center.x - g.half_dimension);
  const float oy = uniform(center.y - g.half_dimension);
  const float oz = uniform(center.z - g.half_dimension);
  const int dim = g.dim;
  const int ntypes = g.ntypes;

  const __amdgpu_buffer_rsrc_t coords_buf = buffer_of(coords + (size_t)begin * 3, (size_t)natoms * 12);
  const __amdgpu_buffer_rsrc_t radii_buf = buffer_of(radii + begin, (size_t)natoms * 4);
  const __amdgpu_buffer_rsrc_t types_buf = buffer_of(types + begin, (size_t)natoms * 4);
  const size_t chan_stride = (size_t)dim * dim * dim;
  // the grids of this example; the host has checked that they fit a buffer's 32-bit extent
  const __amdgpu_buffer_rsrc_t out_buf =
      buffer_of(out + (size_t)b * ntypes * chan_stride, (size_t)ntypes * chan_stride * 4);

  // which four columns and which z slab
  const int groups_per_row = (cols_per_side + kWaves - 1) / kWaves;
  const int ngroups = cols_per_side * groups_per_row;
  const int slab = blockIdx.x / ngroups;
  const int grp = blockIdx.x - slab * ngroups;
  const int x0 = (grp / groups_per_row) * kColXY;
  const int gy0 = (grp % groups_per_row) * (kColXY * kWaves);
  const int y0 = gy0 + wave * kColXY;              // this wave's column
  const int z0 = slab * kSlabZ;
  const int zend = min(z0 + kSlabZ, dim);          // exclusive
  const bool column_live = y0 < dim;

  // box of the whole group (first/last voxel centre inside the grid) and of this wave's column
  const float clx = uniform(grid_coord(ox, x0, g.resolution));
  const float chx = uniform(grid_coord(ox, min(x0 + kColXY, dim) - 1, g.resolution));
  const float gly = uniform(grid_coord(oy, gy0, g.resolution));
  const float ghy = uniform(grid_coord(oy, min(gy0 + kColXY * kWaves, dim) - 1, g.resolution));
  const float clz = uniform(grid_coord(oz, z0, g.resolution));
  const float chz = uniform(grid_coord(oz, zend - 1, g.resolution));
  const float cly = uniform(grid_coord(oy, min(y0, dim - 1), g.resolution));
  const float chy = uniform(grid_coord(oy, min(y0 + kColXY, dim) - 1, g.resolution));

  // the voxels this lane owns: one in each of the column's twelve blocks; a voxel outside the
  // grid sits at infinity, where no atom reaches it
  const int lx = lane >> 4, ly = (lane >> 2) & 3, lz = lane & 3;
  const int vxi = x0 + lx, vyi = y0 + ly;
  const float vx = grid_coord(ox, vxi, g.resolution);
  const float vy = grid_coord(oy, vyi, g.resolution);
  float vz[kBlocks];
#pragma unroll
  for (int q = 0; q < kBlocks; ++q) {
    const int vzi = z0 + q * 4 + lz;
    vz[q] = (vxi < dim && vyi < dim && vzi < zend) ? grid_coord(oz, vzi, g.resolution) : INFINITY;
  }
  float* const stage = s_stage + wave * kPlane;    // this wave's column
  const int stage_lane = (lx * 4 + ly) * kRowPad + lz;

  float quad_c = g.C;
  asm volatile("" : "+v"(quad_c));          // vector register (an fma takes one scalar operand)
  const float frm2 = uniform(g.frm * g.frm);
  const float grm2 = uniform(g.grm * g.grm);
  const float cull_mult = BINARY ? 1.0f : g.frm;   // support radius / ar

  // this lane's part in the write-out of a channel: for each of the column's four x, lane
  // (y, granule) takes one float4 piece of a z row; the four rows of an x follow each other in
  // memory, so one store instruction of the wave covers 768 contiguous bytes
  const int st_y = lane / 12, st_f4 = lane - st_y * 12;           // lanes 48..63 idle
  const int st_gz = z0 + st_f4 * 4;
  const bool st_lane_live = st_y < 4 && y0 + st_y < dim && st_gz < zend;
  const int st_lds = st_y * kRowPad + st_f4 * 4;
  const unsigned st_off = (unsigned)((x0 * dim + y0 + st_y) * dim + st_gz) * 4u;
  const unsigned st_xstride = (unsigned)(dim * dim) * 4u;

  // One channel of the wave's stage (or zeros) -> global memory as z rows.
  auto store_channel = [&](int c, bool from_stage) {
    const unsigned chan_off = (unsigned)c * (unsigned)(chan_stride * 4);   // < 4 GB in total
#pragma unroll
    for (int k = 0; k < kColXY; ++k) {
      if (st_lane_live && x0 + k < dim) {
        v4f v = {0.f, 0.f, 0.f, 0.f};
        if (from_stage) v = *reinterpret_cast<const v4f*>(stage + st_lds + k * 4 * kRowPad);
        const unsigned off = chan_off + st_off + k * st_xstride;
        if (aligned_rows && st_gz + 3 < dim) {
          // non-temporal: nothing reads the grids back soon enough to find them in the last-level
          // cache, and without the hint its write-back runs on into the next kernel
          __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, v), out_buf, (int)off, 0, 2);
        } else {
          const float e[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
          for (int t = 0; t < 4; ++t)
            if (st_gz + t < dim)
              __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, e[t]), out_buf,
                                                    (int)(off + 4u * t), 0, 0);
        }
      }
    }
  };

  int segstart[kWaves + 1];
  int ncand = 0;

  // ---- scan: atoms [s0, s1) against the group's box -> per-wave index segments --------------
  // Each wave takes a contiguous quarter of the range and keeps up to kSeg survivors (offsets
  // from s0 as 16-bit values, so s1 - s0 <= 65536).  `only` >= 0 keeps atoms of that channel
  // only.  Returns false if a segment overflowed.
  auto scan = [&](int s0, int s1, int only) -> bool {
    const int quarter = (s1 - s0 + kWaves - 1) / kWaves;
    int wcnt = 0;
    const int wb = s0 + wave * quarter, we = min(s1, wb + quarter);
    constexpr int U = 2;
    for (int a0 = wb; a0 < we; a0 += kWave * U) {
      float rr[U], cx[U], cy[U], cz[U], ty[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int a = min(a0 + u * kWave + lane, we - 1);
        rr[u] = buffer_float(radii_buf, a);
        const float3 c = buffer_float3(coords_buf, a);
        cx[u] = c.x;
        cy[u] = c.y;
        cz[u] = c.z;
        ty[u] = only >= 0 ? buffer_float(types_buf, a) : 0.f;
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int a = a0 + u * kWave + lane;
        const float reach = rr[u] * g.radius_scale * cull_mult;
        bool p = (a < we) && box_distance2(cx[u], cy[u], cz[u], clx, gly, clz, chx, ghy, chz) <=
                                 reach * reach * kCullSlack;
        if (only >= 0) p = p && floorf(ty[u]) == (float)only;
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
    for (int w = 0; w < kWaves; ++w) {
      const int c = __builtin_amdgcn_readfirstlane(s_wcount[w]);
      fits = fits && c <= kSeg;
      segstart[w + 1] = segstart[w] + min(c, kSeg);
    }
    ncand = segstart[kWaves];
    lds_barrier();   // every wave has read the counts before any of them scans again
    return fits;
  };

  // candidate gi of the current scan -> its atom; the record of that atom
  auto atom_of = [&](int s0, int gi) -> int {
    int w = 0;
#pragma unroll
    for (int k = 1; k < kWaves; ++k) w += (gi >= segstart[k]) ? 1 : 0;
    return s0 + s_idx[w][min(gi - segstart[w], kSeg - 1)];
  };
  auto record_of = [&](int a) -> float4 {
    const float3 at = buffer_float3(coords_buf, a);
    const float ax = at.x, ay = at.y, az = at.z;
    float ar, ar2;
    {
#pragma clang fp contract(off)
      ar = buffer_float(radii_buf, a) * g.radius_scale;
      ar2 = ar * ar;
    }
    return make_float4(ax, ay, az, BINARY ? ar2 : 1.0f / ar2);
  };

  // the sums of the current channel at this lane's twelve voxels
  float acc[kBlocks];
#pragma unroll
  for (int q = 0; q < kBlocks; ++q) acc[q] = 0.f;
  // sums -> the wave's stage (and cleared for the next channel); the wave reads them back itself,
  // and LDS keeps the order of one wave's accesses
  auto stage_sums = [&]() {
#pragma unroll
    for (int q = 0; q < kBlocks; ++q) {
      stage[stage_lane + q * 4] = acc[q];
      acc[q] = 0.f;
    }
  };

  // ---- records [lo, hi) of s_rec, all of one channel, added to the sums -----------------------
  // A cull round takes 64 records, one per lane: the lane finds the interval of z the atom can
  // reach inside the column (its reach shrunk by the distance to the column's footprint in x and
  // y) and from it the range of blocks, as a bit mask.  The records that reach the column are then
  // taken one at a time, in record order, each over the blocks of its mask; the record comes
  // straight from the lane that tested it.
  const float inv_block = 0.25f / g.resolution;             // blocks per unit length along z
  const int last_block = (zend - z0 + 3) / 4 - 1;
  auto splat_records = [&](int lo, int hi) {
    for (int r0 = lo; r0 < hi; r0 += kWave) {
      const int i = r0 + lane;
      const bool valid = i < hi;
      const float4 rec = s_rec[valid ? i : lo];
      const float ex = fmaxf(fmaxf(clx - rec.x, rec.x - chx), 0.f);
      const float ey = fmaxf(fmaxf(cly - rec.y, rec.y - chy), 0.f);
      // squared reach (with the slack that keeps the cull a superset) minus the part spent in x, y
      const float reach2 = (BINARY ? rec.w : frm2 * __builtin_amdgcn_rcpf(rec.w)) * kCullSlack;
      const float rz2 = reach2 - (ex * ex + ey * ey);
      unsigned blocks = 0;
      if (valid && rz2 >= 0.f) {
        const float rz = __builtin_amdgcn_sqrtf(rz2);
        // block q holds the voxel centres clz + (4q .. 4q+3) * resolution
        const float top = (rec.z + rz - clz) * inv_block + 1e-3f;
        const float bottom = (rec.z - rz - clz) * inv_block - (0.75f + 1e-3f);
        const int qhi = min((int)floorf(top), last_block), qlo = max((int)ceilf(bottom), 0);
        if (qlo <= qhi) blocks = (2u << qhi) - (1u << qlo);
      }
      // the records that reach the column, in record order; the part of the distance that lies in
      // x and y is the same for every block of a record
      unsigned long long todo = __ballot(blocks != 0);
#pragma unroll 1
      while (todo != 0) {                          // loses a bit per trip
        const int src = __builtin_ctzll(todo);
        todo &= todo - 1ull;
        const float rx = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(rec.x), src));
        const float ry = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(rec.y), src));
        const float rz = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(rec.z), src));
        const float rw = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(rec.w), src));
        const unsigned reach = (unsigned)__builtin_amdgcn_readlane((int)blocks, src);
        const float dx = vx - rx, dy = vy - ry;
        float dxy2;
        if (BINARY) {
#pragma clang fp contract(off)
          dxy2 = dx * dx + dy * dy;
        } else {
          dxy2 = fmaf(dx, dx, dy * dy);
        }
#pragma unroll
        for (int q0 = 0; q0 < kBlocks; q0 += 4) {
          if (((reach >> q0) & 0xfu) == 0) continue;
#pragma unroll
          for (int q = q0; q < q0 + 4; ++q) {
            if (((reach >> q) & 1u) == 0) continue;
            const float dz = vz[q] - rz;
            if (BINARY) {
              float rsq;
              {
#pragma clang fp contract(off)
                rsq = dxy2 + dz * dz;
              }
              if (rsq < rw) acc[q] = 1.0f;
            } else {
              const float u = fmaf(dz, dz, dxy2) * rw;
              if (u <= frm2) {
                const float gauss = __builtin_amdgcn_exp2f(u * kNeg2Log2e);
                const float su = __builtin_amdgcn_sqrtf(u);
                const float quad = fmaxf(fmaf(g.A, u, fmaf(g.B, su, quad_c)), 0.f);
                acc[q] += (u <= grm2) ? gauss : quad;
              }
            }
          }
        }
      }
    }
  };

  // ---- common case: one scan, survivors sorted by channel into resident records --------------
  bool sorted = false;
  if (natoms <= 65536 && ntypes <= kSortChannels) {
    const bool one_pass = scan(0, natoms, -1);
    if (one_pass && ncand <= kRecMax) {
      sorted = true;
      for (int i = tid; i < kSegs * kSortChannels; i += kThreads) (&s_cnt[0][0])[i] = 0;
      __syncthreads();
      constexpr int kMine = kRecMax / kThreads;   // records per thread
      float4 rec[kMine];
      int chan[kMine], rank[kMine];
#pragma unroll
      for (int k = 0; k < kMine; ++k) {
        const int gi = tid + k * kThreads;
        const bool have = gi < ncand;
        const int a = have ? atom_of(0, gi) : 0;
        rec[k] = record_of(a);
        const float tf = floorf(buffer_float(types_buf, a));
        const bool act = have && tf >= 0.f && tf < (float)ntypes;   // others feed no channel
        chan[k] = act ? (int)tf : 0;
        // lanes of this wave with the same channel
        unsigned long long same = __ballot(act);
#pragma unroll
        for (int bit = 0; bit < 6; ++bit) {
          const bool set = (chan[k] >> bit) & 1;
          const unsigned long long bm = __ballot(act && set);
          same &= set ? bm : ~bm;
        }
        rank[k] = act ? __popcll(same & ((1ull << lane) - 1ull)) : -1;
        if (rank[k] == 0) s_cnt[wave + k * kWaves][chan[k]] = __popcll(same);
      }
      __syncthreads();
      if (wave == 0) {
        // lane = channel: pieces in order, then channels in order
        int run = 0;
#pragma unroll
        for (int s = 0; s < kSegs; ++s) {
          const int v = s_cnt[s][lane];
          s_cnt[s][lane] = run;
          run += v;
        }
        int incl = run;
#pragma unroll
        for (int d = 1; d < kWave; d <<= 1) {
          const int t = __shfl_up(incl, d);
          if (lane >= d) incl += t;
        }
        const int excl = incl - run;
        s_start[lane] = excl;
        if (lane == kWave - 1) s_start[kWave] = incl;
#pragma unroll
        for (int s = 0; s < kSegs; ++s) s_cnt[s][lane] += excl;
      }
      __syncthreads();
#pragma unroll
      for (int k = 0; k < kMine; ++k)
        if (rank[k] >= 0) s_rec[min(s_cnt[wave + k * kWaves][chan[k]] + rank[k], kRecMax - 1)] = rec[k];
      __syncthreads();
    }
  }

  if (sorted) {
    if (!column_live) return;
    // Most or all workgroups of a launch are resident at once, and a wave's time grows with the
    // atoms around its column: waves with many records get a higher issue priority, so that they
    // finish less far behind the others.
    if (ncand >= 384) __builtin_amdgcn_s_setprio(3);
    else if (ncand >= 256) __builtin_amdgcn_s_setprio(2);
    else if (ncand >= 128) __builtin_amdgcn_s_setprio(1);
    // Channels differ a lot in work (some hold most atoms, many hold none, and an empty channel is
    // stores only), so the waves start at different channels: at any time some compute while
    // others store.  The order of the channels does not matter to the sums.
    const int first = (int)((blockIdx.x * 7u + blockIdx.y * 3u + wave * 5u) % (unsigned)ntypes);
    for (int i = 0; i < ntypes; ++i) {
      const int c = first + i < ntypes ? first + i : first + i - ntypes;
      const int lo = __builtin_amdgcn_readfirstlane(s_start[c]);
      const int hi = __builtin_amdgcn_readfirstlane(s_start[c + 1]);
      if (hi > lo) {
        splat_records(lo, hi);
        stage_sums();
        store_channel(c, true);
      } else {
        store_channel(c, false);
      }
    }
    return;
  }

  // ---- any size: every channel scans the atoms again, keeping its own -------------------------
  for (int c = 0; c < ntypes; ++c) {
    for (int s0 = 0; s0 < natoms; s0 += kSuper) {
      scan(s0, min(natoms, s0 + kSuper), c);
      for (int c0 = 0; c0 < ncand; c0 += kRecMax) {
        const int m = min(kRecMax, ncand - c0);
        for (int r = tid; r < m; r += kThreads) s_rec[r] = record_of(atom_of(s0, c0 + r));
        __syncthreads();
        if (column_live) splat_records(0, m);
        lds_barrier();   // before the records are built again
      }
    }
    if (column_live) {
      stage_sums();
      store_channel(c, true);
    }
    lds_barrier();   // the stage holds the next scan's survivors
  }
}

}  // namespace

// Returns hipErrorInvalidValue when the kernel does not cover the case (the caller then uses the
// column kernel): the grids of one example must fit a buffer's 32-bit extent.
hipError_t launch_forward_channel(const GridArg& g, const BatchArg& batch, int nbatch,
                                  const Vec3Arg& centers, const float* coords,
                                  const float* type_index, const float* radii, float* out,
                                  bool binary, hipStream_t stream) {
  const size_t chan_stride = (size_t)g.dim * g.dim * g.dim;
  if ((size_t)g.ntypes * chan_stride * 4 >= 0xfffffff0ull) return hipErrorInvalidValue;
  const int cols_per_side = (g.dim + kColXY - 1) / kColXY;
  const int slabs = (g.dim + kSlabZ - 1) / kSlabZ;
  const int aligned = ((g.dim % 4 == 0) && ((reinterpret_cast<uintptr_t>(out) & 15) == 0)) ? 1 : 0;
  const int groups = cols_per_side * ((cols_per_side + kWaves - 1) / kWaves);
  const dim3 grid(groups * slabs, nbatch), block(kThreads);
  if (binary)
    hipLaunchKernelGGL((splat_channel_kernel<true>), grid, block, 0, stream, g, batch, centers,
                       coords, type_index, radii, out, cols_per_side, aligned);
  else
    hipLaunchKernelGGL((splat_channel_kernel<false>), grid, block, 0, stream, g, batch, centers,
                       coords, type_index, radii, out, cols_per_side, aligned);
  return hipGetLastError();
}

}  // namespace mg
