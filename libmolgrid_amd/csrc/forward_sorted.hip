// Forward splat for index types (GridMaker::forward, src/grid_maker.cpp:153-212,
// src/grid_maker.cu:95-130), in two launches.
//
// 1. sort_atoms_kernel: the atoms of every example become 16-byte records (x, y, z, ar =
//    radius * radius_scale), sorted by (channel, x slab of the centre) and, within a key, in
//    ascending atom order (a stable counting sort, one workgroup per example and group of a few
//    channels).  Atoms without a
//    channel drop out.  The workgroup also finds the rank of its example by size and writes the
//    example's tables -- grid origin, example number, and for every (channel, x slab) the run of
//    records that can reach the slab -- at that rank, so that the second launch meets the examples
//    largest first.
// 2. splat_sorted_kernel: one wave per work item, no workgroup of more than one wave, nothing
//    shared between waves.  An item is a territory of 4 x (4 * COLS) x 48 voxels -- COLS columns
//    of 4 x 4 voxels in (x, y), consecutive in y, each twelve 4x4x4 blocks tall -- of one example,
//    for every R-th channel.  For each of these channels the first launch has left the run of
//    records whose atoms can reach the territory's four x planes.  The wave first writes zeros for
//    its channels with an empty run.  Then it walks the others: the records are read 64 at a time
//    (one per lane, the next 64 in flight), each lane finds the blocks its record can reach, the
//    records that reach the territory are taken one at a time, in record order, and summed in
//    registers (one voxel of every block per lane); each column then goes through the wave's LDS
//    stage and is written out as whole z rows.  The hardware hands out the items in order, the
//    largest example first, so the last ones running are small.
//
// Sums run in record order: by x slab of the atom's centre, then by atom number.  That is a fixed
// order (results are the same from run to run) but not the CPU loop's plain atom order, so
// Gaussian densities agree with it to rounding, not to the bit; binary densities are exact.
//
// Every global access of the splat kernel goes through buffer instructions that carry the
// extent of the array they address: an index outside it reads zero or is dropped.
#include <algorithm>
#include <atomic>

#include "kernels.h"
#include "splat_common.h"

namespace mg {
namespace {

constexpr int kColXY = 4;                        // column footprint in x and y
constexpr int kBlocks = 12;                      // 4x4x4 blocks of a column
constexpr int kSlabZ = kBlocks * 4;              // 48
constexpr int kRowPad = 52;                      // staged z row, padded against bank conflicts
constexpr int kPlane = 16 * kRowPad;             // one staged column (floats)
constexpr int kPieces = 16 * (kSlabZ / 4) / kWave;   // float4 pieces of a column per lane: 3
constexpr int kBufferFlags = 0x00020000;         // untyped 32-bit elements, no swizzle
constexpr int kItemChannels = 4;                 // channels an item takes, about
constexpr int kItemChannelsMax = 64;             // ... and at most (one per lane)
constexpr int kSortChannels = 4;                 // channels a workgroup of the sort takes, about

// Paged write-out: a workgroup of one wave per pair of columns owns a whole slab of four x planes
// of ONE channel -- a contiguous run of the output -- collects the sums of its waves in LDS and
// writes the run as bursts of whole 4 KB pages, each page by one wave in four back-to-back
// stores.  For grids of up to kPagedDim voxels a side, whose slab fits the LDS.
constexpr int kPagedDim = 48;
constexpr int kPagedWaves = (kPagedDim + 2 * kColXY - 1) / (2 * kColXY);   // 6
constexpr int kPageBytes = 4096;
// LDS slab [4 planes][dim rows][dim + 4]: rows padded by four floats and planes spaced 16 banks
// (mod 32) apart, so that the 32 lanes of a half wave (2 planes x 4 rows x 4 voxels) hit 32 banks
__host__ __device__ constexpr int paged_row(int dim) { return dim + 4; }
__host__ __device__ constexpr int paged_plane(int dim) {
  return dim * paged_row(dim) + ((16 - dim * paged_row(dim)) % 32 + 32) % 32;
}
constexpr int kSlabFloats = kColXY * paged_plane(kPagedDim);               // 10,048 floats

constexpr int kSortWaves = 16;
constexpr int kSortThreads = kSortWaves * kWave;
constexpr int kKeyGroup = 512;                   // keys a workgroup of the sort handles, at most
constexpr int kCached = 4;                       // atoms a thread keeps in registers

typedef unsigned int v4u __attribute__((ext_vector_type(4)));
typedef unsigned int v2u __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float uniform(float v) {
  return __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(v)));
}
__device__ __forceinline__ __amdgpu_buffer_rsrc_t buffer_of(const void* p, size_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0,
                                           (int)(bytes < 0xffffffffull ? bytes : 0xffffffffull),
                                           kBufferFlags);
}
__device__ __forceinline__ float lane_value(float v, int src) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), src));
}

// ------------------------------------------------------------------------------------------
// Workspace: slot_info [nbatch] | cand [nbatch * ntypes * nxs * 2] | records [capacity]
// A key is (channel, x slab), where the slab of an atom is the group of four x planes its centre
// lies in (clamped to the grid); nxs slabs.
// ------------------------------------------------------------------------------------------
constexpr size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

struct SortedAtoms {
  float4* slot_info;   // per launch slot (examples in descending size): grid origin, example number
  int* cand;           // per launch slot, channel and x slab: first and one-past-last record of the
                       // channel that can reach the slab's four x planes
  float4* records;
  int capacity;        // records
};

SortedAtoms carve(void* workspace, int nbatch, int nkeys, long long capacity) {
  unsigned char* p = static_cast<unsigned char*>(workspace);
  SortedAtoms s;
  s.slot_info = reinterpret_cast<float4*>(p);
  p += align256((size_t)nbatch * 16);
  s.cand = reinterpret_cast<int*>(p);
  p += align256((size_t)nbatch * nkeys * 8);
  s.records = reinterpret_cast<float4*>(p);
  s.capacity = (int)capacity;
  return s;
}

// slab of an x coordinate, as a float in [0, nxs - 1]; monotone in x
__device__ __forceinline__ float slab_of(float x, float ox, float inv_slab, int nxs) {
  return fminf(fmaxf(floorf((x - ox) * inv_slab + 0.125f), 0.f), (float)(nxs - 1));
}

// ------------------------------------------------------------------------------------------
// Launch 1: a stable counting sort of the atoms by key.  Workgroup (part, example) takes the
// channels [part * per_part, (part + 1) * per_part) of its example: it reads all atoms of the
// example, counts those of lower channels (their records come first), and sorts its own.
// per_part * nxs <= kKeyGroup.
// ------------------------------------------------------------------------------------------
__global__ __launch_bounds__(kSortThreads) void sort_atoms_kernel(
    GridArg g, BatchArg batch, int nbatch, int nxs, int parts, int per_part, float reach_mult,
    Vec3Arg centers, const float* __restrict__ coords, const float* __restrict__ types,
    const float* __restrict__ radii, float4* __restrict__ slot_info, int* __restrict__ cand,
    float4* __restrict__ records, int capacity) {
  __shared__ int s_cnt[kSortWaves][kKeyGroup];   // atoms per (wave, key), then write positions
  __shared__ int s_tot[kKeyGroup + 1];
  __shared__ int s_rank, s_rmax, s_below;
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid >> 6;
  const int e = blockIdx.x / parts, part = blockIdx.x - e * parts;
  const int c0 = part * per_part, c1 = min(g.ntypes, c0 + per_part);
  const int nkeys = (c1 - c0) * nxs;
  const int key_bits = 32 - __builtin_clz(max(nkeys - 1, 1));   // bits that tell the keys apart
  const int kpad = (nkeys + kWave - 1) & ~(kWave - 1);          // keys the tables below cover
  // the small loads first and together: this example's atoms, the size of one other example
  // (for the rank below), the grid centre
  const int32_t* const off = batch.offsets;
  int begin = e * batch.per_example, end = begin + batch.per_example, first = 0, other_size = -1;
  if (off != nullptr) {
    first = off[0];
    begin = off[e];
    end = off[e + 1];
    const int i = min(tid, nbatch - 1);
    other_size = off[i + 1] - off[i];
  }
  const int n = max(end - begin, 0);
  const int ntypes = g.ntypes;
  const float radius_scale = g.radius_scale;
  const float inv_slab = 0.25f / g.resolution;
  const float3 center = load3(centers, e);
  const float ox = center.x - g.half_dimension;
  // every wave takes a contiguous run of whole 64-atom rounds, in atom order
  const int per = ((n + kSortThreads - 1) / kSortThreads) * kWave;
  const int wb = begin + wave * per, we = min(end, wb + per);
  const bool cached = per <= kCached * kWave;

  // key of an atom among this workgroup's; -1: a higher channel, -2: a lower one, -3: none.
  // An atom whose radius is not positive (or not a number) reaches no voxel (its index box,
  // src/grid_maker.cu:66-79, is empty) and drops out like an atom without a channel.
  auto key_of = [&](float type, float x, float ar) -> int {
    const float tf = floorf(type);
    if (!(tf >= 0.f && tf < (float)ntypes) || !(ar > 0.f)) return -3;
    const int c = (int)tf;
    if (c < c0) return -2;
    if (c >= c1) return -1;
    return (c - c0) * nxs + (int)slab_of(x, ox, inv_slab, nxs);
  };

  auto scaled = [&](float radius) -> float {
#pragma clang fp contract(off)
    return radius * radius_scale;
  };
  // the atoms of this thread, read once when they fit its registers
  int c_key[kCached];
  float c_x[kCached], c_y[kCached], c_z[kCached], c_r[kCached];
  float my_rmax = 0.f;
  int my_below = 0;
  if (cached) {
    // all loads first, unconditionally (a clamped atom number), so that they are in flight
    // together; what they returned is looked at afterwards
    float c_t[kCached];
    const int last = max(end - 1, 0);
#pragma unroll
    for (int k = 0; k < kCached; ++k) c_t[k] = c_x[k] = c_y[k] = c_z[k] = c_r[k] = 0.f;
    if (n > 0) {                               // an example without atoms may come with no arrays
#pragma unroll
      for (int k = 0; k < kCached; ++k) {
        const int ac = min(wb + k * kWave + lane, last);
        c_t[k] = types[ac];
        c_x[k] = coords[3 * ac];
        c_y[k] = coords[3 * ac + 1];
        c_z[k] = coords[3 * ac + 2];
        c_r[k] = radii[ac];
      }
    }
#pragma unroll
    for (int k = 0; k < kCached; ++k) {
      const bool have = n > 0 && wb + k * kWave + lane < we;
      {
#pragma clang fp contract(off)
        c_r[k] = c_r[k] * radius_scale;
      }
      c_key[k] = have ? key_of(c_t[k], c_x[k], c_r[k]) : -3;
      if (c_key[k] != -3) my_rmax = fmaxf(my_rmax, c_r[k]);
      my_below += c_key[k] == -2 ? 1 : 0;
    }
  } else {
    for (int a = wb + lane; a < we; a += kWave) {
      const float ar = scaled(radii[a]);
      const int key = key_of(types[a], coords[3 * a], ar);
      if (key != -3) my_rmax = fmaxf(my_rmax, ar);
      my_below += key == -2 ? 1 : 0;
    }
  }

  if (tid == 0) {
    s_rank = 0;
    s_rmax = 0;
    s_below = 0;
  }
  for (int k = lane; k < kpad; k += kWave) s_cnt[wave][k] = 0;
  __syncthreads();
  // atoms of lower channels; the largest ar of the example; the rank of the example by size
  // (descending, ties in input order)
  // (reduced over the wave first: one LDS atomic per wave, not one per lane on one address)
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    my_below += __shfl_xor(my_below, d);
    my_rmax = fmaxf(my_rmax, __shfl_xor(my_rmax, d));
  }
  if (lane == 0) {
    if (my_below) atomicAdd(&s_below, my_below);
    if (my_rmax > 0.f) atomicMax(&s_rmax, __float_as_int(my_rmax));   // positive floats order as ints
  }
  if (off != nullptr) {
    int before = 0;
    for (int i = tid; i < nbatch; i += kSortThreads) {
      const int other = i == tid ? other_size : off[i + 1] - off[i];
      before += (other > end - begin || (other == end - begin && i < e)) ? 1 : 0;
    }
    if (before) atomicAdd(&s_rank, before);
  }
  auto count = [&](int key) {
    if (key >= 0) atomicAdd(&s_cnt[wave][key], 1);
  };
  if (cached) {
#pragma unroll
    for (int k = 0; k < kCached; ++k) count(c_key[k]);
  } else {
    for (int a = wb + lane; a < we; a += kWave)
      count(key_of(types[a], coords[3 * a], scaled(radii[a])));
  }
  __syncthreads();
  const int slot = off != nullptr ? s_rank : e;
  if (tid == 0 && part == 0)
    slot_info[slot] = make_float4(ox, center.y - g.half_dimension, center.z - g.half_dimension,
                                  __int_as_float(e));
  // how far in x the atoms of this example reach, at most (with a margin over the cull's slack)
  const float reach = __int_as_float(s_rmax) * reach_mult * 1.0001f + 1e-3f;
  const int base = begin - first + s_below;      // first record of this workgroup's channels

  // per key: waves in order
  for (int k = tid; k < kpad; k += kSortThreads) {
    int run = 0;
#pragma unroll
    for (int w = 0; w < kSortWaves; ++w) {
      const int v = s_cnt[w][k];
      s_cnt[w][k] = run;
      run += v;
    }
    s_tot[k] = run;
  }
  __syncthreads();
  // keys in order: every lane of wave 0 owns kpad / 64 consecutive keys
  if (wave == 0) {
    const int kper = kpad / kWave;
    int sum = 0;
    for (int j = 0; j < kper; ++j) sum += s_tot[lane * kper + j];
    int incl = sum;
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
      const int t = __shfl_up(incl, d);
      if (lane >= d) incl += t;
    }
    int run = incl - sum;
    for (int j = 0; j < kper; ++j) {
      const int v = s_tot[lane * kper + j];
      s_tot[lane * kper + j] = run;
      run += v;
    }
    if (lane == kWave - 1) s_tot[kpad] = incl;
  }
  __syncthreads();
  for (int k = lane; k < kpad; k += kWave) s_cnt[wave][k] += base + s_tot[k];
  // per channel and x slab: the run of records whose atoms can reach the slab's x planes; slab_of
  // is monotone, so an atom inside [low plane - reach, high plane + reach] has its slab in range.
  // Keys past the last one hold no atoms, so their start is the end of the last.
  int* const crow = cand + ((size_t)slot * ntypes + c0) * nxs * 2;
  for (int i = tid; i < nkeys; i += kSortThreads) {
    const int c = i / nxs, xs = i - c * nxs;
    const float clx = grid_coord(ox, xs * kColXY, g.resolution);
    const float chx = grid_coord(ox, min(xs * kColXY + kColXY, g.dim) - 1, g.resolution);
    const int s_lo = (int)slab_of(clx - reach, ox, inv_slab, nxs);
    const int s_hi = (int)slab_of(chx + reach, ox, inv_slab, nxs);
    crow[2 * i] = base + s_tot[c * nxs + s_lo];
    crow[2 * i + 1] = base + s_tot[c * nxs + s_hi + 1];
  }
  __syncthreads();
  // scatter, in atom order within (wave, key): the lanes of a round that share a key take
  // consecutive positions from the key's running position
  auto scatter = [&](int key, float x, float y, float z, float ar) {
    const bool act = key >= 0;
    if (!act) key = 0;
    unsigned long long same = __ballot(act);
    if (same == 0) return;
    for (int bit = 0; bit < key_bits; ++bit) {
      const bool set = (key >> bit) & 1;
      const unsigned long long bm = __ballot(act && set);
      same &= set ? bm : ~bm;
    }
    const int leader = act ? (int)__builtin_ctzll(same) : lane;
    int pos = 0;
    if (act && lane == leader) pos = atomicAdd(&s_cnt[wave][key], (int)__popcll(same));
    pos = __shfl(pos, leader);
    if (act) {
      pos += __popcll(same & ((1ull << lane) - 1ull));
      if (pos < capacity) records[pos] = make_float4(x, y, z, ar);
    }
  };
  if (cached) {
#pragma unroll
    for (int k = 0; k < kCached; ++k)
      if (wb + k * kWave < we)                 // uniform over the wave
        scatter(c_key[k], c_x[k], c_y[k], c_z[k], c_r[k]);
  } else {
    for (int a0 = wb; a0 < we; a0 += kWave) {
      const int a = a0 + lane;
      const int ac = a < we ? a : we - 1;
      const float x = coords[3 * ac];
      const float ar = scaled(radii[ac]);
      scatter(a < we ? key_of(types[ac], x, ar) : -3, x, coords[3 * ac + 1], coords[3 * ac + 2], ar);
    }
  }
}

// ------------------------------------------------------------------------------------------
// Launch 2
// ------------------------------------------------------------------------------------------
// Last block at or below `top` and first block at or above `bottom` of a column's blocks
// 0 .. last: -1 and last + 1 when there is none.  The clamps are float operations, so that the
// conversion never sees a value outside the range of int (fminf and fmaxf return the other
// operand for not-a-number: a record with such a coordinate selects every block of the column).
__device__ __forceinline__ int block_below(float top, int last) {
  return (int)fmaxf(fminf(floorf(top), (float)last), -1.f);
}
__device__ __forceinline__ int block_above(float bottom) {
  return (int)fminf(fmaxf(ceilf(bottom), 0.f), 32.f);
}

// CORE (Gaussian density, fast predicates only): the cull also finds, per column, the blocks that
// the Gaussian core of an atom can reach; the blocks of its reach beyond them take the quadratic
// tail without evaluating the exponential.  The same sums bit for bit.
template <bool BINARY, bool EXACT, int COLS, bool PAGED, bool CORE = false>
__global__ __launch_bounds__(PAGED ? kPagedWaves * kWave : kWave) void splat_sorted_kernel(
    GridArg g, const float4* __restrict__ slot_info, const int* __restrict__ cand,
    const float4* __restrict__ records, int capacity, float* __restrict__ out,
    int nxs, int nyp, int nzs, int nranges, int aligned_rows, int slab_z, int nbatch) {
  // one column of one wave (rows padded), or the workgroup's slab of four x planes
  __shared__ __align__(16) float stage[PAGED ? kSlabFloats : kPlane];

  const int lane = threadIdx.x & (kWave - 1);
  const int dim = g.dim;
  const int ntypes = g.ntypes;
  const size_t chan_stride = (size_t)dim * dim * dim;   // the host has checked: < 2^30 floats

  // lane-constant part of the write-out of a column: the 192 float4 pieces of its 16 z rows in
  // memory order (x, y, z), 64 at a time; the four rows of an x follow each other in memory
  const int lx = lane >> 4, ly = (lane >> 2) & 3, lz = lane & 3;
  const int stage_lane = (lx * 4 + ly) * kRowPad + lz;
  int st_lds[kPieces], st_rx[kPieces], st_ry[kPieces], st_z[kPieces];
  unsigned st_rel[kPieces];
#pragma unroll
  for (int k = 0; k < kPieces; ++k) {
    const int p = lane + k * kWave;
    const int r = p / 12, f4 = p - r * 12;
    st_lds[k] = r * kRowPad + f4 * 4;
    st_rx[k] = r >> 2;
    st_ry[k] = r & 3;
    st_z[k] = f4 * 4;
    st_rel[k] = (unsigned)((st_rx[k] * dim + st_ry[k]) * dim + st_z[k]) * 4u;
  }
  float quad_c = g.C;
  keep_in_vgpr(quad_c);
  const float frm2 = uniform(g.frm * g.frm);
  const float grm2 = uniform(g.grm * g.grm);
  const float inv_block = 0.25f / g.resolution;             // blocks per unit length along z
  const __amdgpu_buffer_rsrc_t rec_buf = buffer_of(records, (size_t)capacity * 16);
  auto load_round = [&](int first) -> v4u {
    return __builtin_amdgcn_raw_buffer_load_b128(rec_buf, (int)((unsigned)(first + lane) * 16u), 0, 0);
  };

  // which item: channel range fastest, then the territory, then the example's slot; paged:
  // the x slab fastest, then the channel (consecutive workgroups write consecutive runs of the
  // output), the wave of the workgroup is the pair of columns
  int t = blockIdx.x;
  int range, yp, zs, xs, slot;
  if (PAGED) {
    xs = t % nxs;
    t /= nxs;
    range = t % nranges;
    slot = t / nranges;
    yp = threadIdx.x >> 6;
    zs = 0;
  } else {
    range = t % nranges;
    t /= nranges;
    yp = t % nyp;
    t /= nyp;
    zs = t % nzs;
    t /= nzs;
    xs = t % nxs;
    slot = t / nxs;
  }
  const int nmine = (ntypes - range + nranges - 1) / nranges;   // channels range, range + R, ...
  if (nmine <= 0) return;

  const float4 info = slot_info[slot];
  // (what comes out of the workspace is held inside its bounds, so that a workspace that the sort
  // launch did not fill for these sizes gives wrong grids, not a fault or an endless loop)
  const int e = min(max(__builtin_amdgcn_readfirstlane(__float_as_int(info.w)), 0), nbatch - 1);
  // first and one-past-last candidate record of this lane's channel
  const __amdgpu_buffer_rsrc_t cand_buf =
      buffer_of(cand + (size_t)slot * ntypes * nxs * 2, (size_t)ntypes * nxs * 8);
  const int my_chan = range + lane * nranges;
  v2u se = {0u, 0u};
  if (lane < nmine) se = __builtin_amdgcn_raw_buffer_load_b64(cand_buf, (my_chan * nxs + xs) * 8, 0, 0);
  se.x = min(se.x, (unsigned)capacity);
  se.y = min(se.y, (unsigned)capacity);

  const int x0 = xs * kColXY, y0 = yp * (kColXY * COLS), z0 = zs * slab_z;
  const int zend = min(z0 + slab_z, dim);
  float* const out_e = out + (size_t)e * ntypes * chan_stride;
  const unsigned base_off = (unsigned)((x0 * dim + y0) * dim + z0) * 4u;

  bool st_live[kPieces][COLS];
#pragma unroll
  for (int k = 0; k < kPieces; ++k)
#pragma unroll
    for (int col = 0; col < COLS; ++col)
      st_live[k][col] = x0 + st_rx[k] < dim && y0 + col * kColXY + st_ry[k] < dim && z0 + st_z[k] < zend;

  // One column of one channel -> global memory as z rows, from the stage or as zeros.
  auto store_column = [&](int c, int col, bool from_stage) {
    const __amdgpu_buffer_rsrc_t out_buf = buffer_of(out_e + (size_t)c * chan_stride, chan_stride * 4);
    const unsigned col_off = (unsigned)(col * kColXY * dim) * 4u;
#pragma unroll
    for (int k = 0; k < kPieces; ++k) {
      if (st_live[k][col]) {
        v4f v = {0.f, 0.f, 0.f, 0.f};
        if (from_stage) v = *reinterpret_cast<const v4f*>(stage + st_lds[k]);
        const unsigned off = base_off + col_off + st_rel[k];
        if (aligned_rows && z0 + st_z[k] + 3 < dim) {
          // non-temporal: nothing reads the grids back soon enough to find them in the
          // last-level cache, and without the hint its write-back runs on into the next kernel
          __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, v), out_buf, (int)off, 0, 2);
        } else {
          const float ev[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
          for (int j = 0; j < 4; ++j)
            if (z0 + st_z[k] + j < dim)
              __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, ev[j]), out_buf,
                                                    (int)(off + 4u * j), 0, 0);
        }
      }
    }
  };

  // Paged: the slab of channel c -> global memory, whole 4 KB pages (by their address), a page
  // per wave in four back-to-back stores; from the LDS slab or as zeros.
  auto store_pages = [&](int c, bool from_slab) {
    float* const chan = out_e + (size_t)c * chan_stride;
    const __amdgpu_buffer_rsrc_t out_buf = buffer_of(chan, chan_stride * 4);
    const unsigned plane_bytes = (unsigned)(dim * dim) * 4u;
    const unsigned first = (unsigned)x0 * plane_bytes;                  // of the slab, in the channel
    const unsigned bytes = (unsigned)(min(x0 + kColXY, dim) - x0) * plane_bytes;
    // bytes from the slab's start back to the page boundary at or before it
    const unsigned lead = (unsigned)((reinterpret_cast<uintptr_t>(chan) + first) & (kPageBytes - 1));
    const int npages = (int)((lead + bytes + kPageBytes - 1) / kPageBytes);
    const float inv_pieces = 4.0f / (float)dim, inv_dim = 1.0f / (float)dim;
    // the slab in 16-byte pieces (rows and planes are whole pieces: dim % 4 == 0)
    const v4f* const slab = reinterpret_cast<const v4f*>(stage);
    const int prow4 = paged_row(dim) >> 2, pplane4 = paged_plane(dim) >> 2, dim4 = dim >> 2;
    const unsigned dropped = (unsigned)(chan_stride * 4);               // an offset past the channel
    constexpr int kStores = kPageBytes / (kWave * 16);                  // 4 stores of 1 KB a page
    for (int page = (int)(threadIdx.x >> 6); page < npages; page += (int)(blockDim.x >> 6)) {
      // All four pieces are read from LDS first and then stored by four instructions in a row,
      // none of them in a branch: the memory system takes a page fastest as one burst.  A piece
      // before the slab's first byte or after its last (a page shared with the neighbouring slab)
      // is stored to an offset past the end of the channel, which the hardware drops.
      unsigned off[kStores];
      v4f v[kStores];
#pragma unroll
      for (int k = 0; k < kStores; ++k) {
        // byte of this lane's piece relative to the slab's start
        const int rel = page * kPageBytes + (k * kWave + lane) * 16 - (int)lead;
        const bool mine = rel >= 0 && rel < (int)bytes;
        off[k] = mine ? first + (unsigned)rel : dropped;
        v[k] = v4f{0.f, 0.f, 0.f, 0.f};
        if (from_slab) {
          const int piece = mine ? rel >> 4 : 0;
          const int row = (int)(((float)piece + 0.5f) * inv_pieces);     // piece / (dim / 4)
          const int px = (int)(((float)row + 0.5f) * inv_dim);           // row / dim
          v[k] = slab[px * pplane4 + (row - px * dim) * prow4 + (piece - row * dim4)];
        }
      }
#pragma unroll
      for (int k = 0; k < kStores; ++k)
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, v[k]), out_buf, (int)off[k], 0, 2);
    }
  };

  unsigned long long full = __ballot(lane < nmine && se.y > se.x);    // my channels with atoms
  unsigned long long empty = __ballot(lane < nmine && se.y <= se.x);  // and without
  v4u pre = {0u, 0u, 0u, 0u};
  if (full) pre = load_round(__builtin_amdgcn_readlane((int)se.x, (int)__builtin_ctzll(full)));

  // ---- channels none of whose atoms can reach these x planes: zeros ----------------------------
  while (empty != 0) {
    const int j = __builtin_ctzll(empty);
    empty &= empty - 1ull;
    if (PAGED) {
      store_pages(range + j * nranges, false);
    } else {
#pragma unroll
      for (int col = 0; col < COLS; ++col) store_column(range + j * nranges, col, false);
    }
  }
  if (full == 0) return;

  // ---- geometry of the territory -----------------------------------------------------------------
  const float ox = uniform(info.x), oy = uniform(info.y), oz = uniform(info.z);
  // first/last voxel centre of the territory inside the grid
  const float clx = uniform(grid_coord(ox, x0, g.resolution));
  const float chx = uniform(grid_coord(ox, min(x0 + kColXY, dim) - 1, g.resolution));
  const float clz = uniform(grid_coord(oz, z0, g.resolution));
  float cly[COLS], chy[COLS];
  const int vxi = x0 + lx;
  const float vx = grid_coord(ox, vxi, g.resolution);
  // a voxel outside the grid sits at infinity, where no atom reaches it
  float vy[COLS], vz[kBlocks];
#pragma unroll
  for (int col = 0; col < COLS; ++col) {
    const int cy0 = y0 + col * kColXY;
    cly[col] = uniform(grid_coord(oy, min(cy0, dim - 1), g.resolution));
    chy[col] = uniform(grid_coord(oy, min(cy0 + kColXY, dim) - 1, g.resolution));
    const int vyi = cy0 + ly;
    vy[col] = (vxi < dim && vyi < dim) ? grid_coord(oy, vyi, g.resolution) : INFINITY;
  }
#pragma unroll
  for (int q = 0; q < kBlocks; ++q) {
    const int vzi = z0 + q * 4 + lz;
    vz[q] = vzi < zend ? grid_coord(oz, vzi, g.resolution) : INFINITY;
  }
  const int last_block = (zend - z0 + 3) / 4 - 1;

  // ---- channels with atoms ---------------------------------------------------------------------
  while (full != 0) {
    const int j = __builtin_ctzll(full);
    full &= full - 1ull;
    const int c = range + j * nranges;
    const int lo = __builtin_amdgcn_readlane((int)se.x, j);
    const int hi = __builtin_amdgcn_readlane((int)se.y, j);
    // where the records of my next channel with atoms begin
    const int next_lo = full ? __builtin_amdgcn_readlane((int)se.x, (int)__builtin_ctzll(full)) : lo;

    float acc[COLS][kBlocks];
#pragma unroll
    for (int col = 0; col < COLS; ++col)
#pragma unroll
      for (int q = 0; q < kBlocks; ++q) acc[col][q] = 0.f;
    unsigned touched = 0;                        // columns some record reaches

    // A cull round takes 64 records, one per lane: for every column the lane finds the interval
    // of z the atom can reach inside it (its reach shrunk by the distance to the column's
    // footprint in x and y) and from it the range of blocks, as a bit mask.  The records that
    // reach the territory are then taken one at a time, in record order, each over the blocks
    // of its masks; record and masks come straight from the lane that tested it.
    for (int r0 = lo; r0 < hi; r0 += kWave) {
      const bool valid = r0 + lane < hi;
      const v4u raw = pre;
      pre = load_round(r0 + kWave < hi ? r0 + kWave : next_lo);   // in flight during this round
      const float rec_x = __uint_as_float(raw.x), rec_y = __uint_as_float(raw.y);
      const float rec_z = __uint_as_float(raw.z), rec_ar = __uint_as_float(raw.w);
      float ar2;
      {
#pragma clang fp contract(off)
        ar2 = rec_ar * rec_ar;
      }
      const float rec_w = BINARY ? ar2 : 1.0f / ar2;
      // squared reach, with the slack that keeps the cull a superset of the exact test
      const float reach2 = (BINARY ? ar2 : frm2 * ar2) * kCullSlack;
      const float core2 = grm2 * ar2 * kCullSlack;            // squared radius of the Gaussian core
      const float ex = fmaxf(fmaxf(clx - rec_x, rec_x - chx), 0.f);
      unsigned mask[COLS];
      unsigned any = 0;
#pragma unroll
      for (int col = 0; col < COLS; ++col) {
        const float ey = fmaxf(fmaxf(cly[col] - rec_y, rec_y - chy[col]), 0.f);
        const float rz2 = reach2 - (ex * ex + ey * ey);
        mask[col] = 0;
        if (valid && y0 + col * kColXY < dim && rz2 >= 0.f) {
          const float rz = __builtin_amdgcn_sqrtf(rz2);
          // block q holds the voxel centres clz + (4q .. 4q+3) * resolution
          const float top = (rec_z + rz - clz) * inv_block + 1e-3f;
          const float bottom = (rec_z - rz - clz) * inv_block - (0.75f + 1e-3f);
          // (clamped as floats, so that no record -- huge, infinite, not a number -- reaches the
          // conversion out of range)
          const int qhi = block_below(top, last_block), qlo = block_above(bottom);
          if (qlo <= qhi) mask[col] = (2u << qhi) - (1u << qlo);
          if (CORE) {
            // bits 16..27: the blocks that the Gaussian core of the atom (u <= grm^2) can reach,
            // a subset of the above; the others take the quadratic tail without the exponential
            const float cz2 = core2 - (ex * ex + ey * ey);
            if (cz2 >= 0.f) {
              const float cz = __builtin_amdgcn_sqrtf(cz2);
              const float ctop = (rec_z + cz - clz) * inv_block + 1e-3f;
              const float cbottom = (rec_z - cz - clz) * inv_block - (0.75f + 1e-3f);
              const int chi = block_below(ctop, last_block), clo = block_above(cbottom);
              if (clo <= chi) mask[col] |= (((2u << chi) - (1u << clo)) & mask[col]) << 16;
            }
          }
        }
        any |= mask[col];
      }
      uint3 clip = make_uint3(0, 0, 0);
      if (EXACT) {
        // index box of the CPU loops (src/grid_maker.cpp:181-189)
        float densityrad;
        {
#pragma clang fp contract(off)
          densityrad = rec_ar * g.frm;
        }
        int blo[3], bhi[3];
        bounds_1d(ox, rec_x, densityrad, g.resolution, dim, blo[0], bhi[0]);
        bounds_1d(oy, rec_y, densityrad, g.resolution, dim, blo[1], bhi[1]);
        bounds_1d(oz, rec_z, densityrad, g.resolution, dim, blo[2], bhi[2]);
        clip = make_uint3((unsigned)blo[0] | ((unsigned)bhi[0] << 16),
                          (unsigned)blo[1] | ((unsigned)bhi[1] << 16),
                          (unsigned)blo[2] | ((unsigned)bhi[2] << 16));
      }

      unsigned long long todo = __ballot(any != 0);
#pragma unroll 1
      while (todo != 0) {                        // loses a bit per trip
        const int src = __builtin_ctzll(todo);
        todo &= todo - 1ull;
        const float rx = lane_value(rec_x, src), ry = lane_value(rec_y, src);
        const float rz = lane_value(rec_z, src), rw = lane_value(rec_w, src);
        float rar = 0.f;
        uint3 rclip = make_uint3(0, 0, 0);
        if (EXACT) {
          rar = lane_value(rec_ar, src);
          rclip = make_uint3((unsigned)__builtin_amdgcn_readlane((int)clip.x, src),
                             (unsigned)__builtin_amdgcn_readlane((int)clip.y, src),
                             (unsigned)__builtin_amdgcn_readlane((int)clip.z, src));
        }
        const float dx = vx - rx;
#pragma unroll
        for (int col = 0; col < COLS; ++col) {
          const unsigned both = (unsigned)__builtin_amdgcn_readlane((int)mask[col], src);
          const unsigned reach = CORE ? both & 0xffffu : both, core = both >> 16;
          if (reach == 0) continue;
          touched |= 1u << col;
          const float dy = vy[col] - ry;
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
              if (EXACT) {
                float val;
                const bool inside = inside_clip(vxi, y0 + col * kColXY + ly, z0 + q * 4 + lz, rclip);
                const bool hit = density_hit<BINARY, true>(g, dx, dy, dz, rw, rar, frm2, grm2,
                                                           quad_c, val);
                if (hit && inside) acc[col][q] = BINARY ? 1.0f : acc[col][q] + val;
              } else if (BINARY) {
                float rsq;
                {
#pragma clang fp contract(off)
                  rsq = dxy2 + dz * dz;
                }
                if (rsq < rw) acc[col][q] = 1.0f;
              } else {
                const float u = fmaf(dz, dz, dxy2) * rw;
                if (u <= frm2) {
                  if (CORE) {
                    const float su = __builtin_amdgcn_sqrtf(u);
                    float val = fmaxf(fmaf(g.A, u, fmaf(g.B, su, quad_c)), 0.f);
                    if ((core >> q) & 1u) {        // scalar test: else no voxel of the block
                      keep_branch();
                      const float gauss = __builtin_amdgcn_exp2f(u * kNeg2Log2e);   // is in the core
                      val = (u <= grm2) ? gauss : val;
                    }
                    acc[col][q] += val;
                  } else {
                    const float gauss = __builtin_amdgcn_exp2f(u * kNeg2Log2e);
                    const float su = __builtin_amdgcn_sqrtf(u);
                    const float quad = fmaxf(fmaf(g.A, u, fmaf(g.B, su, quad_c)), 0.f);
                    acc[col][q] += (u <= grm2) ? gauss : quad;
                  }
                }
              }
            }
          }
        }
      }
    }

    if (PAGED) {
      // sums -> the workgroup's slab (every wave its own rows; voxels outside the grid have no
      // place in it), then the slab -> pages.  All waves of the workgroup have the same channels
      // with atoms (one table entry serves them all), so they meet at the barriers.
      const int prow = paged_row(dim), pplane = paged_plane(dim);
#pragma unroll
      for (int col = 0; col < COLS; ++col) {
        const int y = y0 + col * kColXY + ly;
        if (vxi < dim && y < dim) {
          float* const dst = stage + lx * pplane + y * prow + lz;
#pragma unroll
          for (int q = 0; q < kBlocks; ++q)
            if (q * 4 + lz < dim) dst[q * 4] = acc[col][q];
        }
      }
      lds_barrier();
      store_pages(c, true);
      if (full != 0) lds_barrier();            // the slab is written again for the next channel
      continue;
    }
    // write-out, column by column: sums -> the stage -> z rows (or zeros straight away); LDS
    // keeps the order of one wave's accesses, so no barrier is involved
#pragma unroll
    for (int col = 0; col < COLS; ++col) {
      if (y0 + col * kColXY >= dim) break;
      const bool from_stage = (touched >> col) & 1u;
      if (from_stage) {
        wave_lds_fence();                      // the previous column has been read
#pragma unroll
        for (int q = 0; q < kBlocks; ++q) stage[stage_lane + q * 4] = acc[col][q];
        wave_lds_fence();
      }
      store_column(c, col, from_stage);
    }
  }
}

// Whether the paged write-out serves this grid: whole float4 pieces in a row, one z slab, a slab of
// four x planes that fits the LDS.
bool paged_serves(const GridArg& g, const float* out) {
  return g.dim % 4 == 0 && g.dim <= kPagedDim && (reinterpret_cast<uintptr_t>(out) & 15) == 0;
}

template <bool BINARY, bool CORE>
hipError_t launch_splat_paged(const GridArg& g, const SortedAtoms& s, int nbatch, float* out,
                              hipStream_t stream) {
  const int dim = g.dim;
  const int nxs = (dim + kColXY - 1) / kColXY;
  const int nyp = (dim + 2 * kColXY - 1) / (2 * kColXY);      // waves of a workgroup, <= kPagedWaves
  const long long nitems = (long long)nbatch * nxs * g.ntypes;
  if (nitems >= 0x7fffffffll) return hipErrorInvalidValue;
  hipLaunchKernelGGL((splat_sorted_kernel<BINARY, false, 2, true, CORE>), dim3((unsigned)nitems),
                     dim3(nyp * kWave), 0, stream, g, s.slot_info, s.cand, s.records, s.capacity, out,
                     nxs, nyp, 1, g.ntypes, 1, kSlabZ, nbatch);
  return hipGetLastError();
}

template <bool BINARY, bool EXACT, int COLS, bool CORE = false>
hipError_t launch_splat(const GridArg& g, const SortedAtoms& s, int nbatch, float* out,
                        hipStream_t stream) {
  const int dim = g.dim;
  const int nxs = (dim + kColXY - 1) / kColXY;
  const int nyp = (dim + kColXY * COLS - 1) / (kColXY * COLS);
  // Height of a z slab: 48 voxels (all twelve blocks of a column), except for grids of 64, 128,
  // 160 ... voxels a side, which 48 would cut into 48 + 16 -- two waves then write the two parts
  // of every second cache line of a row at different times; 32 voxels are whole 128-byte lines
  // (measured on 28 x 64^3: 0.31 ms against 0.35 ms)
  const int slab_z = (dim > kSlabZ && dim % 32 == 0 && dim % kSlabZ != 0) ? 32 : kSlabZ;
  const int nzs = (dim + slab_z - 1) / slab_z;
  const int nranges = std::max((g.ntypes + kItemChannels - 1) / kItemChannels,
                               (g.ntypes + kItemChannelsMax - 1) / kItemChannelsMax);
  const long long nitems = (long long)nbatch * nxs * nzs * nyp * nranges;
  if (nitems >= 0x7fffffffll) return hipErrorInvalidValue;
  const int aligned = ((dim % 4 == 0) && ((reinterpret_cast<uintptr_t>(out) & 15) == 0)) ? 1 : 0;
  hipLaunchKernelGGL((splat_sorted_kernel<BINARY, EXACT, COLS, false, CORE>), dim3((unsigned)nitems), dim3(kWave),
                     0, stream, g, s.slot_info, s.cand, s.records, s.capacity, out, nxs, nyp, nzs,
                     nranges, aligned, slab_z, nbatch);
  return hipGetLastError();
}

// 1: grids that the paged write-out serves take it
std::atomic<int> g_paged{0};
// 1: Gaussian densities take the kernel instances that skip the exponential for tail-only blocks
std::atomic<int> g_core_skip{0};

}  // namespace

size_t forward_sorted_workspace_bytes(int nbatch, int atoms_per_example, int ntypes, int dim) {
  const long long capacity = (long long)nbatch * atoms_per_example;
  const size_t nkeys = (size_t)ntypes * ((dim + kColXY - 1) / kColXY);
  return align256((size_t)nbatch * 16) + align256((size_t)nbatch * nkeys * 8) +
         (size_t)capacity * 16;
}

// The sizes the two launches address with 32 bits: a channel below 4 GB, the records of the batch
// below 4 GB, the table of (channel, x slab) keys below 2^26 entries.
bool forward_sorted_supports(const GridArg& g, int nbatch, int per_example) {
  const size_t chan_stride = (size_t)g.dim * g.dim * g.dim;
  if (chan_stride * 4 >= 0xfffffff0ull) return false;
  if ((long long)nbatch * per_example * 16 >= 0xfffffff0ll) return false;
  const int nxs = (g.dim + kColXY - 1) / kColXY;
  return (long long)g.ntypes * nxs < (1 << 26);
}

namespace {

// hipErrorInvalidValue = the case is not covered (a channel of 4 GB or more, more records than a
// buffer addresses, a workspace that is too small).
hipError_t sorted_layout(const GridArg& g, int nbatch, int per_example, void* workspace,
                         size_t workspace_bytes, SortedAtoms* s, int* nxs_out) {
  if (!forward_sorted_supports(g, nbatch, per_example)) return hipErrorInvalidValue;
  const long long capacity = (long long)nbatch * per_example;
  if (workspace == nullptr ||
      workspace_bytes < forward_sorted_workspace_bytes(nbatch, per_example, g.ntypes, g.dim))
    return hipErrorInvalidValue;
  const int nxs = (g.dim + kColXY - 1) / kColXY;
  *s = carve(workspace, nbatch, g.ntypes * nxs, capacity);
  *nxs_out = nxs;
  return hipSuccess;
}

}  // namespace

// First launch of the forward pass: the atoms -> sorted records and tables in the workspace.
hipError_t launch_sort_atoms(const GridArg& g, const BatchArg& batch, int nbatch,
                             const Vec3Arg& centers, const float* coords, const float* type_index,
                             const float* radii, bool binary, void* workspace,
                             size_t workspace_bytes, hipStream_t stream) {
  SortedAtoms s;
  int nxs = 0;
  const hipError_t e = sorted_layout(g, nbatch, batch.per_example, workspace, workspace_bytes, &s, &nxs);
  if (e != hipSuccess) return e;
  // channels per workgroup of the sort: a few, and no more keys than it handles
  const int per_part = std::max(1, std::min(kSortChannels, kKeyGroup / nxs));
  const int parts = (g.ntypes + per_part - 1) / per_part;
  hipLaunchKernelGGL(sort_atoms_kernel, dim3((unsigned)(parts * nbatch)), dim3(kSortThreads), 0, stream, g,
                     batch, nbatch, nxs, parts, per_part, binary ? 1.0f : g.frm, centers, coords,
                     type_index, radii, s.slot_info, s.cand, s.records, s.capacity);
  return hipGetLastError();
}

// Second launch: the workspace that launch_sort_atoms filled for the same sizes and the same
// density mode -> the grids.
hipError_t launch_splat_sorted(const GridArg& g, int nbatch, int atoms_per_example, float* out,
                               bool binary, bool exact, void* workspace, size_t workspace_bytes,
                               hipStream_t stream) {
  SortedAtoms s;
  int nxs = 0;
  const hipError_t e = sorted_layout(g, nbatch, atoms_per_example, workspace, workspace_bytes, &s, &nxs);
  if (e != hipSuccess) return e;
  if (exact) {
    if (binary) return launch_splat<true, true, 1>(g, s, nbatch, out, stream);
    return launch_splat<false, true, 1>(g, s, nbatch, out, stream);
  }
  const bool core = !binary && g_core_skip.load(std::memory_order_relaxed) != 0;
  if (g_paged.load(std::memory_order_relaxed) != 0 && paged_serves(g, out)) {
    if (binary) return launch_splat_paged<true, false>(g, s, nbatch, out, stream);
    if (core) return launch_splat_paged<false, true>(g, s, nbatch, out, stream);
    return launch_splat_paged<false, false>(g, s, nbatch, out, stream);
  }
  if (binary) return launch_splat<true, false, 2>(g, s, nbatch, out, stream);
  if (core) return launch_splat<false, false, 2, true>(g, s, nbatch, out, stream);
  return launch_splat<false, false, 2>(g, s, nbatch, out, stream);
}

hipError_t launch_forward_sorted(const GridArg& g, const BatchArg& batch, int nbatch,
                                 const Vec3Arg& centers, const float* coords,
                                 const float* type_index, const float* radii, float* out,
                                 bool binary, bool exact, void* workspace, size_t workspace_bytes,
                                 hipStream_t stream) {
  const hipError_t e = launch_sort_atoms(g, batch, nbatch, centers, coords, type_index, radii, binary,
                                         workspace, workspace_bytes, stream);
  if (e != hipSuccess) return e;
  return launch_splat_sorted(g, nbatch, batch.per_example, out, binary, exact, workspace,
                             workspace_bytes, stream);
}

int set_forward_paged(int on) { return g_paged.exchange(on ? 1 : 0); }
int set_forward_core_skip(int on) { return g_core_skip.exchange(on ? 1 : 0); }

}  // namespace mg
