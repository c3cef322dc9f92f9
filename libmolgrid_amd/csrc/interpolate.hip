// Trilinear resampling of a batch of 4-D grids through an inverse rigid transform
// (GridInterpolater::forward, src/grid_interpolater.cpp:16-48).
//
// Main kernel (interpolate_tiled_kernel): one workgroup owns an 8x16x16 tile of output voxels (16
// along z, so that its stores are 64-byte pieces; four voxels per thread).  The tile maps to a
// rotated box in the input grid; the workgroup finds that box's bounding window (at most 26^3
// voxels), marks the window positions that some tap of the tile reads (a sixth of the window: the rest of the
// bounding box is never touched; a bit per position, one word per (x, y) row), numbers the marked
// positions in window order, and deals them out evenly to its threads.  Per channel the threads
// stage those positions -- and nothing else -- into an LDS buffer in that order (12 KB instead
// of the 70 KB of the whole window; about 2,850 values for the 2,048 voxels of a tile, 1.4 each,
// where an 8x8x16 tile needs 1.5 each); a position outside the
// input grid is staged as zero (its load lies past the end of the buffer descriptor, which
// returns zero).  Every thread reads its eight taps from the slots it looked up once, the two of
// a row, which are neighbours, with one LDS instruction.  The source position, the tap slots and
// the weights are computed once per output voxel and reused for every channel.  Staging runs two
// channels ahead of the interpolation: two register sets and two LDS buffers, one barrier per
// channel.  Workgroups are numbered so that all tiles of one example run on the same XCD (they
// share its input through that XCD's L2) and z-neighbouring tiles, which complete each other's
// cache lines in the output, run back to back.
//
// Fallback kernel (interpolate_gather_kernel): one thread per output voxel gathering its taps
// straight from global memory; used when a tile's window would not fit (strong down-sampling).
//
// The coordinate chain keeps the reference's rounding order; taps outside the input grid read as
// zero and integral coordinates get weight zero (src/grid_interpolater.cu:17-58).
#include <atomic>

#include "kernels.h"

namespace mg {

namespace {

constexpr int kThreads = 256;  // gather kernel

struct SourcePoint {
  float gx, gy, gz;  // position in input grid coordinates (not rounded)
};

// Where output voxel (i, j, k) comes from, in the reference's float op order:
// grid2cart -> un-translate -> inverse rotation -> cart2grid.
__device__ __forceinline__ SourcePoint source_point(const InterpArg& p, float3 ic, float3 oc,
                                                    float3 c, float3 t, float4 qinv,
                                                    float4 qinvinv, int i, int j, int k) {
#pragma clang fp contract(off)
  const float ox = oc.x - p.out_half + (float)i * p.out_resolution;
  const float oy = oc.y - p.out_half + (float)j * p.out_resolution;
  const float oz = oc.z - p.out_half + (float)k * p.out_resolution;
  const float ux = -t.x - c.x, uy = -t.y - c.y, uz = -t.z - c.z;
  const float3 r = quat_rotate(qinv, qinvinv, ox + ux, oy + uy, oz + uz);
  SourcePoint s;
  s.gx = (r.x + c.x - (ic.x - p.in_half)) / p.in_resolution;
  s.gy = (r.y + c.y - (ic.y - p.in_half)) / p.in_resolution;
  s.gz = (r.z + c.z - (ic.z - p.in_half)) / p.in_resolution;
  return s;
}

__device__ __forceinline__ float lerp3(float p000, float p001, float p010, float p011, float p100,
                                       float p101, float p110, float p111, float xd, float yd,
                                       float zd) {
  const float c00 = p000 * (1 - xd) + p100 * xd;
  const float c01 = p001 * (1 - xd) + p101 * xd;
  const float c10 = p010 * (1 - xd) + p110 * xd;
  const float c11 = p011 * (1 - xd) + p111 * xd;
  const float c0 = c00 * (1 - yd) + c10 * yd;
  const float c1 = c01 * (1 - yd) + c11 * yd;
  return c0 * (1 - zd) + c1 * zd;
}

// ---------------------------------------------------------------------------------------------
struct alignas(4) TapPair { float lo, hi; };   // the taps at z and z + 1: neighbours in a buffer

constexpr int kTileX = 8, kTileY = 16, kTileZ = 16;  // output tile; 16 voxels of z = one 64-byte line
constexpr int kTileThreads = 512;              // four output voxels (x, x + 2, x + 4, x + 6) per thread
constexpr int kTileWaves = kTileThreads / 64;
constexpr int kVox = kTileX * kTileY * kTileZ / kTileThreads;
constexpr int kWin = 26;                       // largest window side (the tile's bounding box in the input)
constexpr int kRows = kWin * kWin;             // (x, y) rows of the window
constexpr int kRowsPad = 704;
constexpr int kRowsPer = (kRows + kTileThreads - 1) / kTileThreads;   // window rows a thread plans: 2
constexpr int kFewRounds = 6;                   // staged elements per thread and channel
constexpr int kSlots = kFewRounds * kTileThreads;   // 3,072: a tile needs 2,830 input voxels on average, 2,940 at
                                               // most over random rotations (more: the gather path below)
constexpr int kBuf = kSlots + 4;               // floats per buffer
// longest image of the tile's diagonal, in units of (out_res / in_res) input voxels
constexpr float kTileDiagonal = 22.339f;       // sqrt(7^2 + 15^2 + 15^2)

__global__ __launch_bounds__(kTileThreads) void interpolate_tiled_kernel(
    InterpArg p, int nbatch, int tiles_x, int tiles_y, int tiles_z, Vec3Arg in_centers,
    const float* __restrict__ in, Vec4Arg quats, Vec3Arg rot_centers, Vec3Arg translations,
    Vec3Arg out_centers, float* __restrict__ out, int gather_only) {
  // Two buffers of staged input values, in plan order (below).  While the plan is made the same
  // memory holds its tables: per window row the z positions in use (a bit mask) and the row's
  // first slot, then the list of source offsets.
  __shared__ __align__(16) float s_buf[2 * kBuf];
  __shared__ float s_lo[3], s_hi[3];
  __shared__ int s_scan[kTileWaves];
  unsigned* const s_rowmask = reinterpret_cast<unsigned*>(s_buf);
  int* const s_rowstart = reinterpret_cast<int*>(s_buf) + kRowsPad;
  int* const s_list = reinterpret_cast<int*>(s_buf) + 2 * kRowsPad;
  static_assert(kBuf * 4 + 4 < 65536, "16-bit byte offsets");
  static_assert(2 * kRowsPad + kSlots <= 2 * kBuf, "the plan's tables fit the buffers");

  // workgroup -> (example, tile): consecutive workgroups are dealt round-robin to the 8 XCDs, so
  // example b is pinned to XCD b % 8 and its tiles run there in z-fastest order
  const int tiles = tiles_x * tiles_y * tiles_z;
  const int xcd = blockIdx.x & 7, slot_id = blockIdx.x >> 3;
  const int b = (slot_id / tiles) * 8 + xcd;
  if (b >= nbatch) return;
  const int tile = slot_id % tiles;
  const int tz = tile % tiles_z, ty = (tile / tiles_z) % tiles_y;
  const int tx = tile / (tiles_z * tiles_y);

  const int od = p.out_dim, id = p.in_dim;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  // 16 consecutive lanes run along z: one store instruction writes whole 64-byte lines
  static_assert(kTileZ == 16 && kTileY == 16 && kTileX * kTileY * kTileZ == kVox * kTileThreads, "thread to voxel map");
  const int i0 = tx * kTileX + (tid >> 8), j = ty * kTileY + ((tid >> 4) & 15), k = tz * kTileZ + (tid & 15);

  const float3 ic = load3(in_centers, b), oc = load3(out_centers, b);
  const float3 c = load3(rot_centers, b), t = load3(translations, b);
  const float4 qinv = quat_inverse(load4(quats, b));
  const float4 qinvinv = quat_inverse(qinv);

  // ---- window of the tile: bounding box of the images of its eight corners -----------------
  for (int r = tid; r < kRowsPad; r += kTileThreads) s_rowmask[r] = 0u;
  {
    // (every group of eight lanes does this, so that the shuffles are not inside a branch;
    // thread 0 publishes the result)
    const int ci = min(tx * kTileX + ((tid >> 2) & 1) * (kTileX - 1), od - 1);
    const int cj = min(ty * kTileY + ((tid >> 1) & 1) * (kTileY - 1), od - 1);
    const int ck = min(tz * kTileZ + (tid & 1) * (kTileZ - 1), od - 1);
    const SourcePoint s = source_point(p, ic, oc, c, t, qinv, qinvinv, ci, cj, ck);
    float lo[3] = {s.gx, s.gy, s.gz}, hi[3] = {s.gx, s.gy, s.gz};
    // min / max over the 8 corner lanes
#pragma unroll
    for (int d = 0; d < 3; ++d) {
#pragma unroll
      for (int m = 1; m < 8; m <<= 1) {
        lo[d] = fminf(lo[d], __shfl_xor(lo[d], m));
        hi[d] = fmaxf(hi[d], __shfl_xor(hi[d], m));
      }
    }
    if (tid == 0) {
      for (int d = 0; d < 3; ++d) { s_lo[d] = lo[d]; s_hi[d] = hi[d]; }
    }
  }
  __syncthreads();
  // first voxel of the window and its extent; the slack keeps every tap of every voxel of the tile
  // inside although interior points are rounded independently of the corners
  int wlo[3], wn[3];
#pragma unroll
  for (int d = 0; d < 3; ++d) {
    const float flo = floorf(s_lo[d] - 1e-3f), fhi = floorf(s_hi[d] + 1e-3f) + 1.f;
    // entirely outside the input: clamp so that the window stays small (it holds zeros only)
    const float clo = fminf(fmaxf(flo, -2.f), (float)id + 1.f);
    const float chi = fminf(fmaxf(fhi, clo + 1.f), clo + (float)(kWin - 1));   // at least two voxels
    wlo[d] = (int)clo;
    wn[d] = (int)chi - (int)clo + 1;
  }

  // ---- this thread's taps and corner weights (channel independent) ---------------------------
  int wpos[kVox];      // window position of the low tap: (x * kWin + y) << 8 | z
  float frac[kVox][3];   // fractional parts of the source position
  bool live[kVox];
#pragma unroll
  for (int v = 0; v < kVox; ++v) {
    const int i = i0 + v * (kTileX / kVox);
    live[v] = i < od && j < od && k < od;
    const SourcePoint s = source_point(p, ic, oc, c, t, qinv, qinvinv, min(i, od - 1),
                                       min(j, od - 1), min(k, od - 1));
    const float fx = floorf(s.gx), fy = floorf(s.gy), fz = floorf(s.gz);
    // fractional parts; an integral coordinate gives weight 0 to the upper tap
    const float xd = s.gx - fx, yd = s.gy - fy, zd = s.gz - fz;
    frac[v][0] = xd;
    frac[v][1] = yd;
    frac[v][2] = zd;
    // window-relative tap position, clamped into the window (a clamped tap is outside the input
    // grid on that side and its neighbours there are zero as well)
    const int wx = min(max((int)fminf(fmaxf(fx, -4.f), (float)id + 4.f) - wlo[0], 0), wn[0] - 2);
    const int wy = min(max((int)fminf(fmaxf(fy, -4.f), (float)id + 4.f) - wlo[1], 0), wn[1] - 2);
    const int wz = min(max((int)fminf(fmaxf(fz, -4.f), (float)id + 4.f) - wlo[2], 0), wn[2] - 2);
    wpos[v] = ((wx * kWin + wy) << 8) | wz;
    // ---- which window positions any voxel of the tile reads: the window is the bounding box of a
    // rotated tile, so most of it is never touched
    if (live[v]) {
      const unsigned bits = 3u << wz;
      const int r = wx * kWin + wy;
      atomicOr(&s_rowmask[r], bits);
      atomicOr(&s_rowmask[r + 1], bits);
      atomicOr(&s_rowmask[r + kWin], bits);
      atomicOr(&s_rowmask[r + kWin + 1], bits);
    }
  }
  __syncthreads();

  // ---- staging plan: the window positions in use and inside the input grid, numbered in window
  // order (row by row, z ascending): slot n of a buffer holds the n-th of them, and thread t stages
  // slots t, t + 512, ...  One thread per row counts the row's positions, a prefix sum over the
  // workgroup gives the row its first slot.
  // (a thread plans the window rows tid, tid + 512, ...: their slots follow each other)
  unsigned zmask[kRowsPer], zinside[kRowsPer];   // positions in use; those inside the input grid
  int row_src[kRowsPer];
  int mine = 0;
#pragma unroll
  for (int u = 0; u < kRowsPer; ++u) {
    const int row = tid + u * kTileThreads;
    zmask[u] = zinside[u] = 0;
    row_src[u] = 0;
    if (row < kRows) {
      const int ex = row / kWin, ey = row - ex * kWin;
      const int gx = wlo[0] + ex, gy = wlo[1] + ey;
      row_src[u] = (gx * id + gy) * id + wlo[2];
      if (ex < wn[0] && ey < wn[1]) {
        zmask[u] = s_rowmask[row];
        const int zl = max(0, -wlo[2]), zh = min(wn[2], id - wlo[2]);   // z positions inside the grid
        if (gx >= 0 && gx < id && gy >= 0 && gy < id && zh > zl)
          zinside[u] = zmask[u] & ((1u << zh) - 1u) & ~((1u << zl) - 1u);
      }
    }
    mine += __popc(zmask[u]);
  }
  int incl = mine;                                         // inclusive scan over the wave
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const int up = __shfl_up(incl, d);
    if (lane >= d) incl += up;
  }
  if (lane == 63) s_scan[wave] = incl;
  __syncthreads();   // wave totals complete; every row has read its marks
  int slot0 = incl - mine, planned = 0;
#pragma unroll
  for (int w = 0; w < kTileWaves; ++w) {
    const int n = s_scan[w];
    slot0 += w < wave ? n : 0;
    planned += n;
  }
  const int rounds_used = (planned + kTileThreads - 1) / kTileThreads;   // uniform
  // (the buffer loads of the main path address one example's input with 32 bits)
  const bool gather = rounds_used > kFewRounds || gather_only ||
                      (size_t)p.channels * id * id * id * sizeof(float) >= 0x7fffffffull;
#pragma unroll
  for (int u = 0; u < kRowsPer; ++u) {
    const int row = tid + u * kTileThreads;
    if (row < kRows) {
      s_rowmask[row] = zmask[u];
      s_rowstart[row] = slot0;
      unsigned m = zmask[u];
      if (!gather) {
        int slot = slot0;
        while (m != 0) {
          const int ez = __builtin_ctz(m);
          m &= m - 1u;
          s_list[slot++] = ((zinside[u] >> ez) & 1u) ? row_src[u] + ez : -1;   // -1: outside, stays zero
        }
      }
      slot0 += __popc(zmask[u]);
    }
  }
  __syncthreads();

  const size_t in_chan = (size_t)id * id * id;
  const size_t out_points = (size_t)od * od * od;
  const float* src = in + (size_t)b * p.channels * in_chan;
  const size_t vox_step = (size_t)(kTileX / kVox) * od * od;
  const int C = p.channels;

  if (gather) {
    // More positions than the buffers hold.  The launcher sends only resolution ratios here for
    // which a tile needs fewer input voxels than the buffers hold, so this is a safety net (and a test hook):
    // every thread gathers its taps from global memory, with the weights and the order of the
    // sums of the main path.
    float* dst = out + (size_t)b * C * out_points + ((size_t)i0 * od + j) * od + k;
#pragma unroll
    for (int v = 0; v < kVox; ++v) {
      if (!live[v]) continue;
      const int wx = (wpos[v] >> 8) / kWin, wy = (wpos[v] >> 8) - wx * kWin, wz = wpos[v] & 255;
      int o[8];
      bool ok[8];
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        const int gx = wlo[0] + wx + (q >> 2), gy = wlo[1] + wy + ((q >> 1) & 1), gz = wlo[2] + wz + (q & 1);
        ok[q] = gx >= 0 && gx < id && gy >= 0 && gy < id && gz >= 0 && gz < id;
        o[q] = ok[q] ? (gx * id + gy) * id + gz : 0;
      }
      for (int ch = 0; ch < C; ++ch) {
        const float* chan = src + (size_t)ch * in_chan;
        float t8[8];
#pragma unroll
        for (int q = 0; q < 8; ++q) t8[q] = ok[q] ? chan[o[q]] : 0.f;
        dst[(size_t)ch * out_points + v * vox_step] =
            lerp3(t8[0], t8[1], t8[2], t8[3], t8[4], t8[5], t8[6], t8[7], frac[v][0], frac[v][1], frac[v][2]);
      }
    }
    return;
  }

  // ---- slots of this thread's taps (byte offsets inside a buffer; the zero cell for a tap that
  // lies outside the input grid), and the sources of the slots it stages
  // The taps at z and z + 1 of a row are both in use (this voxel marked them), so they sit in
  // consecutive slots: one byte offset per (x, y) row of the voxel, two 16-bit offsets a register.
  unsigned tap_off[kVox][2];
#pragma unroll
  for (int v = 0; v < kVox; ++v) {
    const int r0 = wpos[v] >> 8, wz = wpos[v] & 255;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int r = r0 + (q >> 1) * kWin + (q & 1);
      const unsigned m = s_rowmask[r];
      const int slot = s_rowstart[r] + __popc(m & ((1u << wz) - 1u));
      // (a voxel outside the output grid marked nothing: its offsets stay inside the buffer and
      // its values are dropped)
      const unsigned off = (unsigned)min(slot, kSlots - 2) * 4u;
      if (q & 1) tap_off[v][q >> 1] |= off << 16;
      else tap_off[v][q >> 1] = off;
    }
  }
  int st_src[kFewRounds];   // byte offset inside one input channel
#pragma unroll
  for (int e = 0; e < kFewRounds; ++e) {
    const int slot = tid + e * kTileThreads;
    // a position outside the input grid, or a slot past the plan, is an offset past the end of the
    // descriptor below: the load returns zero without touching memory
    const int src_elem = slot < planned ? s_list[slot] : -1;
    st_src[e] = src_elem >= 0 ? src_elem * 4 : 0x7ffffff0;
  }
  __syncthreads();   // the tables have been read: the buffers can be filled

  // Two register sets, so that the loads of a channel are issued a whole channel before they are
  // needed: while channel ch is interpolated from one buffer, channel ch + 1 is written to the
  // other and channel ch + 2 is in flight.  Every load and store of the loop is issued
  // unconditionally -- slots past the plan stage element 0, voxels outside the output grid store
  // through a buffer descriptor to an offset past its end, which the hardware drops -- because
  // loads and stores share one in-order counter: only with a fixed number of them per iteration
  // can a wait for channel ch + 1 leave the loads of channel ch + 2 and the stores of channel ch
  // in flight.
  float ra[kFewRounds], rb[kFewRounds];
  // (buffer loads: the channel's offset is a scalar operand, the slot's source a 32-bit offset)
  const __amdgpu_buffer_rsrc_t in_buf = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<float*>(src), 0, (int)((size_t)C * in_chan * sizeof(float)), 0x00020000);
  auto fetch = [&](float (&r)[kFewRounds], int ch) {
    const int chan_off = __builtin_amdgcn_readfirstlane((int)((size_t)ch * in_chan * sizeof(float)));
#pragma unroll
    for (int e = 0; e < kFewRounds; ++e)
      r[e] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(in_buf, st_src[e], chan_off, 0));
  };
  auto deposit = [&](const float (&r)[kFewRounds], int ch) {
    float* buf = s_buf + (ch & 1) * kBuf + tid;
#pragma unroll
    for (int e = 0; e < kFewRounds; ++e) buf[e * kTileThreads] = r[e];
  };
  const size_t out_bytes = (size_t)C * out_points * sizeof(float);
  const bool buffered = out_bytes < 0x7fffffffull;
  const __amdgpu_buffer_rsrc_t out_buf = __builtin_amdgcn_make_buffer_rsrc(
      out + (size_t)b * C * out_points, 0, buffered ? (int)out_bytes : 0, 0x00020000);
  float* const dst = out + (size_t)b * C * out_points + ((size_t)i0 * od + j) * od + k;
  unsigned off[kVox];
#pragma unroll
  for (int v = 0; v < kVox; ++v)
    off[v] = live[v] ? (unsigned)((((size_t)i0 * od + j) * od + k + v * vox_step) * sizeof(float))
                     : (unsigned)out_bytes;            // past the end for every channel
  auto interpolate_channel = [&](int ch, int which) {
    const char* buf = reinterpret_cast<const char*>(s_buf + which * kBuf);
    const unsigned chan_off = (unsigned)((size_t)ch * out_points * sizeof(float));
#pragma unroll
    for (int v = 0; v < kVox; ++v) {
      float t8[8];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const unsigned off = (q & 1) ? tap_off[v][q >> 1] >> 16 : tap_off[v][q >> 1] & 0xffffu;
        const TapPair pair = *reinterpret_cast<const TapPair*>(buf + off);   // one ds_read2_b32
        t8[2 * q] = pair.lo;
        t8[2 * q + 1] = pair.hi;
      }
      const float val = lerp3(t8[0], t8[1], t8[2], t8[3], t8[4], t8[5], t8[6], t8[7], frac[v][0],
                              frac[v][1], frac[v][2]);
      if (buffered)
        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, val), out_buf,
                                              (int)(off[v] + chan_off), 0, 0);
      else if (live[v])   // grids of 2 GB or more per example
        dst[(size_t)ch * out_points + v * vox_step] = val;
    }
  };
  fetch(ra, 0);
  deposit(ra, 0);
  fetch(ra, C > 1 ? 1 : 0);
  __syncthreads();
  for (int ch = 0; ch < C; ch += 2) {
    fetch(rb, ch + 2 < C ? ch + 2 : ch);
    if (ch + 1 < C) deposit(ra, ch + 1);
    interpolate_channel(ch, 0);
    __syncthreads();
    if (ch + 1 >= C) break;
    fetch(ra, ch + 3 < C ? ch + 3 : ch);
    if (ch + 2 < C) deposit(rb, ch + 2);
    interpolate_channel(ch + 1, 1);
    __syncthreads();
  }
}

// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(kThreads) void interpolate_gather_kernel(
    InterpArg p, Vec3Arg in_centers, const float* __restrict__ in, Vec4Arg quats,
    Vec3Arg rot_centers, Vec3Arg translations, Vec3Arg out_centers, float* __restrict__ out) {
  const int b = blockIdx.y;
  const int od = p.out_dim, id = p.in_dim;
  const int out_points = od * od * od;
  const int n = blockIdx.x * kThreads + threadIdx.x;
  if (n >= out_points) return;
  const int k = n % od;
  const int j = (n / od) % od;
  const int i = n / (od * od);

  const float3 ic = load3(in_centers, b), oc = load3(out_centers, b);
  const float3 c = load3(rot_centers, b), t = load3(translations, b);
  const float4 qinv = quat_inverse(load4(quats, b));
  const float4 qinvinv = quat_inverse(qinv);
  const SourcePoint s = source_point(p, ic, oc, c, t, qinv, qinvinv, i, j, k);
  const float gx = s.gx, gy = s.gy, gz = s.gz;

  const float fxl = floorf(gx), fyl = floorf(gy), fzl = floorf(gz);
  const float fxh = ceilf(gx), fyh = ceilf(gy), fzh = ceilf(gz);
  // weights are zero when the coordinate is integral (high == low)
  const float xd = fxh > fxl ? (gx - fxl) / (fxh - fxl) : 0.f;
  const float yd = fyh > fyl ? (gy - fyl) / (fyh - fyl) : 0.f;
  const float zd = fzh > fzl ? (gz - fzl) / (fzh - fzl) : 0.f;

  // clamp before the int conversion so that far-away points cannot overflow
  const float lim = (float)id + 1.f;
  const int xl = (int)fminf(fmaxf(fxl, -2.f), lim), xh = (int)fminf(fmaxf(fxh, -2.f), lim);
  const int yl = (int)fminf(fmaxf(fyl, -2.f), lim), yh = (int)fminf(fmaxf(fyh, -2.f), lim);
  const int zl = (int)fminf(fmaxf(fzl, -2.f), lim), zh = (int)fminf(fmaxf(fzh, -2.f), lim);
  const bool vxl = xl >= 0 && xl < id, vxh = xh >= 0 && xh < id;
  const bool vyl = yl >= 0 && yl < id, vyh = yh >= 0 && yh < id;
  const bool vzl = zl >= 0 && zl < id, vzh = zh >= 0 && zh < id;
  const int o000 = (xl * id + yl) * id + zl, o001 = (xl * id + yl) * id + zh;
  const int o010 = (xl * id + yh) * id + zl, o011 = (xl * id + yh) * id + zh;
  const int o100 = (xh * id + yl) * id + zl, o101 = (xh * id + yl) * id + zh;
  const int o110 = (xh * id + yh) * id + zl, o111 = (xh * id + yh) * id + zh;
  const bool m000 = vxl && vyl && vzl, m001 = vxl && vyl && vzh;
  const bool m010 = vxl && vyh && vzl, m011 = vxl && vyh && vzh;
  const bool m100 = vxh && vyl && vzl, m101 = vxh && vyl && vzh;
  const bool m110 = vxh && vyh && vzl, m111 = vxh && vyh && vzh;
  const bool any = m000 || m001 || m010 || m011 || m100 || m101 || m110 || m111;

  const size_t in_chan = (size_t)id * id * id;
  const float* src = in + (size_t)b * p.channels * in_chan;
  float* dst = out + (size_t)b * p.channels * out_points + n;
  for (int ch = 0; ch < p.channels; ++ch, src += in_chan, dst += out_points) {
    float val = 0.f;
    if (any) {
      val = lerp3(m000 ? src[o000] : 0.f, m001 ? src[o001] : 0.f, m010 ? src[o010] : 0.f,
                  m011 ? src[o011] : 0.f, m100 ? src[o100] : 0.f, m101 ? src[o101] : 0.f,
                  m110 ? src[o110] : 0.f, m111 ? src[o111] : 0.f, xd, yd, zd);
    }
    __builtin_nontemporal_store(val, dst);
  }
}

std::atomic<int> g_force_gather{0};

}  // namespace

int set_interpolate_force_gather(int on) { return g_force_gather.exchange(on != 0 ? 1 : 0); }

hipError_t launch_interpolate(const InterpArg& p, int nbatch, const Vec3Arg& in_centers,
                              const float* in, const Vec4Arg& quats, const Vec3Arg& rot_centers,
                              const Vec3Arg& translations, const Vec3Arg& out_centers, float* out,
                              hipStream_t stream) {
  // The image of an 8 x 16 x 16 output tile spans at most kTileDiagonal * (out_res / in_res) input
  // voxels along an axis; with the two extra taps and the rounding slack it must fit the window.
  const float span = kTileDiagonal * (p.out_resolution / p.in_resolution);
  if (span + 3.0f <= (float)kWin) {
    const int tiles_x = (p.out_dim + kTileX - 1) / kTileX;
    const int tiles_y = (p.out_dim + kTileY - 1) / kTileY;
    const int tiles_z = (p.out_dim + kTileZ - 1) / kTileZ;
    const int tiles = tiles_x * tiles_y * tiles_z;
    const int groups = (nbatch + 7) / 8;
    // test hook: every tile takes the gather path (otherwise only a safety net)
    const int gather_only = g_force_gather.load();
    hipLaunchKernelGGL(interpolate_tiled_kernel, dim3(groups * tiles * 8), dim3(kTileThreads), 0,
                       stream, p, nbatch, tiles_x, tiles_y, tiles_z, in_centers, in, quats, rot_centers,
                       translations, out_centers, out, gather_only);
    return hipGetLastError();
  }
  const int out_points = p.out_dim * p.out_dim * p.out_dim;
  dim3 grid((out_points + kThreads - 1) / kThreads, nbatch), block(kThreads);
  hipLaunchKernelGGL(interpolate_gather_kernel, grid, block, 0, stream, p, in_centers, in, quats,
                     rot_centers, translations, out_centers, out);
  return hipGetLastError();
}

}  // namespace mg
