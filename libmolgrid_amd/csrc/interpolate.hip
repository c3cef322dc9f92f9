// Trilinear resampling of a batch of 4-D grids through an inverse rigid transform
// (GridInterpolater::forward, src/grid_interpolater.cpp:16-48).
//
// Main kernel (interpolate_tiled_kernel): one workgroup owns an 8x8x8 tile of output voxels.  The
// tile maps to a rotated cube in the input grid; the workgroup finds that cube's bounding window
// (at most 17^3 voxels), stages the window of one channel at a time into LDS with row-coalesced
// loads (zero outside the input grid, so the taps need no bounds tests), and every thread reads
// its eight taps from LDS.  The source position, tap offsets and weights are computed once per
// output voxel and reused for every channel; while a channel is being interpolated the next
// channel's window is already in flight (double-buffered LDS, one barrier per channel).
// Workgroups are numbered so that all tiles of one example run on the same XCD (they share its
// input through that XCD's L2) and z-neighbouring tiles, which complete each other's cache lines
// in the output, run back to back.
//
// Fallback kernel (interpolate_gather_kernel): one thread per output voxel gathering its taps
// straight from global memory; used when a tile's window would not fit (strong down-sampling).
//
// The coordinate chain keeps the reference's rounding order; taps outside the input grid read as
// zero and integral coordinates get weight zero (src/grid_interpolater.cu:17-58).
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
constexpr int kTileT = 8;                      // output tile side
constexpr int kTileThreads = 512;              // one output voxel per thread
constexpr int kWin = 17;                       // largest staged window side
constexpr int kWinZ = 18;                      // z stride of the window in LDS (even: 8-byte pairs)
constexpr int kWinSize = kWin * kWin * kWinZ;  // floats per buffer
constexpr int kStagePer = (kWin * kWin * kWin + kTileThreads - 1) / kTileThreads;  // 10

__global__ __launch_bounds__(kTileThreads) void interpolate_tiled_kernel(
    InterpArg p, int nbatch, int tiles_per_side, Vec3Arg in_centers, const float* __restrict__ in,
    Vec4Arg quats, Vec3Arg rot_centers, Vec3Arg translations, Vec3Arg out_centers,
    float* __restrict__ out) {
  __shared__ float s_win[2][kWinSize];
  __shared__ float s_lo[3], s_hi[3];

  // workgroup -> (example, tile): consecutive workgroups are dealt round-robin to the 8 XCDs, so
  // example b is pinned to XCD b % 8 and its tiles run there in z-fastest order
  const int tiles = tiles_per_side * tiles_per_side * tiles_per_side;
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int b = (slot / tiles) * 8 + xcd;
  if (b >= nbatch) return;
  const int tile = slot % tiles;
  const int tz = tile % tiles_per_side, ty = (tile / tiles_per_side) % tiles_per_side;
  const int tx = tile / (tiles_per_side * tiles_per_side);

  const int od = p.out_dim, id = p.in_dim;
  const int tid = threadIdx.x;
  const int i = tx * kTileT + (tid >> 6), j = ty * kTileT + ((tid >> 3) & 7), k = tz * kTileT + (tid & 7);
  const bool live = i < od && j < od && k < od;

  const float3 ic = load3(in_centers, b), oc = load3(out_centers, b);
  const float3 c = load3(rot_centers, b), t = load3(translations, b);
  const float4 qinv = quat_inverse(load4(quats, b));
  const float4 qinvinv = quat_inverse(qinv);

  // ---- window of the tile: bounding box of the images of its eight corners -----------------
  if (tid < 8) {
    const int ci = min(tx * kTileT + ((tid >> 2) & 1) * (kTileT - 1), od - 1);
    const int cj = min(ty * kTileT + ((tid >> 1) & 1) * (kTileT - 1), od - 1);
    const int ck = min(tz * kTileT + (tid & 1) * (kTileT - 1), od - 1);
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

  // ---- this thread's taps and weights (channel independent) --------------------------------
  const SourcePoint s = source_point(p, ic, oc, c, t, qinv, qinvinv, min(i, od - 1), min(j, od - 1),
                                     min(k, od - 1));
  const float fx = floorf(s.gx), fy = floorf(s.gy), fz = floorf(s.gz);
  const float xd = s.gx - fx, yd = s.gy - fy, zd = s.gz - fz;
  // window-relative tap position, clamped into the window (a clamped tap is outside the input
  // grid on that side and its neighbours there are zero as well)
  const int wx = min(max((int)fminf(fmaxf(fx, -4.f), (float)id + 4.f) - wlo[0], 0), wn[0] - 2);
  const int wy = min(max((int)fminf(fmaxf(fy, -4.f), (float)id + 4.f) - wlo[1], 0), wn[1] - 2);
  const int wz = min(max((int)fminf(fmaxf(fz, -4.f), (float)id + 4.f) - wlo[2], 0), wn[2] - 2);
  const int tap = (wx * kWin + wy) * kWinZ + wz;

  // ---- staging plan of this thread: up to kStagePer window elements per channel ---------------
  const int wcount = wn[0] * wn[1] * wn[2];
  const int plane = wn[1] * wn[2];
  int st_src[kStagePer];   // offset inside one input channel, or -1 for zero padding / unused
  int st_dst[kStagePer];   // offset inside the LDS window, or -1 when unused
#pragma unroll
  for (int e = 0; e < kStagePer; ++e) {
    const int n = tid + e * kTileThreads;
    st_dst[e] = -1;
    st_src[e] = -1;
    if (n < wcount) {
      const int ex = n / plane, r = n - ex * plane, ey = r / wn[2], ez = r - ey * wn[2];
      st_dst[e] = (ex * kWin + ey) * kWinZ + ez;
      const int gx = wlo[0] + ex, gy = wlo[1] + ey, gz = wlo[2] + ez;
      if (gx >= 0 && gx < id && gy >= 0 && gy < id && gz >= 0 && gz < id)
        st_src[e] = (gx * id + gy) * id + gz;
    }
  }

  const size_t in_chan = (size_t)id * id * id;
  const size_t out_points = (size_t)od * od * od;
  const float* src = in + (size_t)b * p.channels * in_chan;
  float* dst = out + (size_t)b * p.channels * out_points + ((size_t)i * od + j) * od + k;

  float staged[kStagePer];
  auto fetch = [&](const float* chan) {
#pragma unroll
    for (int e = 0; e < kStagePer; ++e) staged[e] = st_src[e] >= 0 ? chan[st_src[e]] : 0.f;
  };
  auto deposit = [&](float* win) {
#pragma unroll
    for (int e = 0; e < kStagePer; ++e)
      if (st_dst[e] >= 0) win[st_dst[e]] = staged[e];
  };

  fetch(src);
  deposit(s_win[0]);
  __syncthreads();
  for (int ch = 0; ch < p.channels; ++ch) {
    const bool more = ch + 1 < p.channels;
    if (more) fetch(src + (size_t)(ch + 1) * in_chan);   // in flight during the interpolation
    const float* w = s_win[ch & 1] + tap;
    const float val = lerp3(w[0], w[1], w[kWinZ], w[kWinZ + 1], w[kWin * kWinZ],
                            w[kWin * kWinZ + 1], w[kWin * kWinZ + kWinZ],
                            w[kWin * kWinZ + kWinZ + 1], xd, yd, zd);
    if (live) dst[(size_t)ch * out_points] = val;
    if (more) deposit(s_win[(ch + 1) & 1]);
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

}  // namespace

hipError_t launch_interpolate(const InterpArg& p, int nbatch, const Vec3Arg& in_centers,
                              const float* in, const Vec4Arg& quats, const Vec3Arg& rot_centers,
                              const Vec3Arg& translations, const Vec3Arg& out_centers, float* out,
                              hipStream_t stream) {
  // A tile of 8 output voxels per side spans 7 * sqrt(3) * (out_res / in_res) input voxels at
  // most; with the two extra taps and the rounding slack it must fit the 17-voxel window.
  const float span = 7.0f * 1.7320508f * (p.out_resolution / p.in_resolution);
  if (span + 4.0f <= (float)kWin) {
    const int tiles_per_side = (p.out_dim + kTileT - 1) / kTileT;
    const int tiles = tiles_per_side * tiles_per_side * tiles_per_side;
    const int groups = (nbatch + 7) / 8;
    hipLaunchKernelGGL(interpolate_tiled_kernel, dim3(groups * tiles * 8), dim3(kTileThreads), 0,
                       stream, p, nbatch, tiles_per_side, in_centers, in, quats, rot_centers,
                       translations, out_centers, out);
    return hipGetLastError();
  }
  const int out_points = p.out_dim * p.out_dim * p.out_dim;
  dim3 grid((out_points + kThreads - 1) / kThreads, nbatch), block(kThreads);
  hipLaunchKernelGGL(interpolate_gather_kernel, grid, block, 0, stream, p, in_centers, in, quats,
                     rot_centers, translations, out_centers, out);
  return hipGetLastError();
}

}  // namespace mg
