// Trilinear resampling of a batch of 4-D grids through an inverse rigid
// transform (GridInterpolater::forward, src/grid_interpolater.cpp:16-48).
//
// One thread owns one output voxel: the source position, the eight tap offsets
// and the three weights are worked out once and reused for every channel (the
// reference's GPU path repeats them per channel in separate launches).  Lanes
// run along z, so every channel's store is one contiguous run per wave.  The
// coordinate chain keeps the reference's rounding order; taps outside the input
// grid read as zero (src/grid_interpolater.cu:17-23).
#include "kernels.h"

namespace mg {

namespace {

constexpr int kThreads = 256;

__global__ __launch_bounds__(kThreads) void interpolate_kernel(
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

  float gx, gy, gz;
  {
#pragma clang fp contract(off)
    const float ox = oc.x - p.out_half + (float)i * p.out_resolution;
    const float oy = oc.y - p.out_half + (float)j * p.out_resolution;
    const float oz = oc.z - p.out_half + (float)k * p.out_resolution;
    const float ux = -t.x - c.x, uy = -t.y - c.y, uz = -t.z - c.z;
    const float3 r = quat_rotate(qinv, qinvinv, ox + ux, oy + uy, oz + uz);
    gx = (r.x + c.x - (ic.x - p.in_half)) / p.in_resolution;
    gy = (r.y + c.y - (ic.y - p.in_half)) / p.in_resolution;
    gz = (r.z + c.z - (ic.z - p.in_half)) / p.in_resolution;
  }
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
      const float p000 = m000 ? src[o000] : 0.f, p001 = m001 ? src[o001] : 0.f;
      const float p010 = m010 ? src[o010] : 0.f, p011 = m011 ? src[o011] : 0.f;
      const float p100 = m100 ? src[o100] : 0.f, p101 = m101 ? src[o101] : 0.f;
      const float p110 = m110 ? src[o110] : 0.f, p111 = m111 ? src[o111] : 0.f;
      const float c00 = p000 * (1 - xd) + p100 * xd;
      const float c01 = p001 * (1 - xd) + p101 * xd;
      const float c10 = p010 * (1 - xd) + p110 * xd;
      const float c11 = p011 * (1 - xd) + p111 * xd;
      const float c0 = c00 * (1 - yd) + c10 * yd;
      const float c1 = c01 * (1 - yd) + c11 * yd;
      val = c0 * (1 - zd) + c1 * zd;
    }
    __builtin_nontemporal_store(val, dst);
  }
}

}  // namespace

hipError_t launch_interpolate(const InterpArg& p, int nbatch, const Vec3Arg& in_centers,
                              const float* in, const Vec4Arg& quats, const Vec3Arg& rot_centers,
                              const Vec3Arg& translations, const Vec3Arg& out_centers, float* out,
                              hipStream_t stream) {
  const int out_points = p.out_dim * p.out_dim * p.out_dim;
  dim3 grid((out_points + kThreads - 1) / kThreads, nbatch), block(kThreads);
  hipLaunchKernelGGL(interpolate_kernel, grid, block, 0, stream, p, in_centers, in, quats,
                     rot_centers, translations, out_centers, out);
  return hipGetLastError();
}

}  // namespace mg
