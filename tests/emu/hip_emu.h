// TEST INFRASTRUCTURE -- a host-side emulation of the HIP device model, just wide enough to run the
// library's gfx950 kernels on the CPU: every thread of a workgroup is a fiber, a wave is 64 of
// them, cross-lane operations (ballot, shuffles, readlane, DPP, the 16x16x4 matrix instruction)
// are rendezvous among the live lanes of a wave, __syncthreads is one among the live threads of
// the workgroup, __shared__ is static storage (workgroups run one after the other), buffer
// instructions check their offset against the descriptor's extent (out of range: loads give
// zero, stores are dropped, like the hardware) and against the emulator's allocations (a
// descriptor that covers memory nobody allocated is an error).  Nothing in the product uses this;
// tests compile the product's kernel sources against it to check results, bounds and
// synchronisation without a GPU.
//
// Not modelled: divergence inside a wave around a cross-lane operation (all live lanes of the
// wave must reach it, otherwise the emulator reports a deadlock), memory ordering, timing.
#pragma once

#include <algorithm>
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <cstring>
#include <functional>

// ---- qualifiers -------------------------------------------------------------------------------
#define __global__
#define __device__
#define __host__
#define __forceinline__ inline __attribute__((always_inline))
#define __launch_bounds__(...)
// (all LDS arrays go into one section of the library, which the emulator fills with 0xCB bytes
// before every workgroup: a kernel that reads LDS it has not written sees garbage, as on the
// hardware, not the zeros of static storage or the previous workgroup's leftovers)
#define __shared__ static __attribute__((section("emu_lds")))
#define __align__(n) __attribute__((aligned(n)))
#define __constant__ static const
#define amdgpu_waves_per_eu(...) unused
#define amdgpu_flat_work_group_size(...) unused
#define HIP_DYNAMIC_SHARED(type, var) type* var = static_cast<type*>(emu::dynamic_shared);

// ---- vector types -----------------------------------------------------------------------------
struct float2 { float x, y; };
struct float3 { float x, y, z; };
struct float4 { float x, y, z, w; };
struct int2 { int x, y; };
struct int3 { int x, y, z; };
struct int4 { int x, y, z, w; };
struct uint2 { unsigned x, y; };
struct uint3 { unsigned x, y, z; };
struct uint4 { unsigned x, y, z, w; };
struct dim3 {
  unsigned x, y, z;
  dim3(unsigned x_ = 1, unsigned y_ = 1, unsigned z_ = 1) : x(x_), y(y_), z(z_) {}
};
inline float2 make_float2(float x, float y) { return {x, y}; }
inline float3 make_float3(float x, float y, float z) { return {x, y, z}; }
inline float4 make_float4(float x, float y, float z, float w) { return {x, y, z, w}; }
inline int2 make_int2(int x, int y) { return {x, y}; }
inline int3 make_int3(int x, int y, int z) { return {x, y, z}; }
inline int4 make_int4(int x, int y, int z, int w) { return {x, y, z, w}; }
inline uint2 make_uint2(unsigned x, unsigned y) { return {x, y}; }
inline uint3 make_uint3(unsigned x, unsigned y, unsigned z) { return {x, y, z}; }
inline uint4 make_uint4(unsigned x, unsigned y, unsigned z, unsigned w) { return {x, y, z, w}; }

template <class T> inline T min(T a, T b) { return b < a ? b : a; }
template <class T> inline T max(T a, T b) { return a < b ? b : a; }
inline unsigned min(unsigned a, int b) { return min(a, (unsigned)b); }
inline unsigned min(int a, unsigned b) { return min((unsigned)a, b); }
inline size_t min(size_t a, int b) { return min(a, (size_t)b); }

// ---- host API -----------------------------------------------------------------------------------
typedef void* hipStream_t;
enum hipError_t {
  hipSuccess = 0,
  hipErrorInvalidValue = 1,
  hipErrorOutOfMemory = 2,
  hipErrorInvalidSymbol = 13,
  hipErrorInvalidDevice = 101,
  hipErrorLaunchFailure = 719,
};
enum hipFuncAttribute { hipFuncAttributeMaxDynamicSharedMemorySize = 8 };
#define HIP_SYMBOL(x) (emu::remember(&(x), sizeof(x)))

namespace emu {

struct Ctx {
  uint3 tid, bid;
  dim3 bdim, gdim;
  int lane, wave, linear;
};
extern Ctx* cur;
extern void* dynamic_shared;          // extern __shared__ arrays of the running launch

void launch(dim3 grid, dim3 block, size_t shared_bytes, const std::function<void()>& body,
            const char* name);
hipError_t last_error();
void* allocate(size_t bytes, size_t align = 256);   // guarded: the pages around it are inaccessible
void release(void* p);
bool known(const void* p, size_t bytes);
const void* remember(const void* p, size_t bytes);   // memory of the program itself (a __device__ array)
[[noreturn]] void fail(const char* what);

// rendezvous of the live lanes of the calling lane's wave: every lane deposits `mine`; returns a
// pointer to the 64 deposited values (lanes that have left the kernel hold zero) that stays valid
// until the lane's next rendezvous.  live_mask gets the lanes that took part.
const uint64_t* gather(uint64_t mine, uint64_t* live_mask, const char* what);
void barrier();

struct Rsrc {
  char* base;
  uint32_t bytes;
};
bool buffer_ok(const Rsrc& r, uint32_t offset, uint32_t size, bool store);

}  // namespace emu

#define threadIdx (emu::cur->tid)
#define blockIdx (emu::cur->bid)
#define blockDim (emu::cur->bdim)
#define gridDim (emu::cur->gdim)

inline hipError_t hipGetLastError() { return emu::last_error(); }
inline hipError_t hipGetDevice(int* d) { *d = 0; return hipSuccess; }
inline hipError_t hipMalloc(void** p, size_t n) { *p = emu::allocate(n); return *p ? hipSuccess : hipErrorOutOfMemory; }
template <class T> inline hipError_t hipMalloc(T** p, size_t n) { return hipMalloc((void**)p, n); }
inline hipError_t hipFree(void* p) { emu::release(p); return hipSuccess; }
// (host code of the C++ classes: "device" memory is host memory here)
enum hipMemcpyKind { hipMemcpyHostToHost, hipMemcpyHostToDevice, hipMemcpyDeviceToHost,
                     hipMemcpyDeviceToDevice, hipMemcpyDefault };
inline hipError_t hipMemcpy(void* dst, const void* src, size_t n, hipMemcpyKind) {
  if (n) std::memmove(dst, src, n);
  return hipSuccess;
}
inline hipError_t hipMemset(void* dst, int value, size_t n) {
  if (n) std::memset(dst, value, n);
  return hipSuccess;
}
inline hipError_t hipDeviceSynchronize() { return hipSuccess; }
inline hipError_t hipSetDevice(int d) { return d == 0 ? hipSuccess : hipErrorInvalidDevice; }
inline hipError_t hipGetSymbolAddress(void** p, const void* symbol) { *p = const_cast<void*>(symbol); return hipSuccess; }
inline const char* hipGetErrorString(hipError_t) { return "emulated HIP error"; }
template <class F> inline hipError_t hipFuncSetAttribute(F, hipFuncAttribute, int) { return hipSuccess; }
#define hipLaunchKernelGGL(kernel, grid, block, shared_bytes, stream, ...) \
  emu::launch(dim3(grid), dim3(block), (shared_bytes), [=]() { kernel(__VA_ARGS__); }, #kernel)

// ---- bit casts, math ----------------------------------------------------------------------------
inline float __int_as_float(int v) { float f; std::memcpy(&f, &v, 4); return f; }
inline float __uint_as_float(unsigned v) { float f; std::memcpy(&f, &v, 4); return f; }
inline int __float_as_int(float f) { int v; std::memcpy(&v, &f, 4); return v; }
inline unsigned __float_as_uint(float f) { unsigned v; std::memcpy(&v, &f, 4); return v; }
inline int __double2loint(double d) { uint64_t v; std::memcpy(&v, &d, 8); return (int)(uint32_t)v; }
inline int __double2hiint(double d) { uint64_t v; std::memcpy(&v, &d, 8); return (int)(uint32_t)(v >> 32); }
inline double __hiloint2double(int hi, int lo) {
  const uint64_t v = ((uint64_t)(uint32_t)hi << 32) | (uint32_t)lo;
  double d; std::memcpy(&d, &v, 8); return d;
}
inline int __popcll(unsigned long long v) { return __builtin_popcountll(v); }
inline int __popc(unsigned v) { return __builtin_popcount(v); }
// The hardware's approximate instructions (v_exp_f32, v_sqrt_f32, v_rsq_f32, v_rcp_f32: about one
// unit in the last place) are the exact results here, moved -- when the environment variable
// EMU_APPROX is "up", "down" or "hash" -- by one unit in the last place up, down, or up, down or
// not at all as a hash of the value decides (unbiased and repeatable, like the hardware; "up" and
// "down" bias every term of a sum the same way, which no tolerance on long sums survives):
// whatever a kernel builds on them (culls with a slack, index arithmetic through a
// reciprocal, the bit-exact binary paths, which must not use them at all) has to hold then too.
namespace emu { float approx(float exact); }
inline float __expf(float x) { return emu::approx(expf(x)); }
#define __builtin_amdgcn_exp2f(x) emu::approx(exp2f(x))
#define __builtin_amdgcn_sqrtf(x) emu::approx(sqrtf(x))
#define __builtin_amdgcn_rsqf(x) emu::approx(1.0f / sqrtf(x))
#define __builtin_amdgcn_rcpf(x) emu::approx(1.0f / (x))
#define __builtin_amdgcn_s_setprio(x) ((void)0)
#define __builtin_amdgcn_s_sleep(x) ((void)0)

// ---- atomics (fibers of a workgroup take turns, workgroups run one after the other) ---------------
template <class T> inline T atomicAdd(T* p, T v) { T o = *p; *p = o + v; return o; }
inline unsigned atomicOr(unsigned* p, unsigned v) { unsigned o = *p; *p = o | v; return o; }
inline int atomicOr(int* p, int v) { int o = *p; *p = o | v; return o; }
inline int atomicMax(int* p, int v) { int o = *p; *p = o > v ? o : v; return o; }
inline unsigned atomicMax(unsigned* p, unsigned v) { unsigned o = *p; *p = o > v ? o : v; return o; }

// ---- cross-lane operations ------------------------------------------------------------------------
inline void __syncthreads() { emu::barrier(); }
inline unsigned long long __ballot(int pred) {
  uint64_t live;
  const uint64_t* v = emu::gather(pred ? 1 : 0, &live, "ballot");
  unsigned long long m = 0;
  for (int i = 0; i < 64; ++i)
    if (((live >> i) & 1) && v[i]) m |= 1ull << i;
  return m;
}
namespace emu {
inline uint32_t pick(uint32_t mine, int src, const char* what) {
  uint64_t live;
  const uint64_t* v = gather(mine, &live, what);
  return (uint32_t)v[src & 63];
}
}  // namespace emu
inline int __shfl(int v, int src) { return (int)emu::pick((uint32_t)v, src, "shfl"); }
inline float __shfl(float v, int src) { return __uint_as_float(emu::pick(__float_as_uint(v), src, "shfl")); }
inline int __shfl_xor(int v, int m) { return (int)emu::pick((uint32_t)v, emu::cur->lane ^ m, "shfl_xor"); }
inline float __shfl_xor(float v, int m) { return __uint_as_float(emu::pick(__float_as_uint(v), emu::cur->lane ^ m, "shfl_xor")); }
inline int __shfl_up(int v, int d) { const int l = emu::cur->lane; return (int)emu::pick((uint32_t)v, l >= d ? l - d : l, "shfl_up"); }
inline float __shfl_up(float v, int d) { const int l = emu::cur->lane; return __uint_as_float(emu::pick(__float_as_uint(v), l >= d ? l - d : l, "shfl_up")); }
inline int __shfl_down(int v, int d) { const int l = emu::cur->lane; return (int)emu::pick((uint32_t)v, l + d < 64 ? l + d : l, "shfl_down"); }
inline int emu_readlane(int v, int src) { return (int)emu::pick((uint32_t)v, src, "readlane"); }
inline int emu_readfirstlane(int v) {
  uint64_t live;
  const uint64_t* vals = emu::gather((uint32_t)v, &live, "readfirstlane");
  return (int)(uint32_t)vals[__builtin_ctzll(live)];
}
#define __builtin_amdgcn_readlane(v, src) emu_readlane((v), (src))
#define __builtin_amdgcn_readfirstlane(v) emu_readfirstlane(v)

// DPP: the controls the kernels use (quad_perm, row_mirror, row_half_mirror, row_bcast15/31), with
// row and bank masks; bound_ctrl false: a lane without a source keeps `old`.
inline int emu_update_dpp(int old, int src, int ctrl, int row_mask, int bank_mask, bool) {
  uint64_t live;
  const uint64_t* v = emu::gather((uint32_t)src, &live, "dpp");
  const int l = emu::cur->lane, row = l >> 4, in_row = l & 15;
  if (!((row_mask >> row) & 1) || !((bank_mask >> (in_row >> 2)) & 1)) return old;
  int from = -1;
  if (ctrl >= 0 && ctrl <= 0xFF) from = (l & ~3) | ((ctrl >> (2 * (l & 3))) & 3);       // quad_perm
  else if (ctrl == 0x140) from = (l & ~15) | (15 - in_row);                              // row_mirror
  else if (ctrl == 0x141) from = (l & ~7) | (7 - (l & 7));                               // row_half_mirror
  else if (ctrl == 0x142) from = row > 0 ? (row - 1) * 16 + 15 : -1;                     // row_bcast15
  else if (ctrl == 0x143) from = row >= 2 ? 31 : -1;                                     // row_bcast31
  else emu::fail("DPP control not modelled");
  if (from < 0 || !((live >> from) & 1)) return old;
  return (int)(uint32_t)v[from];
}
#define __builtin_amdgcn_update_dpp(old, src, ctrl, row_mask, bank_mask, bound) \
  emu_update_dpp((old), (src), (ctrl), (row_mask), (bank_mask), (bound))

// v_mfma_f32_16x16x4f32 (one block): D = A(16x4) * B(4x16) + C.  Lane l holds A[l % 16][l / 16],
// B[l / 16][l % 16] and the four values D[4 * (l / 16) + r][l % 16]; the four products of an
// element are added to its running sum one after the other.
typedef float emu_v4f __attribute__((ext_vector_type(4)));
inline emu_v4f emu_mfma_16x16x4(float a, float b, emu_v4f c) {
  uint64_t live;
  const uint64_t packed = ((uint64_t)__float_as_uint(a) << 32) | __float_as_uint(b);
  const uint64_t* v = emu::gather(packed, &live, "mfma");
  const int l = emu::cur->lane, j = l & 15, g = l >> 4;
  emu_v4f d = c;
  for (int r = 0; r < 4; ++r) {
    const int i = 4 * g + r;
    float sum = c[r];
    for (int k = 0; k < 4; ++k) {
      const float av = __uint_as_float((uint32_t)(v[k * 16 + i] >> 32));
      const float bv = __uint_as_float((uint32_t)v[k * 16 + j]);
      sum = fmaf(av, bv, sum);
    }
    d[r] = sum;
  }
  return d;
}
#define __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, cbsz, abid, blgp) emu_mfma_16x16x4((a), (b), (c))

// ---- buffer instructions ----------------------------------------------------------------------------
#define __amdgpu_buffer_rsrc_t emu::Rsrc
#define __builtin_amdgcn_make_buffer_rsrc(p, stride, num, flags) (emu::Rsrc{(char*)(p), (uint32_t)(num)})
typedef unsigned emu_v4u __attribute__((ext_vector_type(4)));
typedef unsigned emu_v2u __attribute__((ext_vector_type(2)));
template <class T> inline T emu_buffer_load(const emu::Rsrc& r, int voffset, int soffset) {
  const uint32_t off = (uint32_t)voffset + (uint32_t)soffset;
  T v;
  std::memset(&v, 0, sizeof(T));
  if (emu::buffer_ok(r, off, sizeof(T), false)) std::memcpy(&v, r.base + off, sizeof(T));
  return v;
}
template <class T> inline void emu_buffer_store(T v, const emu::Rsrc& r, int voffset, int soffset) {
  const uint32_t off = (uint32_t)voffset + (uint32_t)soffset;
  if (emu::buffer_ok(r, off, sizeof(T), true)) std::memcpy(r.base + off, &v, sizeof(T));
}
#define __builtin_amdgcn_raw_buffer_load_b32(r, vo, so, aux) emu_buffer_load<unsigned>((r), (vo), (so))
#define __builtin_amdgcn_raw_buffer_load_b64(r, vo, so, aux) emu_buffer_load<emu_v2u>((r), (vo), (so))
#define __builtin_amdgcn_raw_buffer_load_b128(r, vo, so, aux) emu_buffer_load<emu_v4u>((r), (vo), (so))
#define __builtin_amdgcn_raw_buffer_store_b32(v, r, vo, so, aux) emu_buffer_store<unsigned>((v), (r), (vo), (so))
#define __builtin_amdgcn_raw_buffer_store_b64(v, r, vo, so, aux) emu_buffer_store<emu_v2u>((v), (r), (vo), (so))
#define __builtin_amdgcn_raw_buffer_store_b128(v, r, vo, so, aux) emu_buffer_store<emu_v4u>((v), (r), (vo), (so))

// ---- the three pieces of inline assembly of the kernels (gfx950_asm.h of the product) --------------
#define LIBMOLGRID_AMD_GFX950_ASM_H_
namespace mg {
// 0 * anything = 0, also for infinities and NaNs
inline float mul_legacy(float a, float b) { return (a == 0.f || b == 0.f) ? 0.f : a * b; }
inline void keep_in_vgpr(float&) {}
inline void keep_branch() {}
inline void compute_here(int&) {}
inline void lds_barrier() { emu::barrier(); }
// the lanes of a wave are fibers here and do not run in step: meet
inline void wave_lds_fence() { uint64_t live; (void)emu::gather(0, &live, "wave_lds_fence"); }
}  // namespace mg
