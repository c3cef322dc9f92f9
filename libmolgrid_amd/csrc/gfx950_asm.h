// The inline assembly of the gfx950 kernels, in one place.
#ifndef LIBMOLGRID_AMD_GFX950_ASM_H_
#define LIBMOLGRID_AMD_GFX950_ASM_H_

#include <hip/hip_runtime.h>

namespace mg {

// a * b with 0 * anything = 0 (also infinities and NaNs): v_mul_legacy_f32
__device__ __forceinline__ float mul_legacy(float a, float b) {
  float r;
  asm("v_mul_legacy_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}

// keeps a wave-uniform value in a vector register (an fma takes one scalar operand)
__device__ __forceinline__ void keep_in_vgpr(float& v) { asm volatile("" : "+v"(v)); }

// The same for an integer, used the other way round: what is computed from the value after this
// point cannot be moved in front of it (out of a loop, where it would occupy registers -- or
// scratch memory -- for the whole loop).
__device__ __forceinline__ void compute_here(int& v) { asm volatile("" : "+v"(v)); }

// workgroup barrier that waits for the wave's LDS traffic only (not for its global loads and
// stores, which __syncthreads would also wait for)
__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// Inside a branch on a scalar condition: keeps the compiler from turning the branch into
// unconditional code plus a select (it would for a few cheap-looking instructions, among them the
// transcendental ones this is used to skip).
__device__ __forceinline__ void keep_branch() { asm volatile(""); }

// Between the LDS writes of a wave and its own reads of what other lanes wrote (and the other
// way round).  The lanes of a wave execute an instruction together and the LDS keeps the order of
// a wave's accesses, so the hardware needs no instruction here; this only keeps the compiler from
// moving LDS accesses across the point.
__device__ __forceinline__ void wave_lds_fence() { __builtin_amdgcn_wave_barrier(); }

}  // namespace mg

#endif
