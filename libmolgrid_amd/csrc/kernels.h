// Host-callable launchers of the gfx950 kernels (internal to the library; the
// public surface is the C ABI in include/molgrid_hip.h).
#ifndef LIBMOLGRID_AMD_KERNELS_H_
#define LIBMOLGRID_AMD_KERNELS_H_

#include <hip/hip_runtime.h>

#include "device_common.h"

namespace mg {

// Channels whose accumulators one workgroup keeps in LDS at a time
// (32 * 512 voxels * 4 B = 64 KiB); grids with more channels take several
// passes over the atom list.
constexpr int kMaxChannelGroup = 32;

struct InterpArg {
  float in_resolution, out_resolution;
  float in_half, out_half;  // (float)(dimension / 2.0)
  int in_dim, out_dim;
  int channels;
};

hipError_t launch_transform(const BatchArg& batch, int nbatch, int launch_atoms,
                            const Vec4Arg& quats, const Vec3Arg& centers,
                            const Vec3Arg& translations, bool dotranslate, bool inverse,
                            const float* in, float* out, hipStream_t stream);

// GridMaker::forward, index types, through sorted atom records (forward_sorted.hip): two launches,
// a workspace of forward_sorted_workspace_bytes() in device memory.  hipErrorInvalidValue = the
// case is not covered (a channel of 4 GB or more, more than 2^28 atom slots) or the workspace is
// too small.
size_t forward_sorted_workspace_bytes(int nbatch, int atoms_per_example, int ntypes, int dim);
hipError_t launch_forward_sorted(const GridArg& g, const BatchArg& batch, int nbatch,
                                 const Vec3Arg& centers, const float* coords,
                                 const float* type_index, const float* radii, float* out,
                                 bool binary, bool exact, void* workspace, size_t workspace_bytes,
                                 hipStream_t stream);

// The two launches of launch_forward_sorted on their own, for callers that enqueue them apart
// (the sort on another stream, beside other work): the splat launch needs the workspace the sort
// launch filled for the same nbatch, atoms_per_example, ntypes, grid and density mode.
hipError_t launch_sort_atoms(const GridArg& g, const BatchArg& batch, int nbatch,
                             const Vec3Arg& centers, const float* coords, const float* type_index,
                             const float* radii, bool binary, void* workspace,
                             size_t workspace_bytes, hipStream_t stream);
hipError_t launch_splat_sorted(const GridArg& g, int nbatch, int atoms_per_example, float* out,
                               bool binary, bool exact, void* workspace, size_t workspace_bytes,
                               hipStream_t stream);

// Which write-out the splat launch uses for grids of up to 48 voxels a side with rows of whole
// float4 pieces: 1 = workgroups that own a slab of four x planes of one channel and write it as
// whole 4 KB pages, 0 = one wave per territory writing its own rows.  Same grids bit for bit.
// Returns the previous setting.
bool forward_sorted_supports(const GridArg& g, int nbatch, int per_example);
int set_forward_paged(int on);
int set_forward_core_skip(int on);

// vector types with per-atom radii, density mode, on the matrix cores (forward_vector_mfma.hip)
// `workspace` (optional, forward_vector_workspace_bytes()): a launch before the splat leaves the
// atoms that can reach each slab of four x planes there, and the splat's workgroups scan their
// slab's list instead of every atom of their example.  Same grids either way.
size_t forward_vector_workspace_bytes(int nbatch, int atoms_per_example, int dim);
hipError_t launch_forward_vector_mfma(const GridArg& g, const BatchArg& batch, int nbatch,
                                      const Vec3Arg& centers, const float* coords,
                                      const float* type_vector, const float* radii, float* out,
                                      bool binary, void* workspace, size_t workspace_bytes,
                                      hipStream_t stream);

hipError_t launch_forward_vector(const GridArg& g, const BatchArg& batch, int nbatch,
                                 const Vec3Arg& centers, const float* coords,
                                 const float* type_vector, const float* radii, float* out,
                                 bool binary, bool radii_type_indexed, bool exact,
                                 void* workspace, size_t workspace_bytes, hipStream_t stream);

hipError_t launch_backward_index(const GridArg& g, const BatchArg& batch, int nbatch,
                                 int launch_atoms, const Vec3Arg& centers, const float* coords,
                                 const float* type_index, const float* radii, const float* diff,
                                 float* atom_gradients, hipStream_t stream);

// the same, followed by Transform::backward(gradients, dotranslate = false) per example
hipError_t launch_backward_index_unrotated(const GridArg& g, const BatchArg& batch, int nbatch,
                                           int launch_atoms, const Vec3Arg& centers,
                                           const float* coords, const float* type_index,
                                           const float* radii, const float* diff,
                                           const Vec4Arg& quats, const Vec3Arg& rot_centers,
                                           float* atom_gradients, hipStream_t stream);

hipError_t launch_backward_vector(const GridArg& g, const BatchArg& batch, int nbatch,
                                  int launch_atoms, const Vec3Arg& centers, const float* coords,
                                  const float* type_vector, const float* radii, const float* diff,
                                  float* atom_gradients, float* type_gradients, bool binary,
                                  bool radii_type_indexed, hipStream_t stream);

hipError_t launch_backward_relevance(const GridArg& g, const BatchArg& batch, int nbatch,
                                     int launch_atoms, const Vec3Arg& centers, const float* coords,
                                     const float* type_index, const float* radii,
                                     const float* density, const float* diff, float* relevance,
                                     bool binary, hipStream_t stream);

hipError_t launch_backward_gradients(const GridArg& g, const BatchArg& batch, int nbatch,
                                     int launch_atoms, const Vec3Arg& centers,
                                     const float* coords, const float* type_vector,
                                     const float* radii, const float* diff,
                                     const float* atom_gradients, const float* type_gradients,
                                     float* diffdiff, float* atom_diffdiff, float* type_diffdiff,
                                     bool radii_type_indexed, hipStream_t stream);

// Test hook: 1 makes every tile of the tiled resampling kernel gather its taps from global memory
// (normally a safety net); returns the previous setting.
int set_interpolate_force_gather(int on);

hipError_t launch_interpolate(const InterpArg& p, int nbatch, const Vec3Arg& in_centers,
                              const float* in, const Vec4Arg& quats, const Vec3Arg& rot_centers,
                              const Vec3Arg& translations, const Vec3Arg& out_centers, float* out,
                              hipStream_t stream);

// float <-> double copies (convert.hip)
hipError_t launch_widen(const float* src, double* dst, size_t n, hipStream_t stream);
hipError_t launch_narrow(const double* src, float* dst, size_t n, hipStream_t stream);

}  // namespace mg

#endif
