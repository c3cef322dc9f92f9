/*
 * molgrid_hip.h -- C ABI of the MI355X (gfx950) gridding kernels.
 *
 * This is the drop-in boundary of the gridding hot path: the host-side
 * GridMaker / Transform / GridInterpolater classes (C++ and Python) validate
 * their arguments exactly as the reference does and then call one of these
 * entry points where the reference launched its CUDA kernels.  Signatures use
 * plain pointers and sizes only.
 *
 * Conventions
 *   - Every array pointer is a DEVICE pointer on the current HIP device unless
 *     its name ends in `_host`.  Arrays are dense, row-major, float32.
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream).  Work
 *     is enqueued asynchronously; no entry point synchronises, and none allocates
 *     except mg_forward_index (see there).
 *   - Batches: example b owns atoms [atom_offsets[b], atom_offsets[b+1]) of the
 *     packed atom arrays, and `atoms_per_example` must then be at least the size
 *     of the largest example (it sizes launches and workspaces); 0 means "no
 *     atoms at all" for every entry point (offsets and atom arrays are then not
 *     looked at and may be NULL), a negative value is rejected.  When
 *     `atom_offsets` is NULL every example owns `atoms_per_example` consecutive
 *     atoms (the reference's padded BxN layout,
 *     include/libmolgrid/grid_maker.h:265-301; nbatch = 1 is the un-batched
 *     call).  Per-example float3/float4 parameters (`centers`, `quats`, ...)
 *     are device arrays with one row per example; when such a pointer is NULL
 *     the `_host` value beside it is used for every example.
 *   - Return value: MG_OK, a negative MG_ERR_* code for a rejected argument
 *     (nothing was launched), or a positive hipError_t from the launch.
 *   - Atoms with a negative type index are ignored.  A type index >= ntypes is
 *     ignored as well (the reference's CPU overload throws std::out_of_range,
 *     src/grid_maker.cpp:172; its GPU kernel silently skips, and a kernel
 *     cannot throw): callers that need the exception check on the host.
 */
#ifndef MOLGRID_HIP_H_
#define MOLGRID_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
  MG_OK = 0,
  MG_ERR_INVALID_ARGUMENT = -1, /* reference: std::invalid_argument */
  MG_ERR_OUT_OF_RANGE = -2,     /* reference: std::out_of_range */
  MG_ERR_UNSUPPORTED = -3,
  MG_ERR_NULL_POINTER = -4
};

/* Scalar state of a GridMaker; replaces the by-value `GridMaker G` kernel
 * argument of the reference (src/grid_maker.cu:212-215) and holds the members
 * declared in include/libmolgrid/grid_maker.h:35-48. */
typedef struct mg_gridmaker {
  float resolution;
  float dimension;
  float radius_scale;
  float gaussian_radius_multiple;
  float final_radius_multiple;
  float A, B, C; /* quadratic tail of the density */
  float D, E;    /* its derivative */
  int32_t binary;
  int32_t radii_type_indexed;
  uint32_t dim; /* points per grid side */
} mg_gridmaker;

/* Host only.  Replaces GridMaker::initialize (src/grid_maker.cpp:15-36) and the
 * constructor (include/libmolgrid/grid_maker.h:70-74). */
int mg_gridmaker_init(mg_gridmaker* g, float resolution, float dimension, int binary,
                      int radii_type_indexed, float radius_scale,
                      float gaussian_radius_multiple);

/* Human readable text for a return code of this library. */
const char* mg_error_string(int code);

/* Library version (major*10000 + minor*100 + patch). */
int mg_version(void);

/* No counterpart in the reference (which has no tracing, only -lineinfo,
 * CMakeLists.txt:74).  on != 0: every entry point that launches kernels wraps
 * its work in a roctx range named after itself (roctxRangePushA / roctxRangePop
 * of libroctx64.so, looked up at run time), so that a rocprofv3 marker trace
 * shows which call a kernel belongs to.  Returns the previous setting, or
 * MG_ERR_UNSUPPORTED when the marker library cannot be loaded.  Process-wide;
 * off by default. */
int mg_trace_ranges(int on);

/* Transform::forward on device coordinates; replaces
 * transform_forward_kernel + its launcher (src/transform.cu:13-32, 66-75).
 * out = rotate_q(in - center) + center + translation; `dotranslate` = 0 drops
 * the translation but still rotates about center.  in == out is allowed. */
int mg_transform_forward(int nbatch, const int32_t* atom_offsets, int atoms_per_example,
                         const float* quats, const float quat_host[4],
                         const float* centers, const float center_host[3],
                         const float* translations, const float translation_host[3],
                         int dotranslate, const float* in_coords, float* out_coords,
                         void* stream);

/* Transform::backward on device coordinates; replaces
 * transform_translate_kernel / transform_rotate_kernel and their launcher
 * (src/transform.cu:35-62, 79-93) with the CPU overload's arithmetic
 * (src/transform.cpp:85-108): out = rotate_{q^-1}(in - translation - center) + center. */
int mg_transform_backward(int nbatch, const int32_t* atom_offsets, int atoms_per_example,
                          const float* quats, const float quat_host[4],
                          const float* centers, const float center_host[3],
                          const float* translations, const float translation_host[3],
                          int dotranslate, const float* in_coords, float* out_coords,
                          void* stream);

/* GridMaker::forward, index types; replaces the cudaMemset + forward_gpu launch
 * per example (src/grid_maker.cu:212-289) for a whole batch, with the values of
 * the CPU overload (src/grid_maker.cpp:153-212).
 *   coords [n,3], type_index [n], radii [n], out [nbatch, ntypes, dim, dim, dim]
 * `out` is overwritten completely (no memset needed before the call).  Two
 * launches: the atoms are sorted by channel into `workspace` (device memory,
 * at least mg_forward_index_workspace_size() bytes, 256-byte aligned, contents
 * undefined before and after; a pointer that is not 256-byte aligned is
 * MG_ERR_INVALID_ARGUMENT), then splatted.  Calls that run concurrently need a
 * workspace each.  `atoms_per_example` sizes the workspace and must be at least
 * the largest example's atom count, also with `atom_offsets`: atoms of an
 * example beyond it are left out of the grid without an error, and 0 means "no
 * atoms at all" (the offsets and arrays are then not looked at).  An atom whose
 * radius * radius_scale is not positive adds nothing, like an atom with a negative
 * type.  MG_ERR_UNSUPPORTED: a channel of 4 GB or more, or
 * nbatch * atoms_per_example >= 2^28. */
int mg_forward_index_ws(const mg_gridmaker* g, int nbatch, const int32_t* atom_offsets,
                        int atoms_per_example, const float* grid_centers,
                        const float grid_center_host[3], const float* coords,
                        const float* type_index, const float* radii, int ntypes, float* out,
                        void* workspace, size_t workspace_bytes, void* stream);

/* The two launches of mg_forward_index_ws as calls of their own, for callers that
 * want the sort off the critical path (enqueued on another stream beside other
 * work, e.g. the backward pass of the previous batch): mg_forward_index_sort
 * reads the atoms and fills `workspace`; mg_forward_index_splat reads only the
 * workspace and writes `out`.  Both must be given the same g, nbatch,
 * atoms_per_example, ntypes and workspace size, and the splat must be ordered
 * after the sort (same stream, or an event).  The grids are those of
 * mg_forward_index_ws, bit for bit.  No counterpart in the reference, whose
 * forward_gpu scans the atoms inside the gridding kernel
 * (src/grid_maker.cu:176-210). */
int mg_forward_index_sort(const mg_gridmaker* g, int nbatch, const int32_t* atom_offsets,
                          int atoms_per_example, const float* grid_centers,
                          const float grid_center_host[3], const float* coords,
                          const float* type_index, const float* radii, int ntypes,
                          void* workspace, size_t workspace_bytes, void* stream);
int mg_forward_index_splat(const mg_gridmaker* g, int nbatch, int atoms_per_example, int ntypes,
                           float* out, const void* workspace, size_t workspace_bytes,
                           void* stream);

/* Host only.  Bytes of workspace mg_forward_index_ws needs for these sizes (0
 * for an empty call). */
size_t mg_forward_index_workspace_size(const mg_gridmaker* g, int nbatch, int atoms_per_example,
                                       int ntypes);

/* The same with a workspace that the library keeps per device and stream: it is
 * allocated (hipMalloc) by the first call on a stream, and a call that needs
 * more gets a new, larger block while the old one stays allocated (launches
 * already enqueued may still use it); nothing is released before the process
 * ends.  Safe for several host threads and several streams: a lock is held
 * until both launches are enqueued, calls on one stream follow each other in
 * that stream, calls on different streams use different blocks (up to 256
 * device/stream pairs, then MG_ERR_UNSUPPORTED).  Callers that must not
 * allocate (HIP graph capture) take mg_forward_index_ws or
 * mg_forward_index_static. */
int mg_forward_index(const mg_gridmaker* g, int nbatch, const int32_t* atom_offsets,
                     int atoms_per_example, const float* grid_centers,
                     const float grid_center_host[3], const float* coords,
                     const float* type_index, const float* radii, int ntypes, float* out,
                     void* stream);

/* No counterpart in the reference.  mg_forward_index for callers that cannot
 * allocate device memory (code under HIP graph capture, serving loops, harnesses
 * that forbid hipMalloc): the workspace is a fixed array of
 * MG_STATIC_SCRATCH_BYTES in the library's device code, one copy per GPU, held
 * until the process ends.  Nothing is allocated or freed.  Sizes whose workspace
 * (mg_forward_index_workspace_size) exceeds the array return MG_ERR_OUT_OF_RANGE
 * and launch nothing.  Every call on a GPU uses that GPU's one array: calls that
 * overlap on one GPU (different streams) race. */
#define MG_STATIC_SCRATCH_BYTES (16u << 20)
int mg_forward_index_static(const mg_gridmaker* g, int nbatch, const int32_t* atom_offsets,
                            int atoms_per_example, const float* grid_centers,
                            const float grid_center_host[3], const float* coords,
                            const float* type_index, const float* radii, int ntypes, float* out,
                            void* stream);

/* No counterpart in the reference.  Selects the write-out of the splat launch of
 * mg_forward_index* for grids of at most 48 voxels a side whose rows are whole
 * 16-byte pieces (dim % 4 == 0, `out` 16-byte aligned): 1 = one workgroup per
 * (example, channel, slab of four x planes) that gathers the sums of its waves
 * in LDS and writes the slab as whole 4 KB pages, 0 = one wave per territory
 * writing its own rows.  The grids are the same bit for bit.  Process-wide;
 * returns the previous setting. */
int mg_forward_index_paged(int on);

/* No counterpart in the reference.  1 = the splat launch of mg_forward_index*
 * for a Gaussian density (fast predicates) takes the kernel instances whose cull
 * also marks the blocks of four voxels that the Gaussian core of an atom can
 * reach, and that skip the exponential in the other blocks of its reach (about
 * half of them on the benchmark batch), 0 = every block evaluates both
 * branches.  The grids are the same bit for bit.  Process-wide; returns the
 * previous setting.  Off by default: the instances without it are the ones
 * that have been timed. */
int mg_forward_index_core_skip(int on);

/* GridMaker::forward, vector types; replaces forward_gpu_vec and its launcher
 * (src/grid_maker.cu:348-441), values of src/grid_maker.cpp:214-271.
 *   type_vector [n, ntypes]; radii [n], or [nbatch, ntypes] when
 *   g->radii_type_indexed. */
int mg_forward_vector(const mg_gridmaker* g, int nbatch, const int32_t* atom_offsets,
                      int atoms_per_example, const float* grid_centers,
                      const float grid_center_host[3], const float* coords,
                      const float* type_vector, const float* radii, int ntypes, float* out,
                      void* stream);

/* The same with an optional workspace in device memory (256-byte aligned,
 * mg_forward_vector_workspace_size() bytes, contents undefined before and
 * after; NULL or too small: as mg_forward_vector).  With it, a launch before
 * the splat lists, for every example and slab of four x planes, the atoms that
 * can reach the slab, and the workgroups of the splat scan their slab's list
 * -- about a fifth of an example at 0.25 A -- instead of every atom of the
 * example (the reference's kernel scans them all per block,
 * src/grid_maker.cu:348-441).  The grids are the same bit for bit; the size is 0
 * for the configurations that do not use lists (type-indexed radii, truncated
 * densities, more than 65,536 atoms per example).  `atoms_per_example` must be
 * at least the largest example. */
int mg_forward_vector_ws(const mg_gridmaker* g, int nbatch, const int32_t* atom_offsets,
                         int atoms_per_example, const float* grid_centers,
                         const float grid_center_host[3], const float* coords,
                         const float* type_vector, const float* radii, int ntypes, float* out,
                         void* workspace, size_t workspace_bytes, void* stream);
size_t mg_forward_vector_workspace_size(const mg_gridmaker* g, int nbatch, int atoms_per_example,
                                        int ntypes);

/* GridMaker::backward, index types; replaces set_atom_gradients and its
 * launcher (src/grid_maker.cu:472-510, 576-595), values of
 * src/grid_maker.cpp:436-467.
 *   diff [nbatch, ntypes, dim, dim, dim] -> atom_gradients [n,3] (overwritten;
 *   ignored atoms get zero). */
int mg_backward_index(const mg_gridmaker* g, int nbatch, const int32_t* atom_offsets,
                      int atoms_per_example, const float* grid_centers,
                      const float grid_center_host[3], const float* coords,
                      const float* type_index, const float* radii, int ntypes,
                      const float* diff, float* atom_gradients, void* stream);

/* GridMaker::backward for index types followed by Transform::backward(gradients,
 * dotranslate = false) per example -- the two calls of the reference's training
 * loop (python/torch_bindings.py:124-136; src/grid_maker.cu:576-595,
 * src/transform.cu:79-93) in one launch; the gradients are those the two calls
 * give, bit for bit. */
int mg_backward_index_unrotated(const mg_gridmaker* g, int nbatch, const int32_t* atom_offsets,
                                int atoms_per_example, const float* grid_centers,
                                const float grid_center_host[3], const float* coords,
                                const float* type_index, const float* radii, int ntypes,
                                const float* diff, const float* quats, const float quat_host[4],
                                const float* rot_centers, const float rot_center_host[3],
                                float* atom_gradients, void* stream);

/* GridMaker::backward, vector types; replaces set_atom_type_gradients and its
 * launcher (src/grid_maker.cu:513-571, 604-642), values of
 * src/grid_maker.cpp:477-519.  type_gradients [n, ntypes] is overwritten. */
int mg_backward_vector(const mg_gridmaker* g, int nbatch, const int32_t* atom_offsets,
                       int atoms_per_example, const float* grid_centers,
                       const float grid_center_host[3], const float* coords,
                       const float* type_vector, const float* radii, int ntypes,
                       const float* diff, float* atom_gradients, float* type_gradients,
                       void* stream);

/* GridMaker::backward_relevance; replaces set_atom_relevance and its launcher
 * (src/grid_maker.cu:922-992), values of src/grid_maker.cpp:392-432, 680-704.
 *   density, diff [nbatch, ntypes, dim, dim, dim] -> relevance [n] (overwritten; ignored atoms
 *   get zero).  Index types only. */
int mg_backward_relevance(const mg_gridmaker* g, int nbatch, const int32_t* atom_offsets,
                          int atoms_per_example, const float* grid_centers,
                          const float grid_center_host[3], const float* coords,
                          const float* type_index, const float* radii, int ntypes,
                          const float* density, const float* diff, float* relevance,
                          void* stream);

/* GridMaker::backward_gradients; replaces set_atom_type_grad_grad and its launcher
 * (src/grid_maker.cu:652-803), values of src/grid_maker.cpp:529-661.  Vector types, not binary.
 *   in:  diff [nbatch, ntypes, dim^3], atom_gradients [n,3], type_gradients [n,ntypes]
 *   out: diffdiff [nbatch, ntypes, dim^3], atom_diffdiff [n,3], type_diffdiff [n,ntypes] (zero);
 *        all three are overwritten.  diffdiff is summed with float atomics: the order of the
 *        additions, hence the last bits, can differ from run to run (as in the reference). */
int mg_backward_gradients(const mg_gridmaker* g, int nbatch, const int32_t* atom_offsets,
                          int atoms_per_example, const float* grid_centers,
                          const float grid_center_host[3], const float* coords,
                          const float* type_vector, const float* radii, int ntypes,
                          const float* diff, const float* atom_gradients,
                          const float* type_gradients, float* diffdiff, float* atom_diffdiff,
                          float* type_diffdiff, void* stream);

/* GridInterpolater::forward; replaces gpu_set_outgrid and its per-channel
 * launch loop (src/grid_interpolater.cu:106-166), values of
 * src/grid_interpolater.cpp:16-48.  One launch for all examples and channels.
 *   in  [nbatch, channels, in_dim, in_dim, in_dim]
 *   out [nbatch, channels, out_dim, out_dim, out_dim], in != out
 * with in_dim = round(in_dimension/in_resolution)+1 and likewise out_dim. */
int mg_interpolate(float in_resolution, float in_dimension, float out_resolution,
                   float out_dimension, int nbatch, int channels,
                   const float* in_centers, const float in_center_host[3], const float* in,
                   const float* quats, const float quat_host[4],
                   const float* rot_centers, const float rot_center_host[3],
                   const float* translations, const float translation_host[3],
                   const float* out_centers, const float out_center_host[3], float* out,
                   void* stream);

/* No counterpart in the reference: a switch for tests.  on != 0 makes every
 * tile of the resampling kernel read its taps straight from global memory
 * instead of staging them in LDS (otherwise only tiles that would overflow the
 * staging buffers do); the values are the same bit for bit.  Process wide;
 * returns the previous setting. */
int mg_interpolate_force_gather(int on);

/* Double precision arrays at the boundary.  The reference instantiates its GPU
 * overloads for Grid<double, N, true> outputs, gradients and coordinates too
 * (src/grid_maker.cu:293-294, 445-446, 460-466, 600; src/transform.cu:96;
 * torch.cuda.DoubleTensor in python/bindings_grids.cpp:108-116) and computes in
 * float there as here.  The kernels of this library read and write float; the
 * host layers stage a double array through a float copy with these two:
 *   mg_narrow: dst[i] = (float)src[i]     mg_widen: dst[i] = (double)src[i] */
int mg_narrow(const double* src, float* dst, size_t n, void* stream);
int mg_widen(const float* src, double* dst, size_t n, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MOLGRID_HIP_H_ */
