// C ABI of the gridding library: argument checks, then the kernel launches of the call on the
// caller's stream.  Nothing here synchronises; the only allocation is the workspace that
// mg_forward_index keeps per device and stream (mg_forward_index_ws takes the caller's instead).
#include <cmath>
#include <cstdint>
#include <dlfcn.h>

#include <atomic>
#include <cstring>
#include <mutex>

#include "kernels.h"
#include "molgrid_hip.h"

// Scratch memory of mg_forward_index_static, part of the loaded code object: every GPU the library
// runs on holds its own copy at its own address until the process ends.  Host code never uses the
// array's name as an address; it asks for the device address once per device (static_scratch()).
static __device__ __align__(256) unsigned char scratch[MG_STATIC_SCRATCH_BYTES];

namespace {

using namespace mg;

Vec3Arg vec3(const float* dev, const float* host) {
  Vec3Arg v;
  v.dev = dev;
  for (int i = 0; i < 3; ++i) v.host[i] = (dev == nullptr && host != nullptr) ? host[i] : 0.f;
  return v;
}

Vec4Arg vec4(const float* dev, const float* host) {
  Vec4Arg v;
  v.dev = dev;
  // identity rotation when nothing is given
  v.host[0] = 1.f;
  v.host[1] = v.host[2] = v.host[3] = 0.f;
  if (dev == nullptr && host != nullptr)
    for (int i = 0; i < 4; ++i) v.host[i] = host[i];
  return v;
}

GridArg grid_arg(const mg_gridmaker* g, int ntypes) {
  GridArg a;
  a.resolution = g->resolution;
  a.half_dimension = (float)(g->dimension / 2.0);  // src/grid_maker.cpp:101
  a.radius_scale = g->radius_scale;
  a.grm = g->gaussian_radius_multiple;
  a.frm = g->final_radius_multiple;
  a.A = g->A;
  a.B = g->B;
  a.C = g->C;
  a.D = g->D;
  a.E = g->E;
  a.dim = (int)g->dim;
  a.ntypes = ntypes;
  return a;
}

// The fast kernels test the cut-offs on (dist/ar)^2 and do not clip to the
// per-atom index box.  That is indistinguishable from the reference when the
// density reaches zero at the cut-off and the box is wider than the support.
// A truncated Gaussian (negative gaussian_radius_multiple at construction:
// no quadratic tail, final == gaussian multiple) or a binary sphere that is not
// narrower than the box (final multiple <= 1; at exactly 1 box and sphere
// coincide and the rounding of the box's edges decides about voxels on them)
// need the reference's exact predicates and its index box.
bool needs_exact(const mg_gridmaker* g) {
  if (g->binary) return g->final_radius_multiple <= 1.0f;
  return g->final_radius_multiple <= g->gaussian_radius_multiple;
}

int check_common(const mg_gridmaker* g, int nbatch, const int32_t* offsets, int per_example,
                 int ntypes) {
  if (g == nullptr) return MG_ERR_NULL_POINTER;
  if (nbatch < 0 || ntypes < 0) return MG_ERR_INVALID_ARGUMENT;
  if (per_example < 0) return MG_ERR_INVALID_ARGUMENT;
  if (g->dim == 0 || g->dim > 65535u) return MG_ERR_OUT_OF_RANGE;
  if (!(g->resolution > 0.f)) return MG_ERR_INVALID_ARGUMENT;
  return MG_OK;
}

int from_hip(hipError_t e) { return e == hipSuccess ? MG_OK : (int)e; }

// Optional roctx ranges around the entry points (mg_trace_ranges): the marker library is looked up
// at run time, so the library does not depend on it.
typedef int (*RangePush)(const char*);
typedef int (*RangePop)(void);
std::atomic<int> g_trace{0};
RangePush g_range_push = nullptr;
RangePop g_range_pop = nullptr;

struct Range {
  bool on;
  explicit Range(const char* name) : on(g_trace.load(std::memory_order_relaxed) != 0) {
    if (on) g_range_push(name);
  }
  ~Range() {
    if (on) g_range_pop();
  }
};

}  // namespace

extern "C" {

int mg_version(void) { return 200; }

int mg_trace_ranges(int on) {
  static std::mutex m;
  std::lock_guard<std::mutex> lock(m);
  if (on && g_range_push == nullptr) {
    void* lib = dlopen("libroctx64.so", RTLD_NOW | RTLD_GLOBAL);
    if (lib == nullptr) lib = dlopen("libroctx64.so.4", RTLD_NOW | RTLD_GLOBAL);
    if (lib == nullptr) return MG_ERR_UNSUPPORTED;
    RangePush push = reinterpret_cast<RangePush>(dlsym(lib, "roctxRangePushA"));
    RangePop pop = reinterpret_cast<RangePop>(dlsym(lib, "roctxRangePop"));
    if (push == nullptr || pop == nullptr) return MG_ERR_UNSUPPORTED;
    g_range_pop = pop;
    g_range_push = push;
  }
  return g_trace.exchange(on ? 1 : 0);
}

const char* mg_error_string(int code) {
  switch (code) {
    case MG_OK: return "success";
    case MG_ERR_INVALID_ARGUMENT: return "invalid argument";
    case MG_ERR_OUT_OF_RANGE: return "argument out of range";
    case MG_ERR_UNSUPPORTED: return "unsupported configuration";
    case MG_ERR_NULL_POINTER: return "required pointer is null";
    default: break;
  }
  if (code > 0) return hipGetErrorString((hipError_t)code);
  return "unknown error";
}

int mg_gridmaker_init(mg_gridmaker* g, float resolution, float dimension, int binary,
                      int radii_type_indexed, float radius_scale, float grm) {
  if (g == nullptr) return MG_ERR_NULL_POINTER;
  std::memset(g, 0, sizeof(*g));
  g->resolution = resolution;
  g->dimension = dimension;
  g->radius_scale = radius_scale;
  g->binary = binary ? 1 : 0;
  g->radii_type_indexed = radii_type_indexed ? 1 : 0;
  // A negative multiple asks for a Gaussian truncated at |grm| with no
  // quadratic tail; otherwise the tail ends at (1 + 2 grm^2) / (2 grm).
  if (grm < 0) {
    g->gaussian_radius_multiple = -grm;
    g->final_radius_multiple = -grm;
  } else {
    g->gaussian_radius_multiple = grm;
    g->final_radius_multiple = (1 + 2 * grm * grm) / (2 * grm);
  }
  // (the reference's arithmetic, include/libmolgrid/grid_maker.h; a quotient that is not a number
  // or out of range must not reach the conversion: such a grid maker gets dim = 0, which every
  // entry point rejects)
  const float points = std::round(dimension / resolution) + 1;
  g->dim = (points >= 1.f && points <= 65535.f) ? (uint32_t)points : 0u;
  // Quadratic a*(d/r)^2 + b*(d/r) + c matching value and slope of the Gaussian
  // at d = grm*r and reaching zero with zero slope at the final multiple; the
  // exponential is taken in double and the results are stored as float.
  const double e = std::exp((double)(-2 * grm * grm));
  g->A = (float)(e * 4 * grm * grm);
  g->B = (float)(-e * (4 * grm + 8 * grm * grm * grm));
  g->C = (float)(e * (4 * grm * grm * grm * grm + 4 * grm * grm + 1));
  g->D = (float)(8 * grm * grm * std::exp(-2.0 * grm * grm));
  g->E = (float)(-(4 * grm + 8 * grm * grm * grm) * e);
  return MG_OK;
}

int mg_transform_forward(int nbatch, const int32_t* atom_offsets, int atoms_per_example,
                         const float* quats, const float quat_host[4], const float* centers,
                         const float center_host[3], const float* translations,
                         const float translation_host[3], int dotranslate,
                         const float* in_coords, float* out_coords, void* stream) {
  const Range range("mg_transform_forward");
  if (nbatch < 0 || atoms_per_example < 0) return MG_ERR_INVALID_ARGUMENT;
  if (nbatch == 0 || atoms_per_example == 0) return MG_OK;   // no atoms at all
  if (in_coords == nullptr || out_coords == nullptr) return MG_ERR_NULL_POINTER;
  BatchArg batch{atoms_per_example > 0 ? atom_offsets : nullptr, atoms_per_example};
  return from_hip(launch_transform(batch, nbatch, atoms_per_example, vec4(quats, quat_host),
                                   vec3(centers, center_host),
                                   vec3(translations, translation_host), dotranslate != 0, false,
                                   in_coords, out_coords, (hipStream_t)stream));
}

int mg_transform_backward(int nbatch, const int32_t* atom_offsets, int atoms_per_example,
                          const float* quats, const float quat_host[4], const float* centers,
                          const float center_host[3], const float* translations,
                          const float translation_host[3], int dotranslate,
                          const float* in_coords, float* out_coords, void* stream) {
  const Range range("mg_transform_backward");
  if (nbatch < 0 || atoms_per_example < 0) return MG_ERR_INVALID_ARGUMENT;
  if (nbatch == 0 || atoms_per_example == 0) return MG_OK;   // no atoms at all
  if (in_coords == nullptr || out_coords == nullptr) return MG_ERR_NULL_POINTER;
  BatchArg batch{atoms_per_example > 0 ? atom_offsets : nullptr, atoms_per_example};
  return from_hip(launch_transform(batch, nbatch, atoms_per_example, vec4(quats, quat_host),
                                   vec3(centers, center_host),
                                   vec3(translations, translation_host), dotranslate != 0, true,
                                   in_coords, out_coords, (hipStream_t)stream));
}

namespace {

int check_forward_index(const mg_gridmaker* g, int nbatch, const int32_t* atom_offsets,
                        int atoms_per_example, const float* coords, const float* type_index,
                        const float* radii, int ntypes, const float* out, bool* nothing_to_do) {
  *nothing_to_do = false;
  int s = check_common(g, nbatch, atom_offsets, atoms_per_example, ntypes);
  if (s != MG_OK) return s;
  // src/grid_maker.cpp:160-162
  if (g->radii_type_indexed) return MG_ERR_INVALID_ARGUMENT;
  if (atoms_per_example < 0) return MG_ERR_INVALID_ARGUMENT;
  if (nbatch == 0 || ntypes == 0) {
    *nothing_to_do = true;
    return MG_OK;
  }
  if (out == nullptr) return MG_ERR_NULL_POINTER;
  // atoms_per_example == 0 means "no atoms at all" (whatever the offsets say: the kernels are then
  // given an empty batch and never touch the arrays, which may be missing)
  const bool has_atoms = atoms_per_example > 0;
  if (has_atoms && (coords == nullptr || type_index == nullptr || radii == nullptr))
    return MG_ERR_NULL_POINTER;
  return MG_OK;
}

int forward_index_with(const mg_gridmaker* g, int nbatch, const int32_t* atom_offsets,
                       int atoms_per_example, const float* grid_centers,
                       const float grid_center_host[3], const float* coords,
                       const float* type_index, const float* radii, int ntypes, float* out,
                       void* workspace, size_t workspace_bytes, void* stream) {
  // no slot for any atom: every example is empty, the offsets are not looked at
  BatchArg batch{atoms_per_example > 0 ? atom_offsets : nullptr, atoms_per_example};
  const hipError_t e = launch_forward_sorted(
      grid_arg(g, ntypes), batch, nbatch, vec3(grid_centers, grid_center_host), coords, type_index,
      radii, out, g->binary != 0, needs_exact(g), workspace, workspace_bytes, (hipStream_t)stream);
  if (e == hipErrorInvalidValue) return MG_ERR_UNSUPPORTED;
  return from_hip(e);
}

// Workspaces of mg_forward_index: one per (device, stream), grown when a call needs more.  A
// block that became too small is kept until the process ends (launches already enqueued may still
// use it, and a free would wait for the device); blocks grow by half at least, so what is kept
// is bounded by twice the largest.
struct StreamWorkspace {
  int device = -1;
  void* stream = nullptr;
  void* ptr = nullptr;
  size_t bytes = 0;
};
constexpr int kMaxDevices = 64;
constexpr int kMaxWorkspaces = 256;
StreamWorkspace g_workspace[kMaxWorkspaces];
int g_workspaces = 0;
std::mutex g_workspace_mutex;

}  // namespace

size_t mg_forward_index_workspace_size(const mg_gridmaker* g, int nbatch, int atoms_per_example,
                                       int ntypes) {
  if (g == nullptr || nbatch <= 0 || ntypes <= 0 || atoms_per_example < 0) return 0;
  return forward_sorted_workspace_bytes(nbatch, atoms_per_example, ntypes, (int)g->dim);
}

int mg_forward_index_ws(const mg_gridmaker* g, int nbatch, const int32_t* atom_offsets,
                        int atoms_per_example, const float* grid_centers,
                        const float grid_center_host[3], const float* coords,
                        const float* type_index, const float* radii, int ntypes, float* out,
                        void* workspace, size_t workspace_bytes, void* stream) {
  const Range range("mg_forward_index_ws");
  bool nothing = false;
  const int s = check_forward_index(g, nbatch, atom_offsets, atoms_per_example, coords, type_index,
                                    radii, ntypes, out, &nothing);
  if (s != MG_OK || nothing) return s;
  if (workspace == nullptr) return MG_ERR_NULL_POINTER;
  if ((reinterpret_cast<uintptr_t>(workspace) & 255u) != 0) return MG_ERR_INVALID_ARGUMENT;
  if (workspace_bytes < mg_forward_index_workspace_size(g, nbatch, atoms_per_example, ntypes))
    return MG_ERR_INVALID_ARGUMENT;
  return forward_index_with(g, nbatch, atom_offsets, atoms_per_example, grid_centers,
                            grid_center_host, coords, type_index, radii, ntypes, out, workspace,
                            workspace_bytes, stream);
}

int mg_forward_index_sort(const mg_gridmaker* g, int nbatch, const int32_t* atom_offsets,
                          int atoms_per_example, const float* grid_centers,
                          const float grid_center_host[3], const float* coords,
                          const float* type_index, const float* radii, int ntypes,
                          void* workspace, size_t workspace_bytes, void* stream) {
  const Range range("mg_forward_index_sort");
  bool nothing = false;
  const float* const no_grid = reinterpret_cast<const float*>(16);    // only tested against NULL
  const int s = check_forward_index(g, nbatch, atom_offsets, atoms_per_example, coords, type_index,
                                    radii, ntypes, no_grid, &nothing);
  if (s != MG_OK || nothing) return s;
  if (workspace == nullptr) return MG_ERR_NULL_POINTER;
  if ((reinterpret_cast<uintptr_t>(workspace) & 255u) != 0) return MG_ERR_INVALID_ARGUMENT;
  if (workspace_bytes < mg_forward_index_workspace_size(g, nbatch, atoms_per_example, ntypes))
    return MG_ERR_INVALID_ARGUMENT;
  BatchArg batch{atoms_per_example > 0 ? atom_offsets : nullptr, atoms_per_example};
  const hipError_t e = launch_sort_atoms(grid_arg(g, ntypes), batch, nbatch,
                                         vec3(grid_centers, grid_center_host), coords, type_index,
                                         radii, g->binary != 0, workspace, workspace_bytes,
                                         (hipStream_t)stream);
  if (e == hipErrorInvalidValue) return MG_ERR_UNSUPPORTED;
  return from_hip(e);
}

int mg_forward_index_splat(const mg_gridmaker* g, int nbatch, int atoms_per_example, int ntypes,
                           float* out, const void* workspace, size_t workspace_bytes,
                           void* stream) {
  const Range range("mg_forward_index_splat");
  int s = check_common(g, nbatch, nullptr, atoms_per_example, ntypes);
  if (s != MG_OK) return s;
  if (g->radii_type_indexed) return MG_ERR_INVALID_ARGUMENT;
  if (nbatch == 0 || ntypes == 0) return MG_OK;
  if (out == nullptr || workspace == nullptr) return MG_ERR_NULL_POINTER;
  if ((reinterpret_cast<uintptr_t>(workspace) & 255u) != 0) return MG_ERR_INVALID_ARGUMENT;
  if (workspace_bytes < mg_forward_index_workspace_size(g, nbatch, atoms_per_example, ntypes))
    return MG_ERR_INVALID_ARGUMENT;
  const hipError_t e = launch_splat_sorted(grid_arg(g, ntypes), nbatch, atoms_per_example, out,
                                           g->binary != 0, needs_exact(g),
                                           const_cast<void*>(workspace), workspace_bytes,
                                           (hipStream_t)stream);
  if (e == hipErrorInvalidValue) return MG_ERR_UNSUPPORTED;
  return from_hip(e);
}

int mg_forward_index(const mg_gridmaker* g, int nbatch, const int32_t* atom_offsets,
                     int atoms_per_example, const float* grid_centers,
                     const float grid_center_host[3], const float* coords,
                     const float* type_index, const float* radii, int ntypes, float* out,
                     void* stream) {
  const Range range("mg_forward_index");
  bool nothing = false;
  const int s = check_forward_index(g, nbatch, atom_offsets, atoms_per_example, coords, type_index,
                                    radii, ntypes, out, &nothing);
  if (s != MG_OK || nothing) return s;
  const size_t need = mg_forward_index_workspace_size(g, nbatch, atoms_per_example, ntypes);
  // (before anything is allocated: sizes that the launches do not cover)
  if (!forward_sorted_supports(grid_arg(g, ntypes), nbatch, atoms_per_example)) return MG_ERR_UNSUPPORTED;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return from_hip(e);
  // The lock is held until both launches are enqueued: calls of several host threads on one
  // stream then follow each other in the stream and may share its block; calls on different
  // streams get different blocks.
  std::lock_guard<std::mutex> lock(g_workspace_mutex);
  StreamWorkspace* w = nullptr;
  for (int i = 0; i < g_workspaces; ++i)
    if (g_workspace[i].device == dev && g_workspace[i].stream == stream) w = &g_workspace[i];
  if (w == nullptr) {
    if (g_workspaces == kMaxWorkspaces) return MG_ERR_UNSUPPORTED;   // use mg_forward_index_ws
    w = &g_workspace[g_workspaces++];
    w->device = dev;
    w->stream = stream;
  }
  if (w->bytes < need) {
    void* block = nullptr;
    const size_t want = need + need / 2;
    e = hipMalloc(&block, want);
    if (e != hipSuccess) return from_hip(e);
    w->ptr = block;                    // the block before it stays allocated
    w->bytes = want;
  }
  return forward_index_with(g, nbatch, atom_offsets, atoms_per_example, grid_centers,
                            grid_center_host, coords, type_index, radii, ntypes, out, w->ptr,
                            w->bytes, stream);
}

namespace {

void* g_scratch_address[kMaxDevices] = {nullptr};   // device address of `scratch`, per device
std::mutex g_scratch_mutex;

// Device address of the current device's copy of `scratch` (asked for on the first call on that
// device); the error of the lookup otherwise.
hipError_t static_scratch(void** address) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_address[dev] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return e;
    if (p == nullptr) return hipErrorInvalidSymbol;
    g_scratch_address[dev] = p;
  }
  *address = g_scratch_address[dev];
  return hipSuccess;
}

}  // namespace

int mg_forward_index_static(const mg_gridmaker* g, int nbatch, const int32_t* atom_offsets,
                            int atoms_per_example, const float* grid_centers,
                            const float grid_center_host[3], const float* coords,
                            const float* type_index, const float* radii, int ntypes, float* out,
                            void* stream) {
  const Range range("mg_forward_index_static");
  bool nothing = false;
  const int s = check_forward_index(g, nbatch, atom_offsets, atoms_per_example, coords, type_index,
                                    radii, ntypes, out, &nothing);
  if (s != MG_OK || nothing) return s;
  if (mg_forward_index_workspace_size(g, nbatch, atoms_per_example, ntypes) > MG_STATIC_SCRATCH_BYTES)
    return MG_ERR_OUT_OF_RANGE;
  void* address = nullptr;
  const hipError_t e = static_scratch(&address);
  if (e != hipSuccess) return from_hip(e);
  // nothing in the scratch has to start at zero: the sort launch writes every table entry and
  // every record that the splat launch reads
  return forward_index_with(g, nbatch, atom_offsets, atoms_per_example, grid_centers,
                            grid_center_host, coords, type_index, radii, ntypes, out, address,
                            MG_STATIC_SCRATCH_BYTES, stream);
}

int mg_forward_index_paged(int on) { return set_forward_paged(on); }
int mg_forward_index_core_skip(int on) { return set_forward_core_skip(on); }

size_t mg_forward_vector_workspace_size(const mg_gridmaker* g, int nbatch, int atoms_per_example,
                                        int ntypes) {
  if (g == nullptr || nbatch <= 0 || ntypes <= 0 || atoms_per_example <= 0) return 0;
  // only the matrix-core kernel (per-atom radii, density reaching zero at the cut-off) uses lists
  if (g->radii_type_indexed || needs_exact(g) || atoms_per_example > 65536) return 0;
  return forward_vector_workspace_bytes(nbatch, atoms_per_example, (int)g->dim);
}

int mg_forward_vector_ws(const mg_gridmaker* g, int nbatch, const int32_t* atom_offsets,
                         int atoms_per_example, const float* grid_centers,
                         const float grid_center_host[3], const float* coords,
                         const float* type_vector, const float* radii, int ntypes, float* out,
                         void* workspace, size_t workspace_bytes, void* stream) {
  const Range range("mg_forward_vector");
  int s = check_common(g, nbatch, atom_offsets, atoms_per_example, ntypes);
  if (s != MG_OK) return s;
  if (nbatch == 0 || ntypes == 0) return MG_OK;
  if (out == nullptr) return MG_ERR_NULL_POINTER;
  const bool has_atoms = atoms_per_example > 0;
  if (has_atoms && (coords == nullptr || type_vector == nullptr || radii == nullptr))
    return MG_ERR_NULL_POINTER;
  if (g->radii_type_indexed && radii == nullptr) return MG_ERR_NULL_POINTER;
  if (workspace != nullptr && (reinterpret_cast<uintptr_t>(workspace) & 255u) != 0)
    return MG_ERR_INVALID_ARGUMENT;
  BatchArg batch{atoms_per_example > 0 ? atom_offsets : nullptr, atoms_per_example};
  return from_hip(launch_forward_vector(grid_arg(g, ntypes), batch, nbatch,
                                        vec3(grid_centers, grid_center_host), coords,
                                        type_vector, radii, out, g->binary != 0,
                                        g->radii_type_indexed != 0, needs_exact(g), workspace,
                                        workspace_bytes, (hipStream_t)stream));
}

int mg_forward_vector(const mg_gridmaker* g, int nbatch, const int32_t* atom_offsets,
                      int atoms_per_example, const float* grid_centers,
                      const float grid_center_host[3], const float* coords,
                      const float* type_vector, const float* radii, int ntypes, float* out,
                      void* stream) {
  return mg_forward_vector_ws(g, nbatch, atom_offsets, atoms_per_example, grid_centers,
                              grid_center_host, coords, type_vector, radii, ntypes, out, nullptr, 0,
                              stream);
}

int mg_backward_index(const mg_gridmaker* g, int nbatch, const int32_t* atom_offsets,
                      int atoms_per_example, const float* grid_centers,
                      const float grid_center_host[3], const float* coords,
                      const float* type_index, const float* radii, int ntypes,
                      const float* diff, float* atom_gradients, void* stream) {
  const Range range("mg_backward_index");
  int s = check_common(g, nbatch, atom_offsets, atoms_per_example, ntypes);
  if (s != MG_OK) return s;
  // src/grid_maker.cpp:442-444
  if (g->radii_type_indexed) return MG_ERR_INVALID_ARGUMENT;
  if (nbatch == 0 || atoms_per_example == 0) return MG_OK;   // no atoms at all
  if (coords == nullptr || type_index == nullptr || radii == nullptr || diff == nullptr ||
      atom_gradients == nullptr)
    return MG_ERR_NULL_POINTER;
  BatchArg batch{atoms_per_example > 0 ? atom_offsets : nullptr, atoms_per_example};
  return from_hip(launch_backward_index(grid_arg(g, ntypes), batch, nbatch, atoms_per_example,
                                        vec3(grid_centers, grid_center_host), coords,
                                        type_index, radii, diff, atom_gradients,
                                        (hipStream_t)stream));
}

int mg_backward_index_unrotated(const mg_gridmaker* g, int nbatch, const int32_t* atom_offsets,
                                int atoms_per_example, const float* grid_centers,
                                const float grid_center_host[3], const float* coords,
                                const float* type_index, const float* radii, int ntypes,
                                const float* diff, const float* quats, const float quat_host[4],
                                const float* rot_centers, const float rot_center_host[3],
                                float* atom_gradients, void* stream) {
  const Range range("mg_backward_index_unrotated");
  int s = check_common(g, nbatch, atom_offsets, atoms_per_example, ntypes);
  if (s != MG_OK) return s;
  if (g->radii_type_indexed) return MG_ERR_INVALID_ARGUMENT;
  if (nbatch == 0 || atoms_per_example == 0) return MG_OK;   // no atoms at all
  if (coords == nullptr || type_index == nullptr || radii == nullptr || diff == nullptr ||
      atom_gradients == nullptr)
    return MG_ERR_NULL_POINTER;
  BatchArg batch{atoms_per_example > 0 ? atom_offsets : nullptr, atoms_per_example};
  return from_hip(launch_backward_index_unrotated(
      grid_arg(g, ntypes), batch, nbatch, atoms_per_example, vec3(grid_centers, grid_center_host),
      coords, type_index, radii, diff, vec4(quats, quat_host), vec3(rot_centers, rot_center_host),
      atom_gradients, (hipStream_t)stream));
}

int mg_backward_vector(const mg_gridmaker* g, int nbatch, const int32_t* atom_offsets,
                       int atoms_per_example, const float* grid_centers,
                       const float grid_center_host[3], const float* coords,
                       const float* type_vector, const float* radii, int ntypes,
                       const float* diff, float* atom_gradients, float* type_gradients,
                       void* stream) {
  const Range range("mg_backward_vector");
  int s = check_common(g, nbatch, atom_offsets, atoms_per_example, ntypes);
  if (s != MG_OK) return s;
  if (nbatch == 0 || atoms_per_example == 0) return MG_OK;   // no atoms at all
  if (coords == nullptr || type_vector == nullptr || radii == nullptr || diff == nullptr ||
      atom_gradients == nullptr || type_gradients == nullptr)
    return MG_ERR_NULL_POINTER;
  BatchArg batch{atoms_per_example > 0 ? atom_offsets : nullptr, atoms_per_example};
  return from_hip(launch_backward_vector(grid_arg(g, ntypes), batch, nbatch, atoms_per_example,
                                         vec3(grid_centers, grid_center_host), coords,
                                         type_vector, radii, diff, atom_gradients,
                                         type_gradients, g->binary != 0,
                                         g->radii_type_indexed != 0, (hipStream_t)stream));
}

int mg_backward_relevance(const mg_gridmaker* g, int nbatch, const int32_t* atom_offsets,
                          int atoms_per_example, const float* grid_centers,
                          const float grid_center_host[3], const float* coords,
                          const float* type_index, const float* radii, int ntypes,
                          const float* density, const float* diff, float* relevance,
                          void* stream) {
  const Range range("mg_backward_relevance");
  int s = check_common(g, nbatch, atom_offsets, atoms_per_example, ntypes);
  if (s != MG_OK) return s;
  if (g->radii_type_indexed) return MG_ERR_INVALID_ARGUMENT;
  if (nbatch == 0 || atoms_per_example == 0) return MG_OK;   // no atoms at all
  if (coords == nullptr || type_index == nullptr || radii == nullptr || density == nullptr ||
      diff == nullptr || relevance == nullptr)
    return MG_ERR_NULL_POINTER;
  BatchArg batch{atoms_per_example > 0 ? atom_offsets : nullptr, atoms_per_example};
  return from_hip(launch_backward_relevance(grid_arg(g, ntypes), batch, nbatch, atoms_per_example,
                                            vec3(grid_centers, grid_center_host), coords,
                                            type_index, radii, density, diff, relevance,
                                            g->binary != 0, (hipStream_t)stream));
}

int mg_backward_gradients(const mg_gridmaker* g, int nbatch, const int32_t* atom_offsets,
                          int atoms_per_example, const float* grid_centers,
                          const float grid_center_host[3], const float* coords,
                          const float* type_vector, const float* radii, int ntypes,
                          const float* diff, const float* atom_gradients,
                          const float* type_gradients, float* diffdiff, float* atom_diffdiff,
                          float* type_diffdiff, void* stream) {
  const Range range("mg_backward_gradients");
  int s = check_common(g, nbatch, atom_offsets, atoms_per_example, ntypes);
  if (s != MG_OK) return s;
  // src/grid_maker.cpp:559
  if (g->binary) return MG_ERR_INVALID_ARGUMENT;
  if (nbatch == 0 || ntypes == 0) return MG_OK;
  if (diffdiff == nullptr) return MG_ERR_NULL_POINTER;
  const bool has_atoms = atoms_per_example > 0;
  if (has_atoms && (coords == nullptr || type_vector == nullptr || radii == nullptr ||
                    diff == nullptr || atom_gradients == nullptr || type_gradients == nullptr ||
                    atom_diffdiff == nullptr || type_diffdiff == nullptr))
    return MG_ERR_NULL_POINTER;
  BatchArg batch{atoms_per_example > 0 ? atom_offsets : nullptr, atoms_per_example};
  return from_hip(launch_backward_gradients(grid_arg(g, ntypes), batch, nbatch, atoms_per_example,
                                            vec3(grid_centers, grid_center_host), coords,
                                            type_vector, radii, diff, atom_gradients,
                                            type_gradients, diffdiff, atom_diffdiff,
                                            type_diffdiff, g->radii_type_indexed != 0,
                                            (hipStream_t)stream));
}

int mg_widen(const float* src, double* dst, size_t n, void* stream) {
  const Range range("mg_widen");
  if (n == 0) return MG_OK;
  if (src == nullptr || dst == nullptr) return MG_ERR_NULL_POINTER;
  return from_hip(launch_widen(src, dst, n, (hipStream_t)stream));
}

int mg_narrow(const double* src, float* dst, size_t n, void* stream) {
  const Range range("mg_narrow");
  if (n == 0) return MG_OK;
  if (src == nullptr || dst == nullptr) return MG_ERR_NULL_POINTER;
  return from_hip(launch_narrow(src, dst, n, (hipStream_t)stream));
}

int mg_interpolate(float in_resolution, float in_dimension, float out_resolution,
                   float out_dimension, int nbatch, int channels, const float* in_centers,
                   const float in_center_host[3], const float* in, const float* quats,
                   const float quat_host[4], const float* rot_centers,
                   const float rot_center_host[3], const float* translations,
                   const float translation_host[3], const float* out_centers,
                   const float out_center_host[3], float* out, void* stream) {
  const Range range("mg_interpolate");
  if (nbatch < 0 || channels < 0) return MG_ERR_INVALID_ARGUMENT;
  if (!(in_resolution > 0.f) || !(out_resolution > 0.f)) return MG_ERR_INVALID_ARGUMENT;
  // src/grid_interpolater.cpp:58-60, 70-75
  if (in == nullptr || out == nullptr) return MG_ERR_INVALID_ARGUMENT;
  if (in == out) return MG_ERR_INVALID_ARGUMENT;
  if (nbatch == 0 || channels == 0) return MG_OK;
  InterpArg p;
  p.in_resolution = in_resolution;
  p.out_resolution = out_resolution;
  p.in_half = (float)(in_dimension / 2.0);
  p.out_half = (float)(out_dimension / 2.0);
  // include/libmolgrid/grid_interpolater.h:59-64
  const float in_points = std::round(in_dimension / in_resolution) + 1;
  const float out_points = std::round(out_dimension / out_resolution) + 1;
  // (also false for a quotient that is not a number, which must not reach the conversion)
  if (!(in_points >= 1.f && in_points <= 1200.f && out_points >= 1.f && out_points <= 1200.f))
    return MG_ERR_OUT_OF_RANGE;
  p.in_dim = (int)in_points;
  p.out_dim = (int)out_points;
  p.channels = channels;
  return from_hip(launch_interpolate(p, nbatch, vec3(in_centers, in_center_host), in,
                                     vec4(quats, quat_host), vec3(rot_centers, rot_center_host),
                                     vec3(translations, translation_host),
                                     vec3(out_centers, out_center_host), out,
                                     (hipStream_t)stream));
}

int mg_interpolate_force_gather(int on) { return mg::set_interpolate_force_gather(on); }

}  // extern "C"
