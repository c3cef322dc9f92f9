// ManagedGrid<Dtype, N>: an owning N-dimensional array with a host buffer and a lazily created
// device mirror (libmolgrid's ManagedGrid, include/libmolgrid/managed_grid.h:31-608).  The data
// lives on exactly one side at a time: gpu() migrates it to the device (allocating the mirror on
// first use), cpu() brings it back; both return non-owning Grid views.  Copies of a ManagedGrid and
// its sub-grids (operator[]) share the same storage.
#ifndef LIBMOLGRID_MANAGED_GRID_H_
#define LIBMOLGRID_MANAGED_GRID_H_

#include <cstdlib>
#include <memory>
#include <type_traits>

#include "libmolgrid/grid.h"

namespace libmolgrid {

namespace detail {
/// storage shared by a managed grid, its copies and its sub-grids
template <typename Dtype>
struct MirroredStorage {
  Dtype* host = nullptr;
  Dtype* device = nullptr;
  size_t capacity = 0;
  bool on_device = false;

  explicit MirroredStorage(size_t n) : capacity(n) {
    host = static_cast<Dtype*>(std::calloc(n ? n : 1, sizeof(Dtype)));
    if (!host) throw std::bad_alloc();
  }
  MirroredStorage(const MirroredStorage&) = delete;
  MirroredStorage& operator=(const MirroredStorage&) = delete;
  ~MirroredStorage() {
    std::free(host);
    if (device) (void)hipFree(device);
  }
  void to_device(bool transfer) {
    if (on_device) return;
    if (!device && capacity) LMG_HIP_CHECK(hipMalloc(reinterpret_cast<void**>(&device), capacity * sizeof(Dtype)));
    if (transfer) raw_copy(device, true, host, false, capacity);
    on_device = true;
  }
  void to_host(bool transfer) {
    if (!on_device) return;
    if (transfer) raw_copy(host, false, device, true, capacity);
    on_device = false;
  }
};
}  // namespace detail

template <typename Dtype, std::size_t NumDims>
class ManagedGrid {
 public:
  using gpu_grid_t = Grid<Dtype, NumDims, true>;
  using cpu_grid_t = Grid<Dtype, NumDims, false>;
  using type = Dtype;
  static constexpr size_t N = NumDims;

 private:
  using storage_t = detail::MirroredStorage<Dtype>;
  std::shared_ptr<storage_t> store;
  size_t start = 0;  // first element of this view inside the storage
  size_t dims[NumDims] = {};
  mutable cpu_grid_t cpu_view;
  mutable gpu_grid_t gpu_view;

  template <typename D, std::size_t M>
  friend class ManagedGrid;

  void refresh_views() const {
    cpu_view = cpu_grid_t(store ? store->host + start : nullptr, dims);
    gpu_view = gpu_grid_t(store && store->device ? store->device + start : nullptr, dims);
  }
  size_t count() const {
    size_t n = 1;
    for (size_t i = 0; i < NumDims; ++i) n *= dims[i];
    return n;
  }

 public:
  ManagedGrid() { refresh_views(); }

  template <typename... I, typename = typename std::enable_if<
                                sizeof...(I) == NumDims && detail::all_integral<I...>::value>::type>
  ManagedGrid(I... sizes) : dims{static_cast<size_t>(sizes)...} {
    store = std::make_shared<storage_t>(count());
    refresh_views();
  }
  explicit ManagedGrid(const size_t* sizes) {
    for (size_t i = 0; i < NumDims; ++i) dims[i] = sizes[i];
    store = std::make_shared<storage_t>(count());
    refresh_views();
  }
  /// slice i of a grid with one more dimension (shares storage)
  explicit ManagedGrid(const ManagedGrid<Dtype, NumDims + 1>& G, size_t i) : store(G.store) {
    for (size_t k = 0; k < NumDims; ++k) dims[k] = G.dims[k + 1];
    start = G.start + i * count();
    refresh_views();
  }

  const size_t* dimensions() const { return dims; }
  size_t dimension(size_t i) const {
    if (i >= NumDims) throw std::out_of_range("Invalid dimension " + itoa(i));
    return dims[i];
  }
  size_t offset(size_t i) const { return cpu_view.offset(i); }
  size_t size() const { return count(); }

  bool ongpu() const { return store && store->on_device; }
  bool oncpu() const { return !ongpu(); }

  /// move the data to the device (whole storage); dotransfer = false skips the copy
  void togpu(bool dotransfer = true) const {
    if (store) store->to_device(dotransfer);
    refresh_views();
  }
  void tocpu(bool dotransfer = true) const {
    if (store) store->to_host(dotransfer);
    refresh_views();
  }
  const gpu_grid_t& gpu() const { togpu(); return gpu_view; }
  gpu_grid_t& gpu() { togpu(); return gpu_view; }
  const cpu_grid_t& cpu() const { tocpu(); return cpu_view; }
  cpu_grid_t& cpu() { tocpu(); return cpu_view; }
  operator cpu_grid_t() const { return cpu(); }
  operator cpu_grid_t&() { return cpu(); }
  operator gpu_grid_t() const { return gpu(); }
  operator gpu_grid_t&() { return gpu(); }

  /// pointer to the data on the side it currently lives on
  Dtype* data() { return ongpu() ? gpu_view.data() : cpu_view.data(); }
  const Dtype* data() const { return ongpu() ? gpu_view.data() : cpu_view.data(); }

  /// element access always happens on the host
  template <typename... I>
  Dtype& operator()(I... indices) { return cpu()(indices...); }
  template <typename... I>
  Dtype operator()(I... indices) const { return cpu()(indices...); }

  /// sub-grid sharing this grid's storage (an element reference for N = 1)
  template <std::size_t M = NumDims>
  typename std::enable_if<(M > 1), ManagedGrid<Dtype, NumDims - 1>>::type operator[](size_t i) const {
    if (i >= dims[0]) throw std::out_of_range("Invalid range. " + itoa(i) + " >= " + itoa(dims[0]));
    return ManagedGrid<Dtype, NumDims - 1>(*this, i);
  }
  template <std::size_t M = NumDims>
  typename std::enable_if<(M == 1), Dtype&>::type operator[](size_t i) { return cpu()[i]; }

  void fill_zero() {
    if (ongpu()) gpu_view.fill_zero();
    else cpu_view.fill_zero();
  }

  template <bool destCUDA>
  size_t copyTo(Grid<Dtype, NumDims, destCUDA>& dest) const {
    return ongpu() ? gpu_view.copyTo(dest) : cpu_view.copyTo(dest);
  }
  size_t copyTo(ManagedGrid& dest) const {
    if (dest.ongpu()) return copyTo(dest.gpu_view);
    return copyTo(dest.cpu_view);
  }
  template <bool srcCUDA>
  size_t copyFrom(const Grid<Dtype, NumDims, srcCUDA>& src) {
    return ongpu() ? gpu_view.copyFrom(src) : cpu_view.copyFrom(src);
  }
  size_t copyFrom(const ManagedGrid& src) {
    return src.ongpu() ? copyFrom(src.gpu_view) : copyFrom(src.cpu_view);
  }
  /// copy src into this grid starting at index `start_index` of the first dimension
  size_t copyInto(size_t start_index, const ManagedGrid& src) {
    const size_t off = cpu_view.offset(0) * start_index;
    if (off >= size()) return 0;
    const size_t n = std::min(size() - off, src.size());
    detail::raw_copy(data() + off, ongpu(), src.data(), src.ongpu(), n);
    return n;
  }

  /// deep copy of this view (same side as the source)
  ManagedGrid clone() const {
    ManagedGrid out(dims);
    if (ongpu()) out.togpu(false);
    detail::raw_copy(out.data(), out.ongpu(), data(), ongpu(), size());
    return out;
  }

  /// a grid of the given extents holding the same leading data; shares storage when it fits
  template <typename... I, typename = typename std::enable_if<
                                sizeof...(I) == NumDims && detail::all_integral<I...>::value>::type>
  ManagedGrid resized(I... sizes) const {
    ManagedGrid out;
    const size_t nd[NumDims] = {static_cast<size_t>(sizes)...};
    size_t n = 1;
    for (size_t i = 0; i < NumDims; ++i) { out.dims[i] = nd[i]; n *= nd[i]; }
    if (store && start == 0 && n <= store->capacity) {
      out.store = store;
      out.refresh_views();
      return out;
    }
    out.store = std::make_shared<storage_t>(n);
    out.refresh_views();
    if (store) {
      if (ongpu()) out.togpu(false);
      detail::raw_copy(out.data(), out.ongpu(), data(), ongpu(), std::min(n, size()));
    }
    return out;
  }

  /// pointer equality, as in the reference
  bool operator==(const ManagedGrid& rhs) const {
    return store == rhs.store && start == rhs.start && size() == rhs.size();
  }
};

#define LMG_MGRID_TYPEDEFS(n)              \
  typedef ManagedGrid<float, n> MGrid##n##f; \
  typedef ManagedGrid<double, n> MGrid##n##d;
LMG_MGRID_TYPEDEFS(1)
LMG_MGRID_TYPEDEFS(2)
LMG_MGRID_TYPEDEFS(3)
LMG_MGRID_TYPEDEFS(4)
LMG_MGRID_TYPEDEFS(5)
LMG_MGRID_TYPEDEFS(6)
LMG_MGRID_TYPEDEFS(7)
LMG_MGRID_TYPEDEFS(8)
#undef LMG_MGRID_TYPEDEFS

}  // namespace libmolgrid

#endif
