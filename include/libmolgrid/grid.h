// Grid<Dtype, N, isCUDA>: a non-owning, row-major, N-dimensional view of host (isCUDA = false)
// or device (isCUDA = true) memory.  Same members as libmolgrid's Grid
// (include/libmolgrid/grid.h:43-325): data(), dimension(i), size(), offset(i), operator()
// (unchecked element access, host views only), operator[] (checked slice), copyTo / copyFrom,
// fill_zero.  Views are cheap to copy and never free anything.
#ifndef LIBMOLGRID_GRID_H_
#define LIBMOLGRID_GRID_H_

#include <algorithm>
#include <cstddef>
#include <cstring>
#include <type_traits>

#include "libmolgrid/common.h"

namespace libmolgrid {

template <typename Dtype, std::size_t NumDims>
class ManagedGrid;

namespace detail {
template <typename... I>
struct all_integral : std::true_type {};
template <typename First, typename... Rest>
struct all_integral<First, Rest...>
    : std::integral_constant<bool, std::is_integral<First>::value && all_integral<Rest...>::value> {};

inline hipMemcpyKind copy_kind(bool src_device, bool dst_device) {
  if (src_device) return dst_device ? hipMemcpyDeviceToDevice : hipMemcpyDeviceToHost;
  return dst_device ? hipMemcpyHostToDevice : hipMemcpyHostToHost;
}
template <typename Dtype>
inline void raw_copy(Dtype* dst, bool dst_device, const Dtype* src, bool src_device, size_t n) {
  if (n == 0) return;
  if (!dst_device && !src_device) {
    std::memcpy(dst, src, n * sizeof(Dtype));
  } else {
    LMG_HIP_CHECK(hipMemcpy(dst, src, n * sizeof(Dtype), copy_kind(src_device, dst_device)));
  }
}
template <typename Dtype>
inline void raw_zero(Dtype* dst, bool device, size_t n) {
  if (n == 0) return;
  if (device) LMG_HIP_CHECK(hipMemset(dst, 0, n * sizeof(Dtype)));
  else std::memset(dst, 0, n * sizeof(Dtype));
}
}  // namespace detail

template <typename Dtype, std::size_t NumDims, bool isCUDA = false>
class Grid {
  Dtype* buffer = nullptr;
  size_t dims[NumDims] = {};
  size_t offs[NumDims] = {};

  void set_strides() {
    size_t stride = 1;
    for (size_t i = NumDims; i-- > 0;) {
      offs[i] = stride;
      stride *= dims[i];
    }
  }

 public:
  using type = Dtype;
  using subgrid_t = Grid<Dtype, NumDims - 1, isCUDA>;
  using managed_t = ManagedGrid<Dtype, NumDims>;
  using cpu_grid_t = Grid<Dtype, NumDims, false>;
  using gpu_grid_t = Grid<Dtype, NumDims, true>;
  static constexpr size_t N = NumDims;
  static constexpr bool GPU = isCUDA;

  Grid() = default;

  /// view of memory at d with the given extents
  template <typename... I, typename = typename std::enable_if<
                                sizeof...(I) == NumDims && detail::all_integral<I...>::value>::type>
  Grid(Dtype* d, I... sizes) : buffer(d), dims{static_cast<size_t>(sizes)...} {
    set_strides();
  }

  Grid(Dtype* d, const size_t* sizes) : buffer(d) {
    for (size_t i = 0; i < NumDims; ++i) dims[i] = sizes[i];
    set_strides();
  }

  /// slice i of a grid with one more dimension
  explicit Grid(const Grid<Dtype, NumDims + 1, isCUDA>& G, size_t i)
      : buffer(G.data() ? G.data() + i * G.offset(0) : nullptr) {
    for (size_t k = 0; k < NumDims; ++k) {
      dims[k] = G.dimension(k + 1);
      offs[k] = G.offset(k + 1);
    }
  }

  const size_t* dimensions() const { return dims; }
  size_t dimension(size_t i) const {
    if (i >= NumDims) throw std::out_of_range("Invalid dimension " + itoa(i));
    return dims[i];
  }
  const size_t* offsets() const { return offs; }
  size_t offset(size_t i) const { return offs[i]; }
  size_t size() const {
    size_t n = 1;
    for (size_t i = 0; i < NumDims; ++i) n *= dims[i];
    return n;
  }
  Dtype* data() const { return buffer; }
  void set_buffer(Dtype* p) { buffer = p; }

  /// checked slice along the first dimension
  subgrid_t operator[](size_t i) const {
    if (i >= dims[0])
      throw std::out_of_range("Invalid range. " + itoa(i) + " >= " + itoa(dims[0]));
    return subgrid_t(*this, i);
  }

  template <typename... I>
  size_t position(I... indices) const {
    static_assert(NumDims == sizeof...(indices), "Incorrect number of grid indices");
    const size_t idx[NumDims] = {static_cast<size_t>(indices)...};
    size_t pos = 0;
    for (size_t i = 0; i < NumDims; ++i) pos += idx[i] * offs[i];
    return pos;
  }
  /// unchecked element access (host memory only)
  template <typename... I>
  Dtype& operator()(I... indices) {
    static_assert(!isCUDA, "element access needs a host view");
    return buffer[position(indices...)];
  }
  template <typename... I>
  Dtype operator()(I... indices) const {
    static_assert(!isCUDA, "element access needs a host view");
    return buffer[position(indices...)];
  }

  /// copy min(size) elements; returns the number copied
  template <bool destCUDA>
  size_t copyTo(Grid<Dtype, NumDims, destCUDA>& dest) const {
    const size_t n = std::min(size(), dest.size());
    detail::raw_copy(dest.data(), destCUDA, buffer, isCUDA, n);
    return n;
  }
  template <bool srcCUDA>
  size_t copyFrom(const Grid<Dtype, NumDims, srcCUDA>& src) {
    const size_t n = std::min(size(), src.size());
    detail::raw_copy(buffer, isCUDA, src.data(), srcCUDA, n);
    return n;
  }
  void fill_zero() { detail::raw_zero(buffer, isCUDA, size()); }

  bool operator==(const Grid& rhs) const {
    for (size_t i = 0; i < NumDims; ++i)
      if (dims[i] != rhs.dims[i]) return false;
    return buffer == rhs.buffer;
  }
};

/// one-dimensional views hand out elements instead of sub-grids
template <typename Dtype, bool isCUDA>
class Grid<Dtype, 1, isCUDA> {
  Dtype* buffer = nullptr;
  size_t dims[1] = {0};

  void check(size_t i) const {
    if (i >= dims[0])
      throw std::out_of_range("Invalid range. " + itoa(i) + " >= " + itoa(dims[0]));
  }

 public:
  using type = Dtype;
  using subgrid_t = Dtype;
  using managed_t = ManagedGrid<Dtype, 1>;
  using cpu_grid_t = Grid<Dtype, 1, false>;
  using gpu_grid_t = Grid<Dtype, 1, true>;
  static constexpr size_t N = 1;
  static constexpr bool GPU = isCUDA;

  Grid() = default;
  Grid(Dtype* d, size_t n) : buffer(d), dims{n} {}
  Grid(Dtype* d, const size_t* sizes) : buffer(d), dims{sizes[0]} {}
  explicit Grid(const Grid<Dtype, 2, isCUDA>& G, size_t i)
      : buffer(G.data() ? G.data() + i * G.offset(0) : nullptr), dims{G.dimension(1)} {}

  const size_t* dimensions() const { return dims; }
  size_t dimension(size_t i) const {
    if (i >= 1) throw std::out_of_range("Invalid dimension " + itoa(i));
    return dims[0];
  }
  size_t size() const { return dims[0]; }
  size_t offset(size_t) const { return 1; }
  Dtype* data() const { return buffer; }
  void set_buffer(Dtype* p) { buffer = p; }

  Dtype& operator[](size_t i) {
    static_assert(!isCUDA, "element access needs a host view");
    check(i);
    return buffer[i];
  }
  Dtype operator[](size_t i) const {
    static_assert(!isCUDA, "element access needs a host view");
    check(i);
    return buffer[i];
  }
  Dtype& operator()(size_t i) {
    static_assert(!isCUDA, "element access needs a host view");
    return buffer[i];
  }
  Dtype operator()(size_t i) const {
    static_assert(!isCUDA, "element access needs a host view");
    return buffer[i];
  }

  template <bool destCUDA>
  size_t copyTo(Grid<Dtype, 1, destCUDA>& dest) const {
    const size_t n = std::min(size(), dest.size());
    detail::raw_copy(dest.data(), destCUDA, buffer, isCUDA, n);
    return n;
  }
  template <bool srcCUDA>
  size_t copyFrom(const Grid<Dtype, 1, srcCUDA>& src) {
    const size_t n = std::min(size(), src.size());
    detail::raw_copy(buffer, isCUDA, src.data(), srcCUDA, n);
    return n;
  }
  void fill_zero() { detail::raw_zero(buffer, isCUDA, size()); }
  bool operator==(const Grid& rhs) const { return dims[0] == rhs.dims[0] && buffer == rhs.buffer; }
};

#define LMG_GRID_TYPEDEFS(n)                       \
  typedef Grid<float, n, false> Grid##n##f;        \
  typedef Grid<double, n, false> Grid##n##d;       \
  typedef Grid<float, n, true> Grid##n##fCUDA;     \
  typedef Grid<double, n, true> Grid##n##dCUDA;
LMG_GRID_TYPEDEFS(1)
LMG_GRID_TYPEDEFS(2)
LMG_GRID_TYPEDEFS(3)
LMG_GRID_TYPEDEFS(4)
LMG_GRID_TYPEDEFS(5)
LMG_GRID_TYPEDEFS(6)
LMG_GRID_TYPEDEFS(7)
LMG_GRID_TYPEDEFS(8)
#undef LMG_GRID_TYPEDEFS

}  // namespace libmolgrid

#endif
