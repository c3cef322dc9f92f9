// Transform: rotate about a centre by a quaternion, then translate.  Same interface as
// libmolgrid's Transform (include/libmolgrid/transform.h:27-150); the numeric work on coordinate
// arrays is one call into the C ABI (mg_transform_forward / mg_transform_backward).
#ifndef LIBMOLGRID_TRANSFORM_H_
#define LIBMOLGRID_TRANSFORM_H_

#include <cmath>
#include <vector>

#include "libmolgrid/coordinateset.h"
#include "libmolgrid/libmolgrid.h"
#include "libmolgrid/quaternion.h"

namespace libmolgrid {

namespace detail {
/// a device copy of host data that goes away with the scope
template <typename T>
class DeviceStaging {
  T* ptr = nullptr;
  size_t count = 0;

 public:
  explicit DeviceStaging(size_t n) : count(n) {
    if (n) LMG_HIP_CHECK(hipMalloc(reinterpret_cast<void**>(&ptr), n * sizeof(T)));
  }
  DeviceStaging(const T* host, size_t n) : DeviceStaging(n) { raw_copy(ptr, true, host, false, n); }
  DeviceStaging(const DeviceStaging&) = delete;
  DeviceStaging& operator=(const DeviceStaging&) = delete;
  ~DeviceStaging() {
    if (ptr) (void)hipFree(ptr);
  }
  T* get() const { return ptr; }
  void download(T* host) const {
    LMG_HIP_CHECK(hipDeviceSynchronize());
    raw_copy(host, false, ptr, true, count);
  }
};

/// A float stand-in for a caller's grid.  For a float grid it is the grid itself.  For a double
/// grid -- the reference instantiates its overloads for Grid<double, ...> as well and computes in
/// float there too (src/grid_maker.cu:293-294, 445-446, 600; src/transform.cu:96) -- it is a float
/// copy, on the device for a device grid and on the host for a host grid: filled from the grid
/// when `load` is set, written back to it by commit().
template <typename Dtype, int N, bool isCUDA>
class AsFloat;

template <int N, bool isCUDA>
class AsFloat<float, N, isCUDA> {
  Grid<float, N, isCUDA> g;

 public:
  AsFloat(const Grid<float, N, isCUDA>& src, bool) : g(src) {}
  Grid<float, N, isCUDA>& grid() { return g; }
  void commit() {}
};

template <int N>
class AsFloat<double, N, true> {
  DeviceStaging<float> buf;
  double* orig;
  size_t count;
  Grid<float, N, true> g;

 public:
  AsFloat(const Grid<double, N, true>& src, bool load)
      : buf(src.size()), orig(const_cast<double*>(src.data())), count(src.size()) {
    size_t d[N];
    for (int i = 0; i < N; ++i) d[i] = src.dimension(i);
    g = Grid<float, N, true>(buf.get(), d);
    if (load) abi_check(mg_narrow(orig, buf.get(), count, nullptr), "double grid");
  }
  Grid<float, N, true>& grid() { return g; }
  void commit() { abi_check(mg_widen(buf.get(), orig, count, nullptr), "double grid"); }
};

template <int N>
class AsFloat<double, N, false> {
  std::vector<float> buf;
  double* orig;
  Grid<float, N, false> g;

 public:
  AsFloat(const Grid<double, N, false>& src, bool load)
      : buf(src.size()), orig(const_cast<double*>(src.data())) {
    size_t d[N];
    for (int i = 0; i < N; ++i) d[i] = src.dimension(i);
    g = Grid<float, N, false>(buf.data(), d);
    if (load)
      for (size_t i = 0; i < buf.size(); ++i) buf[i] = (float)orig[i];
  }
  Grid<float, N, false>& grid() { return g; }
  void commit() {
    for (size_t i = 0; i < buf.size(); ++i) orig[i] = (double)buf[i];
  }
};
}  // namespace detail

class Transform {
  Quaternion Q;
  float3 center = make_float3(0, 0, 0);
  float3 translate = make_float3(0, 0, 0);

  template <typename Dtype, bool isCUDA>
  void checkGrids(const Grid<Dtype, 2, isCUDA>& in, const Grid<Dtype, 2, isCUDA>& out) const {
    if (in.dimension(0) != out.dimension(0))
      throw std::invalid_argument("Different dimensions and input and output coordinates grids.");
    if (in.dimension(1) != 3) throw std::invalid_argument("Input coordinates wrong dimension.");
    if (out.dimension(1) != 3) throw std::invalid_argument("Output coordinates are wrong dimension.");
    if (in.dimension(0) == 0) return;
    if (in.data() == nullptr) throw std::invalid_argument("Input coordinates missing memory");
    if (out.data() == nullptr) throw std::invalid_argument("Output coordinates missing memory");
  }

  void launch(bool inverse, const float* in, float* out, size_t n, bool dotranslate) const {
    const float q[4] = {Q.R_component_1(), Q.R_component_2(), Q.R_component_3(), Q.R_component_4()};
    const float c[3] = {center.x, center.y, center.z};
    const float t[3] = {translate.x, translate.y, translate.z};
    auto fn = inverse ? mg_transform_backward : mg_transform_forward;
    abi_check(fn(1, nullptr, (int)n, nullptr, q, nullptr, c, nullptr, t, dotranslate ? 1 : 0, in, out,
                 nullptr),
              inverse ? "Transform::backward" : "Transform::forward");
  }

  template <typename Dtype, bool isCUDA>
  void apply(bool inverse, const Grid<Dtype, 2, isCUDA>& in, Grid<Dtype, 2, isCUDA>& out,
             bool dotranslate) const {
    checkGrids(in, out);
    const size_t n = in.dimension(0);
    if (n == 0) return;
    detail::AsFloat<Dtype, 2, isCUDA> f_in(in, true), f_out(out, false);
    if (isCUDA) {
      launch(inverse, f_in.grid().data(), f_out.grid().data(), n, dotranslate);
    } else {
      detail::DeviceStaging<float> buf(f_in.grid().data(), n * 3);
      launch(inverse, buf.get(), buf.get(), n, dotranslate);
      buf.download(f_out.grid().data());
    }
    f_out.commit();
  }

 public:
  Transform() = default;
  Transform(const Quaternion& q, float3 c = make_float3(0, 0, 0), float3 t = make_float3(0, 0, 0))
      : Q(q), center(c), translate(t) {}

  /// random transform: translation drawn first (three U(-1,1) values times random_translate),
  /// then, if asked for, a uniformly distributed rotation from three unit samples
  Transform(float3 c, float random_translate = 0.0, bool random_rotate = false) : center(c) {
    std::uniform_real_distribution<double> R(-1.0, 1);
    translate.x = R(random_engine) * random_translate;
    translate.y = R(random_engine) * random_translate;
    translate.z = R(random_engine) * random_translate;
    if (random_rotate) {
      std::uniform_real_distribution<double> unit_sample(0, 1);
      const double u1 = unit_sample(random_engine);
      const double u2 = unit_sample(random_engine);
      const double u3 = unit_sample(random_engine);
      const double s1 = std::sqrt(1 - u1), s2 = std::sqrt(u1);
      Q = Quaternion(s1 * std::sin(2 * M_PI * u2), s1 * std::cos(2 * M_PI * u2),
                     s2 * std::sin(2 * M_PI * u3), s2 * std::cos(2 * M_PI * u3));
    }
  }

  /// out = Q.rotate(in - center) + center (+ translate); in and out may be the same grid
  template <typename Dtype, bool isCUDA>
  void forward(const Grid<Dtype, 2, isCUDA>& in, Grid<Dtype, 2, isCUDA>& out, bool dotranslate = true) const {
    apply(false, in, out, dotranslate);
  }
  /// inverse: remove the translation, rotate back about center
  template <typename Dtype, bool isCUDA>
  void backward(const Grid<Dtype, 2, isCUDA>& in, Grid<Dtype, 2, isCUDA>& out, bool dotranslate = true) const {
    apply(true, in, out, dotranslate);
  }

  /// transform a coordinate set on the side its coordinates currently live on
  void forward(const CoordinateSet& in, CoordinateSet& out, bool dotranslate = true) const {
    if (in.coords.dimension(0) != out.coords.dimension(0))
      throw std::invalid_argument("Incompatible coordinateset sizes");
    if (in.coords.ongpu()) {
      Grid2fCUDA o = out.coords.gpu();
      forward(in.coords.gpu(), o, dotranslate);
    } else {
      Grid2f o = out.coords.cpu();
      forward(in.coords.cpu(), o, dotranslate);
    }
  }
  void forward(const Example& in, Example& out, bool dotranslate = true) const {
    if (in.sets.size() != out.sets.size()) throw std::invalid_argument("Incompatible example sizes");
    for (size_t i = 0; i < in.sets.size(); ++i) forward(in.sets[i], out.sets[i], dotranslate);
  }

  const Quaternion& get_quaternion() const { return Q; }
  float3 get_rotation_center() const { return center; }
  float3 get_translation() const { return translate; }
  void set_quaternion(const Quaternion& q) { Q = q; }
  void set_rotation_center(float3 c) { center = c; }
  void set_translation(float3 t) { translate = t; }

  /// true if applying this transform changes nothing
  bool is_identity() const {
    return Q == Quaternion() && translate.x == 0 && translate.y == 0 && translate.z == 0;
  }
};

}  // namespace libmolgrid

#endif
