// Transform: rotate about a centre by a quaternion, then translate.  Same interface as
// libmolgrid's Transform (include/libmolgrid/transform.h:27-150); the numeric work on coordinate
// arrays is one call into the C ABI (mg_transform_forward / mg_transform_backward).
#ifndef LIBMOLGRID_TRANSFORM_H_
#define LIBMOLGRID_TRANSFORM_H_

#include <cmath>

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
    static_assert(std::is_same<Dtype, float>::value,
                  "the HIP gridding kernels work on single precision coordinates");
    checkGrids(in, out);
    const size_t n = in.dimension(0);
    if (n == 0) return;
    if (isCUDA) {
      launch(inverse, in.data(), out.data(), n, dotranslate);
    } else {
      detail::DeviceStaging<float> buf(in.data(), n * 3);
      launch(inverse, buf.get(), buf.get(), n, dotranslate);
      buf.download(out.data());
    }
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
