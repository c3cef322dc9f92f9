// GridInterpolater: resample a 4-D grid through the inverse of a rigid transform with trilinear
// interpolation and zero padding.  Same interface as libmolgrid's GridInterpolater
// (include/libmolgrid/grid_interpolater.h:33-198); all channels are resampled by one call into
// the C ABI (mg_interpolate).
#ifndef LIBMOLGRID_GRID_INTERPOLATER_H_
#define LIBMOLGRID_GRID_INTERPOLATER_H_

#include <cmath>

#include "libmolgrid/transform.h"

namespace libmolgrid {

class GridInterpolater {
  float in_resolution, out_resolution;  // Angstroms per voxel
  float in_dimension, out_dimension;    // cube side in Angstroms
  unsigned in_dim, out_dim;             // points per side

  static unsigned points(float dimension, float resolution) {
    return std::round(dimension / resolution) + 1;
  }

  template <typename Dtype, bool isCUDA>
  void checkGrids(const Grid<Dtype, 4, isCUDA>& in, const Grid<Dtype, 4, isCUDA>& out) const {
    if (in.data() == out.data())
      throw std::invalid_argument("Input and output grid can not be the same in GridInterpolator.");
    if (in.dimension(0) != out.dimension(0))
      throw std::invalid_argument("Different channel dimensions for input and output  grids.");
    if (in.dimension(1) != in_dim || in.dimension(2) != in_dim || in.dimension(3) != in_dim)
      throw std::invalid_argument("Input grid wrong dimension. Should be " + itoa(in_dim) + " along all axes but is " +
                                  itoa(in.dimension(1)) + "," + itoa(in.dimension(2)) + "," + itoa(in.dimension(3)));
    if (out.dimension(1) != out_dim || out.dimension(2) != out_dim || out.dimension(3) != out_dim)
      throw std::invalid_argument("Output grid wrong dimension. Should be " + itoa(out_dim) + " along all axes but is " +
                                  itoa(out.dimension(1)) + "," + itoa(out.dimension(2)) + "," + itoa(out.dimension(3)));
    if (in.data() == nullptr) throw std::invalid_argument("Input grid not allocated");
    if (out.data() == nullptr) throw std::invalid_argument("Output grid not allocated");
  }

  void launch(float3 in_center, const float* in, size_t channels, const Transform& transform,
              float3 out_center, float* out) const {
    const Quaternion& Q = transform.get_quaternion();
    const float q[4] = {Q.R_component_1(), Q.R_component_2(), Q.R_component_3(), Q.R_component_4()};
    const float3 c = transform.get_rotation_center(), t = transform.get_translation();
    const float ic[3] = {in_center.x, in_center.y, in_center.z}, oc[3] = {out_center.x, out_center.y, out_center.z};
    const float rc[3] = {c.x, c.y, c.z}, tr[3] = {t.x, t.y, t.z};
    abi_check(mg_interpolate(in_resolution, in_dimension, out_resolution, out_dimension, 1, (int)channels,
                             nullptr, ic, in, nullptr, q, nullptr, rc, nullptr, tr, nullptr, oc, out, nullptr),
              "GridInterpolater::forward");
  }

 public:
  GridInterpolater(float inres, float indim, float outres, float outdim)
      : in_resolution(inres), out_resolution(outres), in_dimension(indim), out_dimension(outdim),
        in_dim(points(indim, inres)), out_dim(points(outdim, outres)) {}
  virtual ~GridInterpolater() {}

  float get_in_resolution() const { return in_resolution; }
  float get_out_resolution() const { return out_resolution; }
  float get_in_dimension() const { return in_dimension; }
  float get_out_dimension() const { return out_dimension; }
  void set_in_resolution(float res) { in_resolution = res; in_dim = points(in_dimension, in_resolution); }
  void set_out_resolution(float res) { out_resolution = res; out_dim = points(out_dimension, out_resolution); }
  void set_in_dimension(float d) { in_dimension = d; in_dim = points(in_dimension, in_resolution); }
  void set_out_dimension(float d) { out_dimension = d; out_dim = points(out_dimension, out_resolution); }

  /// in and out share the transform's rotation centre as their centre
  template <typename Dtype, bool isCUDA>
  void forward(const Grid<Dtype, 4, isCUDA>& in, const Transform& transform, Grid<Dtype, 4, isCUDA>& out) const {
    const float3 center = transform.get_rotation_center();
    forward(center, in, transform, center, out);
  }

  /// random transform about the origin
  template <typename Dtype, bool isCUDA>
  void forward(const Grid<Dtype, 4, isCUDA>& in, Grid<Dtype, 4, isCUDA>& out, float random_translation = 0,
               bool random_rotation = false) const {
    Transform t(make_float3(0.0, 0.0, 0.0), random_translation, random_rotation);
    forward(in, t, out);
  }

  /// explicit grid centres, device grids
  template <typename Dtype>
  void forward(float3 in_center, const Grid<Dtype, 4, true>& in, const Transform& transform, float3 out_center,
               Grid<Dtype, 4, true>& out) const {
    static_assert(std::is_same<Dtype, float>::value, "the HIP gridding kernels work on single precision grids");
    checkGrids(in, out);
    launch(in_center, in.data(), in.dimension(0), transform, out_center, out.data());
  }
  /// explicit grid centres, host grids (staged through the device)
  template <typename Dtype>
  void forward(float3 in_center, const Grid<Dtype, 4, false>& in, const Transform& transform, float3 out_center,
               Grid<Dtype, 4, false>& out) const {
    static_assert(std::is_same<Dtype, float>::value, "the HIP gridding kernels work on single precision grids");
    checkGrids(in, out);
    detail::DeviceStaging<float> din(in.data(), in.size()), dout(out.size());
    launch(in_center, din.get(), in.dimension(0), transform, out_center, dout.get());
    dout.download(out.data());
  }
};

/// index -> Cartesian and back (include/libmolgrid/grid_interpolater.h:189-198)
inline float3 cart2grid(float3 origin, float resolution, float x, float y, float z) {
  return make_float3((x - origin.x) / resolution, (y - origin.y) / resolution, (z - origin.z) / resolution);
}
inline float3 grid2cart(float3 origin, float resolution, unsigned i, unsigned j, unsigned k) {
  return make_float3(origin.x + i * resolution, origin.y + j * resolution, origin.z + k * resolution);
}

}  // namespace libmolgrid

#endif
