// GridMaker: atoms -> density grid (forward) and grid gradient -> atom / type gradients (backward).
// Same constructor, accessors and forward/backward overload set as libmolgrid's GridMaker
// (include/libmolgrid/grid_maker.h:34-445); double precision grids are staged through float copies.  Argument checks throw the
// reference's exception types (src/grid_maker.cpp:39-89, 442-451, 487-498); the numeric work is
// one call into the C ABI per overload.  Overloads on host grids (isCUDA = false) stage their
// arrays through device memory -- the kernels are the only implementation.
#ifndef LIBMOLGRID_GRID_MAKER_H_
#define LIBMOLGRID_GRID_MAKER_H_

#include <cmath>
#include <vector>

#include "libmolgrid/coordinateset.h"
#include "libmolgrid/transform.h"

namespace libmolgrid {

class GridMaker {
 protected:
  mg_gridmaker p;           // resolution, dimension, radius multiples, A..E, dim, flags
  float grm_as_given = 1.0; // gaussian_radius_multiple as passed in (may be negative)

  /// the second-order pass exists for single precision grids only, as in the reference
  /// (src/grid_maker.cu:805: one instantiation, float)
  template <typename Dtype>
  static void require_float() {
    if (!std::is_same<Dtype, float>::value)
      throw std::invalid_argument("backward_gradients works on single precision grids");
  }
  void reinit(float res, float d) {
    abi_check(mg_gridmaker_init(&p, res, d, p.binary, p.radii_type_indexed, p.radius_scale, grm_as_given),
              "GridMaker");
  }
  const float* null3() const { return nullptr; }

  template <typename Dtype, bool isCUDA>
  void check_index_args(const Grid<float, 2, isCUDA>& coords, const Grid<float, 1, isCUDA>& type_index,
                        const Grid<float, 1, isCUDA>& radii, const Grid<Dtype, 4, isCUDA>& out) const {
    const size_t N = coords.dimension(0);
    for (int ax = 1; ax <= 3; ++ax)
      if (p.dim != out.dimension(ax))
        throw std::out_of_range("Output grid dimension incorrect: " + itoa(p.dim) + " vs " + itoa(out.dimension(ax)));
    if (type_index.size() != N)
      throw std::out_of_range("type_index does not match number of atoms: " + itoa(type_index.size()) + " vs " + itoa(N));
    if (radii.size() != N)
      throw std::out_of_range("radii does not match number of atoms: " + itoa(radii.size()) + " vs " + itoa(N));
  }
  template <typename Dtype, bool isCUDA>
  void check_vector_args(const Grid<float, 2, isCUDA>& coords, const Grid<float, 2, isCUDA>& type_vector,
                         const Grid<float, 1, isCUDA>& radii, const Grid<Dtype, 4, isCUDA>& out) const {
    const size_t N = coords.dimension(0), T = type_vector.dimension(1);
    for (int ax = 1; ax <= 3; ++ax)
      if (p.dim != out.dimension(ax))
        throw std::out_of_range("Output grid dimension incorrect: " + itoa(p.dim) + " vs " + itoa(out.dimension(ax)));
    if (type_vector.dimension(0) != N)
      throw std::out_of_range("type_vector does not match number of atoms: " + itoa(type_vector.dimension(0)) + " vs " + itoa(N));
    if (T != out.dimension(0))
      throw std::out_of_range("number of types in type_vector does not match number of output channels: " + itoa(T) + " vs " + itoa(out.dimension(0)));
    const size_t want = p.radii_type_indexed ? T : N;
    if (radii.size() != want)
      throw std::out_of_range(std::string("radii does not match number of ") + (p.radii_type_indexed ? "types: " : "atoms: ") + itoa(radii.size()) + " vs " + itoa(want));
  }

 public:
  GridMaker(float res = 0, float d = 0, bool bin = false, bool rti = false, float rscale = 1.0, float grm = 1.0) {
    p = mg_gridmaker{};
    p.binary = bin;
    p.radii_type_indexed = rti;
    p.radius_scale = rscale;
    initialize(res, d, bin, rscale, grm);
  }
  virtual ~GridMaker() {}

  void initialize(float res, float d, bool bin = false, float rscale = 1.0, float grm = 1.0) {
    grm_as_given = grm;
    const int rti = p.radii_type_indexed;
    abi_check(mg_gridmaker_init(&p, res, d, bin, rti, rscale, grm), "GridMaker::initialize");
  }

  float3 get_grid_dims() const { return make_float3(p.dim, p.dim, p.dim); }
  float get_resolution() const { return p.resolution; }
  void set_resolution(float res) { reinit(res, p.dimension); }
  float get_dimension() const { return p.dimension; }
  void set_dimension(float d) { reinit(p.resolution, d); }
  unsigned get_first_dim() const { return p.dim; }
  bool get_binary() const { return p.binary != 0; }
  void set_binary(bool b) { p.binary = b; }
  bool get_radii_type_indexed() const { return p.radii_type_indexed != 0; }
  void set_radii_type_indexed(bool b) { p.radii_type_indexed = b; }
  float get_radiusmultiple() const { return p.radius_scale * p.final_radius_multiple; }
  const mg_gridmaker& params() const { return p; }

  /// first corner of the grid for a given centre
  float3 get_grid_origin(const float3& grid_center) const {
    const float half = p.dimension / 2.0;
    return make_float3(grid_center.x - half, grid_center.y - half, grid_center.z - half);
  }

  // ---- forward ---------------------------------------------------------------------------

  /// coordinate set -> grid, on the side the grid lives on
  template <typename Dtype>
  void forward(float3 grid_center, const CoordinateSet& in, Grid<Dtype, 4, false>& out) const {
    if (in.has_vector_types() && in.size() > 0)
      forward(grid_center, in.coords.cpu(), in.type_vector.cpu(), in.radii.cpu(), out);
    else
      forward(grid_center, in.coords.cpu(), in.type_index.cpu(), in.radii.cpu(), out);
  }
  template <typename Dtype>
  void forward(float3 grid_center, const CoordinateSet& in, Grid<Dtype, 4, true>& out) const {
    if (in.has_vector_types() && in.size() > 0)
      forward(grid_center, in.coords.gpu(), in.type_vector.gpu(), in.radii.gpu(), out);
    else
      forward(grid_center, in.coords.gpu(), in.type_index.gpu(), in.radii.gpu(), out);
  }

  /// example -> grid with an explicit transformation; the transform's centre is the grid centre
  template <typename Dtype, bool isCUDA>
  void forward(const Example& in, const Transform& transform, Grid<Dtype, 4, isCUDA>& out) const {
    CoordinateSet c = in.merge_coordinates();  // a copy: safe to transform in place
    if (c.max_type != out.dimension(0))
      throw std::out_of_range("Incorrect number of channels in output grid: " + itoa(c.max_type) + " vs " + itoa(out.dimension(0)));
    if (isCUDA) c.togpu();
    transform.forward(c, c);
    forward(transform.get_rotation_center(), c, out);
  }

  /// example -> grid with a random transformation about `center` (default: the centre of the
  /// last non-empty coordinate set)
  template <typename Dtype, bool isCUDA>
  void forward(const Example& in, Grid<Dtype, 4, isCUDA>& out, float random_translation = 0.0,
               bool random_rotation = false,
               const float3& center = make_float3(INFINITY, INFINITY, INFINITY)) const {
    float3 c = center;
    if (std::isinf(c.x)) {
      c = make_float3(0, 0, 0);
      for (int i = (int)in.sets.size() - 1; i >= 0; --i) {
        if (in.sets[i].size()) {
          c = in.sets.back().center();
          break;
        }
      }
    }
    Transform t(c, random_translation, random_rotation);
    forward(in, t, out);
  }

  /// batch of examples -> 5-D grid.  Index-typed examples are merged and packed on the host once,
  /// uploaded once, and gridded with two launches for the whole batch (transform, splat); each
  /// example gets its own random transformation about its own centre, as in the per-example call.
  template <typename Dtype, bool isCUDA>
  void forward(const std::vector<Example>& in, Grid<Dtype, 5, isCUDA>& out, float random_translation = 0.0,
               bool random_rotation = false) const {
    if (in.size() != out.dimension(0))
      throw std::out_of_range("output grid dimension does not match size of example vector");
    const size_t B = in.size();
    if (B == 0) return;
    std::vector<CoordinateSet> merged(B);
    bool packable = true;
    size_t total = 0;
    for (size_t i = 0; i < B; ++i) {
      merged[i] = in[i].merge_coordinates();
      if (merged[i].max_type != out.dimension(1))
        throw std::out_of_range("Incorrect number of channels in output grid: " + itoa(merged[i].max_type) + " vs " + itoa(out.dimension(1)));
      if (merged[i].has_vector_types() && merged[i].size() > 0) packable = false;
      total += merged[i].size();
    }
    if (!packable || p.radii_type_indexed) {  // vector-typed sets: example by example
      for (size_t i = 0; i < B; ++i) {
        Grid<Dtype, 4, isCUDA> g(out[i]);
        forward<Dtype, isCUDA>(in[i], g, random_translation, random_rotation);
      }
      return;
    }
    std::vector<float> coords(total * 3), types(total), radii(total), quats(B * 4), centers(B * 3), shifts(B * 3);
    std::vector<int> offsets(B + 1, 0);
    int longest = 1;
    for (size_t i = 0, at = 0; i < B; ++i) {
      const CoordinateSet& c = merged[i];
      const size_t n = c.size();
      float3 cen = make_float3(0, 0, 0);
      for (int k = (int)in[i].sets.size() - 1; k >= 0; --k)
        if (in[i].sets[k].size()) {
          cen = in[i].sets.back().center();
          break;
        }
      Transform t(cen, random_translation, random_rotation);
      const Quaternion& q = t.get_quaternion();
      const float3 tr = t.get_translation();
      const float qv[4] = {q.R_component_1(), q.R_component_2(), q.R_component_3(), q.R_component_4()};
      std::copy(qv, qv + 4, quats.begin() + 4 * i);
      centers[3 * i] = cen.x, centers[3 * i + 1] = cen.y, centers[3 * i + 2] = cen.z;
      shifts[3 * i] = tr.x, shifts[3 * i + 1] = tr.y, shifts[3 * i + 2] = tr.z;
      if (n) {
        std::copy(c.coords.cpu().data(), c.coords.cpu().data() + 3 * n, coords.begin() + 3 * at);
        std::copy(c.type_index.cpu().data(), c.type_index.cpu().data() + n, types.begin() + at);
        std::copy(c.radii.cpu().data(), c.radii.cpu().data() + n, radii.begin() + at);
      }
      at += n;
      offsets[i + 1] = (int)at;
      longest = std::max(longest, (int)n);
    }
    detail::DeviceStaging<float> dc(coords.data(), coords.size()), dt(types.data(), total), dr(radii.data(), total);
    detail::DeviceStaging<float> dq(quats.data(), quats.size()), dcen(centers.data(), centers.size()), dsh(shifts.data(), shifts.size());
    detail::DeviceStaging<int> doff(offsets.data(), offsets.size());
    const float zero3[3] = {0, 0, 0}, ident[4] = {1, 0, 0, 0};
    if (total)
      abi_check(mg_transform_forward((int)B, doff.get(), longest, dq.get(), ident, dcen.get(), zero3, dsh.get(), zero3,
                                     1, dc.get(), dc.get(), nullptr),
                "GridMaker::forward");
    detail::AsFloat<Dtype, 5, isCUDA> f_out(out, false);
    if (isCUDA) {
      abi_check(mg_forward_index(&p, (int)B, doff.get(), longest, dcen.get(), zero3, dc.get(), dt.get(), dr.get(),
                                 (int)out.dimension(1), f_out.grid().data(), nullptr),
                "GridMaker::forward");
      f_out.commit();
      LMG_HIP_CHECK(hipDeviceSynchronize());  // the staged inputs are released on return
    } else {
      detail::DeviceStaging<float> dout(out.size());
      abi_check(mg_forward_index(&p, (int)B, doff.get(), longest, dcen.get(), zero3, dc.get(), dt.get(), dr.get(),
                                 (int)out.dimension(1), dout.get(), nullptr),
                "GridMaker::forward");
      dout.download(f_out.grid().data());
      f_out.commit();
    }
  }

  /// index types, device arrays: one launch
  template <typename Dtype>
  void forward(float3 grid_center, const Grid<float, 2, true>& coords, const Grid<float, 1, true>& type_index,
               const Grid<float, 1, true>& radii, Grid<Dtype, 4, true>& out) const {
    detail::AsFloat<Dtype, 4, true> f_out(out, false);
    check_index_args(coords, type_index, radii, out);
    if (p.radii_type_indexed) throw std::invalid_argument("Type indexed radii not supported with index types.");
    const float c[3] = {grid_center.x, grid_center.y, grid_center.z};
    abi_check(mg_forward_index(&p, 1, nullptr, (int)coords.dimension(0), nullptr, c, coords.data(),
                               type_index.data(), radii.data(), (int)out.dimension(0),
                               f_out.grid().data(), nullptr),
              "GridMaker::forward");
    f_out.commit();
  }
  /// index types, host arrays
  template <typename Dtype>
  void forward(float3 grid_center, const Grid<float, 2, false>& coords, const Grid<float, 1, false>& type_index,
               const Grid<float, 1, false>& radii, Grid<Dtype, 4, false>& out) const {
    detail::AsFloat<Dtype, 4, false> f_out(out, false);
    check_index_args(coords, type_index, radii, out);
    if (p.radii_type_indexed) throw std::invalid_argument("Type indexed radii not supported with index types.");
    const size_t n = coords.dimension(0);
    const int64_t ntypes = out.dimension(0);
    for (size_t i = 0; i < n; ++i) {
      const int64_t t = std::floor(type_index(i));
      if (t >= ntypes) throw std::out_of_range("Type index " + itoa(t) + " larger than allowed " + itoa(ntypes));
    }
    detail::DeviceStaging<float> dc(coords.data(), n * 3), dt(type_index.data(), n), dr(radii.data(), n);
    detail::DeviceStaging<float> dout(out.size());
    Grid<float, 2, true> gc(dc.get(), n, 3);
    Grid<float, 1, true> gt(dt.get(), n), gr(dr.get(), n);
    Grid<float, 4, true> go(dout.get(), out.dimension(0), out.dimension(1), out.dimension(2), out.dimension(3));
    forward(grid_center, gc, gt, gr, go);
    dout.download(f_out.grid().data());
    f_out.commit();
  }

  /// vector types, device arrays: one launch
  template <typename Dtype>
  void forward(float3 grid_center, const Grid<float, 2, true>& coords, const Grid<float, 2, true>& type_vector,
               const Grid<float, 1, true>& radii, Grid<Dtype, 4, true>& out) const {
    detail::AsFloat<Dtype, 4, true> f_out(out, false);
    check_vector_args(coords, type_vector, radii, out);
    const float c[3] = {grid_center.x, grid_center.y, grid_center.z};
    abi_check(mg_forward_vector(&p, 1, nullptr, (int)coords.dimension(0), nullptr, c, coords.data(),
                                type_vector.data(), radii.data(), (int)out.dimension(0),
                                f_out.grid().data(), nullptr),
              "GridMaker::forward");
    f_out.commit();
  }
  /// vector types, host arrays
  template <typename Dtype>
  void forward(float3 grid_center, const Grid<float, 2, false>& coords, const Grid<float, 2, false>& type_vector,
               const Grid<float, 1, false>& radii, Grid<Dtype, 4, false>& out) const {
    detail::AsFloat<Dtype, 4, false> f_out(out, false);
    check_vector_args(coords, type_vector, radii, out);
    const size_t n = coords.dimension(0), T = type_vector.dimension(1);
    detail::DeviceStaging<float> dc(coords.data(), n * 3), dt(type_vector.data(), n * T), dr(radii.data(), radii.size());
    detail::DeviceStaging<float> dout(out.size());
    Grid<float, 2, true> gc(dc.get(), n, 3), gt(dt.get(), n, T);
    Grid<float, 1, true> gr(dr.get(), radii.size());
    Grid<float, 4, true> go(dout.get(), out.dimension(0), out.dimension(1), out.dimension(2), out.dimension(3));
    forward(grid_center, gc, gt, gr, go);
    dout.download(f_out.grid().data());
    f_out.commit();
  }

  /// padded batch: centers (B x 3), coords (B x N x 3), types (B x N) or (B x N x T), radii (B x N)
  /// -> out (B x T x D x D x D).  On the device this is ONE launch for the whole batch.
  template <typename Dtype, int N, bool isCUDA>
  void forward(const Grid<float, 2, isCUDA>& centers, const Grid<float, 3, isCUDA>& coords,
               const Grid<float, N, isCUDA>& types, const Grid<float, 2, isCUDA>& radii,
               Grid<Dtype, 5, isCUDA>& out) const {
    static_assert(N == 2 || N == 3, "Unsupported types dimension");
    const size_t B = centers.dimension(0);
    if (coords.dimension(0) != B) throw std::invalid_argument("Mismatched batch sizes: " + itoa(coords.dimension(0)) + " vs " + itoa(B));
    if (types.dimension(0) != B) throw std::invalid_argument("Mismatched batch sizes: " + itoa(types.dimension(0)) + " vs " + itoa(B));
    if (radii.dimension(0) != B) throw std::invalid_argument("Mismatched batch sizes: " + itoa(radii.dimension(0)) + " vs " + itoa(B));
    if (out.dimension(0) != B) throw std::invalid_argument("Mismatched batch sizes: " + itoa(out.dimension(0)) + " vs " + itoa(B));
    if (B == 0) return;
    if (!isCUDA) {  // host arrays: example by example through the staging overloads
      this->template forward_host_batch<Dtype, N>(centers, coords, types, radii, out,
                                                  std::integral_constant<bool, isCUDA>());
      return;
    }
    {  // validate one example's shapes, they are all alike
      Grid<float, 2, isCUDA> C = coords[0];
      Grid<float, N - 1, isCUDA> T = types[0];
      Grid<float, 1, isCUDA> R = radii[0];
      Grid<Dtype, 4, isCUDA> O = out[0];
      check_batch_example(C, T, R, O);
    }
    const int n = (int)coords.dimension(1);
    auto fn = N == 2 ? mg_forward_index : mg_forward_vector;
    detail::AsFloat<Dtype, 5, isCUDA> f_out(out, false);
    abi_check(fn(&p, (int)B, nullptr, n, centers.data(), nullptr, coords.data(), types.data(), radii.data(),
                 (int)out.dimension(1), f_out.grid().data(), nullptr),
              "GridMaker::forward");
    f_out.commit();
  }

  // ---- backward --------------------------------------------------------------------------

  /// coordinate set with vector types (host / device grids)
  template <typename Dtype>
  void backward(float3 grid_center, const CoordinateSet& in, const Grid<Dtype, 4, false>& diff,
                Grid<Dtype, 2, false>& atomic_gradients, Grid<Dtype, 2, false>& type_gradients) const {
    if (!in.has_vector_types()) throw std::invalid_argument("Vector types missing from coordinate set");
    backward(grid_center, in.coords.cpu(), in.type_vector.cpu(), in.radii.cpu(), diff, atomic_gradients, type_gradients);
  }
  template <typename Dtype>
  void backward(float3 grid_center, const CoordinateSet& in, const Grid<Dtype, 4, true>& diff,
                Grid<Dtype, 2, true>& atomic_gradients, Grid<Dtype, 2, true>& type_gradients) const {
    if (!in.has_vector_types()) throw std::invalid_argument("Vector types missing from coordinate set");
    backward(grid_center, in.coords.gpu(), in.type_vector.gpu(), in.radii.gpu(), diff, atomic_gradients, type_gradients);
  }
  /// coordinate set with index types (host / device grids)
  template <typename Dtype>
  void backward(float3 grid_center, const CoordinateSet& in, const Grid<Dtype, 4, false>& diff,
                Grid<Dtype, 2, false>& atomic_gradients) const {
    if (!in.has_indexed_types()) throw std::invalid_argument("Index types missing from coordinate set");
    backward(grid_center, in.coords.cpu(), in.type_index.cpu(), in.radii.cpu(), diff, atomic_gradients);
  }
  template <typename Dtype>
  void backward(float3 grid_center, const CoordinateSet& in, const Grid<Dtype, 4, true>& diff,
                Grid<Dtype, 2, true>& atomic_gradients) const {
    if (!in.has_indexed_types()) throw std::invalid_argument("Index types missing from coordinate set");
    backward(grid_center, in.coords.gpu(), in.type_index.gpu(), in.radii.gpu(), diff, atomic_gradients);
  }

  /// index types, device arrays
  template <typename Dtype>
  void backward(float3 grid_center, const Grid<float, 2, true>& coords, const Grid<float, 1, true>& type_index,
                const Grid<float, 1, true>& radii, const Grid<Dtype, 4, true>& diff,
                Grid<Dtype, 2, true>& atom_gradients) const {
    detail::AsFloat<Dtype, 4, true> f_diff(diff, true);
    detail::AsFloat<Dtype, 2, true> f_grad(atom_gradients, false);
    check_backward_index(coords, type_index, radii, diff, atom_gradients);
    const float c[3] = {grid_center.x, grid_center.y, grid_center.z};
    abi_check(mg_backward_index(&p, 1, nullptr, (int)coords.dimension(0), nullptr, c, coords.data(),
                                type_index.data(), radii.data(), (int)diff.dimension(0),
                                f_diff.grid().data(), f_grad.grid().data(), nullptr),
              "GridMaker::backward");
    f_grad.commit();
  }
  /// index types, host arrays
  template <typename Dtype>
  void backward(float3 grid_center, const Grid<float, 2, false>& coords, const Grid<float, 1, false>& type_index,
                const Grid<float, 1, false>& radii, const Grid<Dtype, 4, false>& diff,
                Grid<Dtype, 2, false>& atom_gradients) const {
    detail::AsFloat<Dtype, 4, false> f_diff(diff, true);
    detail::AsFloat<Dtype, 2, false> f_grad(atom_gradients, false);
    check_backward_index(coords, type_index, radii, diff, atom_gradients);
    const size_t n = coords.dimension(0);
    for (size_t i = 0; i < n; ++i) {
      const int which = std::round(type_index(i));
      if (which >= 0 && (unsigned)which >= diff.dimension(0))
        throw std::invalid_argument("Incorrect channel size for diff: " + itoa(which) + " vs " + itoa(diff.dimension(0)));
    }
    detail::DeviceStaging<float> dc(coords.data(), n * 3), dt(type_index.data(), n), dr(radii.data(), n);
    detail::DeviceStaging<float> dd(f_diff.grid().data(), diff.size()), dg(n * 3);
    Grid<float, 2, true> gc(dc.get(), n, 3), gg(dg.get(), n, 3);
    Grid<float, 1, true> gt(dt.get(), n), gr(dr.get(), n);
    Grid<float, 4, true> gd(dd.get(), diff.dimension(0), diff.dimension(1), diff.dimension(2), diff.dimension(3));
    backward(grid_center, gc, gt, gr, gd, gg);
    dg.download(f_grad.grid().data());
    f_grad.commit();
  }

  /// vector types, device arrays
  template <typename Dtype>
  void backward(float3 grid_center, const Grid<float, 2, true>& coords, const Grid<float, 2, true>& type_vectors,
                const Grid<float, 1, true>& radii, const Grid<Dtype, 4, true>& diff,
                Grid<Dtype, 2, true>& atom_gradients, Grid<Dtype, 2, true>& type_gradients) const {
    detail::AsFloat<Dtype, 4, true> f_diff(diff, true);
    detail::AsFloat<Dtype, 2, true> f_grad(atom_gradients, false), f_tgrad(type_gradients, false);
    check_backward_vector(coords, type_vectors, radii, diff, atom_gradients, type_gradients);
    const float c[3] = {grid_center.x, grid_center.y, grid_center.z};
    abi_check(mg_backward_vector(&p, 1, nullptr, (int)coords.dimension(0), nullptr, c, coords.data(),
                                 type_vectors.data(), radii.data(), (int)diff.dimension(0),
                                 f_diff.grid().data(), f_grad.grid().data(), f_tgrad.grid().data(), nullptr),
              "GridMaker::backward");
    f_grad.commit();
    f_tgrad.commit();
  }
  /// vector types, host arrays
  template <typename Dtype>
  void backward(float3 grid_center, const Grid<float, 2, false>& coords, const Grid<float, 2, false>& type_vectors,
                const Grid<float, 1, false>& radii, const Grid<Dtype, 4, false>& diff,
                Grid<Dtype, 2, false>& atom_gradients, Grid<Dtype, 2, false>& type_gradients) const {
    detail::AsFloat<Dtype, 4, false> f_diff(diff, true);
    detail::AsFloat<Dtype, 2, false> f_grad(atom_gradients, false), f_tgrad(type_gradients, false);
    check_backward_vector(coords, type_vectors, radii, diff, atom_gradients, type_gradients);
    const size_t n = coords.dimension(0), T = type_vectors.dimension(1);
    detail::DeviceStaging<float> dc(coords.data(), n * 3), dt(type_vectors.data(), n * T), dr(radii.data(), radii.size());
    detail::DeviceStaging<float> dd(f_diff.grid().data(), diff.size()), dg(n * 3), dtg(n * T);
    Grid<float, 2, true> gc(dc.get(), n, 3), gt(dt.get(), n, T), gg(dg.get(), n, 3), gtg(dtg.get(), n, T);
    Grid<float, 1, true> gr(dr.get(), radii.size());
    Grid<float, 4, true> gd(dd.get(), diff.dimension(0), diff.dimension(1), diff.dimension(2), diff.dimension(3));
    backward(grid_center, gc, gt, gr, gd, gg, gtg);
    dg.download(f_grad.grid().data());
    dtg.download(f_tgrad.grid().data());
    f_grad.commit();
    f_tgrad.commit();
  }

  // ---- relevance (include/libmolgrid/grid_maker.h:547-618 of the reference) ----------------
  /// index types, device arrays
  template <typename Dtype>
  void backward_relevance(float3 grid_center, const Grid<float, 2, true>& coords,
                          const Grid<float, 1, true>& type_index, const Grid<float, 1, true>& radii,
                          const Grid<Dtype, 4, true>& density, const Grid<Dtype, 4, true>& diff,
                          Grid<Dtype, 1, true>& relevance) const {
    detail::AsFloat<Dtype, 4, true> f_dens(density, true), f_diff(diff, true);
    detail::AsFloat<Dtype, 1, true> f_rel(relevance, false);
    check_relevance(coords, type_index, radii, density, diff, relevance);
    const float c[3] = {grid_center.x, grid_center.y, grid_center.z};
    abi_check(mg_backward_relevance(&p, 1, nullptr, (int)coords.dimension(0), nullptr, c, coords.data(),
                                    type_index.data(), radii.data(), (int)diff.dimension(0),
                                    f_dens.grid().data(), f_diff.grid().data(), f_rel.grid().data(), nullptr),
              "GridMaker::backward_relevance");
    f_rel.commit();
  }
  /// index types, host arrays
  template <typename Dtype>
  void backward_relevance(float3 grid_center, const Grid<float, 2, false>& coords,
                          const Grid<float, 1, false>& type_index, const Grid<float, 1, false>& radii,
                          const Grid<Dtype, 4, false>& density, const Grid<Dtype, 4, false>& diff,
                          Grid<Dtype, 1, false>& relevance) const {
    detail::AsFloat<Dtype, 4, false> f_dens(density, true), f_diff(diff, true);
    detail::AsFloat<Dtype, 1, false> f_rel(relevance, false);
    check_relevance(coords, type_index, radii, density, diff, relevance);
    const size_t n = coords.dimension(0);
    detail::DeviceStaging<float> dc(coords.data(), n * 3), dt(type_index.data(), n), dr(radii.data(), n);
    detail::DeviceStaging<float> dd(f_dens.grid().data(), density.size());
    detail::DeviceStaging<float> df(f_diff.grid().data(), diff.size()), drel(n);
    Grid<float, 2, true> gc(dc.get(), n, 3);
    Grid<float, 1, true> gt(dt.get(), n), gr(dr.get(), n), grel(drel.get(), n);
    Grid<float, 4, true> gd(dd.get(), diff.dimension(0), diff.dimension(1), diff.dimension(2), diff.dimension(3));
    Grid<float, 4, true> gf(df.get(), diff.dimension(0), diff.dimension(1), diff.dimension(2), diff.dimension(3));
    backward_relevance(grid_center, gc, gt, gr, gd, gf, grel);
    drel.download(f_rel.grid().data());
    f_rel.commit();
  }
  /// coordinate set (host / device grids)
  template <typename Dtype>
  void backward_relevance(float3 grid_center, const CoordinateSet& in, const Grid<Dtype, 4, false>& density,
                          const Grid<Dtype, 4, false>& diff, Grid<Dtype, 1, false>& relevance) const {
    if (!in.has_indexed_types()) throw std::invalid_argument("Index types missing from coordinate set in backward relevance");
    backward_relevance(grid_center, in.coords.cpu(), in.type_index.cpu(), in.radii.cpu(), density, diff, relevance);
  }
  template <typename Dtype>
  void backward_relevance(float3 grid_center, const CoordinateSet& in, const Grid<Dtype, 4, true>& density,
                          const Grid<Dtype, 4, true>& diff, Grid<Dtype, 1, true>& relevance) const {
    if (!in.has_indexed_types()) throw std::invalid_argument("Index types missing from coordinate set in backward relevance");
    backward_relevance(grid_center, in.coords.gpu(), in.type_index.gpu(), in.radii.gpu(), density, diff, relevance);
  }

  // ---- gradients of the backward pass (grid_maker.h:447-545 of the reference) --------------
  /// vector types, device arrays; the three outputs are overwritten
  template <typename Dtype>
  void backward_gradients(float3 grid_center, const Grid<float, 2, true>& coords,
                          const Grid<float, 2, true>& type_vectors, const Grid<float, 1, true>& radii,
                          const Grid<Dtype, 4, true>& diff, const Grid<Dtype, 2, true>& atom_gradients,
                          const Grid<Dtype, 2, true>& type_gradients, Grid<Dtype, 4, true>& diffdiff,
                          Grid<Dtype, 2, true>& atom_diffdiff, Grid<Dtype, 2, true>& type_diffdiff) const {
    require_float<Dtype>();
    check_backward_gradients(coords, type_vectors, radii, diff, atom_gradients, type_gradients, diffdiff,
                             atom_diffdiff, type_diffdiff);
    const float c[3] = {grid_center.x, grid_center.y, grid_center.z};
    abi_check(mg_backward_gradients(&p, 1, nullptr, (int)coords.dimension(0), nullptr, c, coords.data(),
                                    type_vectors.data(), radii.data(), (int)diff.dimension(0),
                                    reinterpret_cast<const float*>(diff.data()),
                                    reinterpret_cast<const float*>(atom_gradients.data()),
                                    reinterpret_cast<const float*>(type_gradients.data()),
                                    reinterpret_cast<float*>(diffdiff.data()),
                                    reinterpret_cast<float*>(atom_diffdiff.data()),
                                    reinterpret_cast<float*>(type_diffdiff.data()), nullptr),
              "GridMaker::backward_gradients");
  }
  /// vector types, host arrays
  template <typename Dtype>
  void backward_gradients(float3 grid_center, const Grid<float, 2, false>& coords,
                          const Grid<float, 2, false>& type_vectors, const Grid<float, 1, false>& radii,
                          const Grid<Dtype, 4, false>& diff, const Grid<Dtype, 2, false>& atom_gradients,
                          const Grid<Dtype, 2, false>& type_gradients, Grid<Dtype, 4, false>& diffdiff,
                          Grid<Dtype, 2, false>& atom_diffdiff, Grid<Dtype, 2, false>& type_diffdiff) const {
    require_float<Dtype>();
    check_backward_gradients(coords, type_vectors, radii, diff, atom_gradients, type_gradients, diffdiff,
                             atom_diffdiff, type_diffdiff);
    const size_t n = coords.dimension(0), T = type_vectors.dimension(1);
    detail::DeviceStaging<float> dc(coords.data(), n * 3), dt(type_vectors.data(), n * T), dr(radii.data(), radii.size());
    detail::DeviceStaging<float> dd(reinterpret_cast<const float*>(diff.data()), diff.size());
    detail::DeviceStaging<float> dag(reinterpret_cast<const float*>(atom_gradients.data()), n * 3);
    detail::DeviceStaging<float> dtg(reinterpret_cast<const float*>(type_gradients.data()), n * T);
    detail::DeviceStaging<float> odd(diff.size()), oad(n * 3), otd(n * T);
    Grid<float, 2, true> gc(dc.get(), n, 3), gt(dt.get(), n, T), gag(dag.get(), n, 3), gtg(dtg.get(), n, T);
    Grid<float, 2, true> goad(oad.get(), n, 3), gotd(otd.get(), n, T);
    Grid<float, 1, true> gr(dr.get(), radii.size());
    Grid<float, 4, true> gd(dd.get(), diff.dimension(0), diff.dimension(1), diff.dimension(2), diff.dimension(3));
    Grid<float, 4, true> godd(odd.get(), diff.dimension(0), diff.dimension(1), diff.dimension(2), diff.dimension(3));
    backward_gradients(grid_center, gc, gt, gr, gd, gag, gtg, godd, goad, gotd);
    odd.download(reinterpret_cast<float*>(diffdiff.data()));
    oad.download(reinterpret_cast<float*>(atom_diffdiff.data()));
    otd.download(reinterpret_cast<float*>(type_diffdiff.data()));
  }
  /// coordinate set with vector types (host / device grids)
  template <typename Dtype>
  void backward_gradients(float3 grid_center, const CoordinateSet& in, const Grid<Dtype, 4, false>& diff,
                          const Grid<Dtype, 2, false>& atom_gradients, const Grid<Dtype, 2, false>& type_gradients,
                          Grid<Dtype, 4, false>& diffdiff, Grid<Dtype, 2, false>& atom_diffdiff,
                          Grid<Dtype, 2, false>& type_diffdiff) const {
    if (!in.has_vector_types()) throw std::invalid_argument("Vector types missing from coordinate set");
    backward_gradients(grid_center, in.coords.cpu(), in.type_vector.cpu(), in.radii.cpu(), diff, atom_gradients,
                       type_gradients, diffdiff, atom_diffdiff, type_diffdiff);
  }
  template <typename Dtype>
  void backward_gradients(float3 grid_center, const CoordinateSet& in, const Grid<Dtype, 4, true>& diff,
                          const Grid<Dtype, 2, true>& atom_gradients, const Grid<Dtype, 2, true>& type_gradients,
                          Grid<Dtype, 4, true>& diffdiff, Grid<Dtype, 2, true>& atom_diffdiff,
                          Grid<Dtype, 2, true>& type_diffdiff) const {
    if (!in.has_vector_types()) throw std::invalid_argument("Vector types missing from coordinate set");
    backward_gradients(grid_center, in.coords.gpu(), in.type_vector.gpu(), in.radii.gpu(), diff, atom_gradients,
                       type_gradients, diffdiff, atom_diffdiff, type_diffdiff);
  }

 private:
  template <typename Dtype, bool isCUDA>
  void check_relevance(const Grid<float, 2, isCUDA>& coords, const Grid<float, 1, isCUDA>& type_index,
                       const Grid<float, 1, isCUDA>& radii, const Grid<Dtype, 4, isCUDA>& density,
                       const Grid<Dtype, 4, isCUDA>& diff, const Grid<Dtype, 1, isCUDA>& relevance) const {
    const unsigned n = coords.dimension(0);
    if (n != type_index.size()) throw std::invalid_argument("Type dimension doesn't equal number of coordinates.");
    if (n != relevance.size()) throw std::invalid_argument("Relevance dimension doesn't equal number of coordinates");
    if (n != radii.size()) throw std::invalid_argument("Radii dimension doesn't equal number of coordinates");
    if (coords.dimension(1) != 3) throw std::invalid_argument("Coordinates and radius wrong secondary dimension");
    for (unsigned i = 0; i <= 3; ++i)
      if (density.dimension(i) != diff.dimension(i) || (i > 0 && diff.dimension(i) != p.dim))
        throw std::invalid_argument("density and diff do not have the grid's dimensions");
  }
  template <typename Dtype, bool isCUDA>
  void check_backward_gradients(const Grid<float, 2, isCUDA>& coords, const Grid<float, 2, isCUDA>& type_vector,
                                const Grid<float, 1, isCUDA>& radii, const Grid<Dtype, 4, isCUDA>& diff,
                                const Grid<Dtype, 2, isCUDA>& atom_gradients,
                                const Grid<Dtype, 2, isCUDA>& type_gradients,
                                const Grid<Dtype, 4, isCUDA>& diffdiff,
                                const Grid<Dtype, 2, isCUDA>& atom_diffdiff,
                                const Grid<Dtype, 2, isCUDA>& type_diffdiff) const {
    check_backward_vector(coords, type_vector, radii, diff, atom_gradients, type_gradients);
    const unsigned n = coords.dimension(0), ntypes = type_vector.dimension(1);
    if (n != atom_diffdiff.dimension(0)) throw std::invalid_argument("Atom gradient gradients dimension doesn't equal number of coordinates");
    if (n != type_diffdiff.dimension(0)) throw std::invalid_argument("Type gradient gradients dimension doesn't equal number of coordinates");
    if (type_diffdiff.dimension(1) != ntypes) throw std::invalid_argument("Type gradient dimension has wrong number of types");
    if (p.binary) throw std::invalid_argument("Binary densities not supported");
    for (unsigned i = 0; i <= 3; ++i)
      if (diffdiff.dimension(i) != diff.dimension(i))
        throw std::invalid_argument("diffdiff does not have the dimensions of diff");
  }

  template <typename Dtype, int N>
  void forward_host_batch(const Grid<float, 2, false>& centers, const Grid<float, 3, false>& coords,
                          const Grid<float, N, false>& types, const Grid<float, 2, false>& radii,
                          Grid<Dtype, 5, false>& out, std::false_type) const {
    for (unsigned i = 0, B = centers.dimension(0); i < B; ++i) {
      const float3 center = make_float3(centers(i, 0), centers(i, 1), centers(i, 2));
      Grid<float, 2, false> C = coords[i];
      Grid<float, N - 1, false> T = types[i];
      Grid<float, 1, false> R = radii[i];
      Grid<Dtype, 4, false> O = out[i];
      forward(center, C, T, R, O);
    }
  }
  template <typename Dtype, int N, typename A, typename B, typename C, typename D, typename E>
  void forward_host_batch(const A&, const B&, const C&, const D&, E&, std::true_type) const {}

  template <typename Dtype, bool isCUDA>
  void check_batch_example(const Grid<float, 2, isCUDA>& C, const Grid<float, 1, isCUDA>& T,
                           const Grid<float, 1, isCUDA>& R, const Grid<Dtype, 4, isCUDA>& O) const {
    check_index_args(C, T, R, O);
    if (p.radii_type_indexed) throw std::invalid_argument("Type indexed radii not supported with index types.");
  }
  template <typename Dtype, bool isCUDA>
  void check_batch_example(const Grid<float, 2, isCUDA>& C, const Grid<float, 2, isCUDA>& T,
                           const Grid<float, 1, isCUDA>& R, const Grid<Dtype, 4, isCUDA>& O) const {
    check_vector_args(C, T, R, O);
  }

  template <typename Dtype, bool isCUDA>
  void check_backward_index(const Grid<float, 2, isCUDA>& coords, const Grid<float, 1, isCUDA>& type_index,
                            const Grid<float, 1, isCUDA>& radii, const Grid<Dtype, 4, isCUDA>& diff,
                            const Grid<Dtype, 2, isCUDA>& atom_gradients) const {
    const unsigned n = coords.dimension(0);
    if (p.radii_type_indexed) throw std::invalid_argument("Type indexed radii not supported with index types.");
    if (n != type_index.size()) throw std::invalid_argument("Type dimension doesn't equal number of coordinates.");
    if (n != atom_gradients.dimension(0)) throw std::invalid_argument("Gradient dimension doesn't equal number of coordinates");
    if (n != radii.size()) throw std::invalid_argument("Radii dimension doesn't equal number of coordinates");
    if (coords.dimension(1) != 3) throw std::invalid_argument("Need x,y,z,r for coord_radius");
    for (unsigned i = 1; i <= 3; ++i)
      if (diff.dimension(i) != p.dim)
        throw std::invalid_argument("diff does not have correct dimension " + itoa(i) + ": " + itoa(diff.dimension(i)) + " vs " + itoa(p.dim));
  }
  template <typename Dtype, bool isCUDA>
  void check_backward_vector(const Grid<float, 2, isCUDA>& coords, const Grid<float, 2, isCUDA>& type_vector,
                             const Grid<float, 1, isCUDA>& radii, const Grid<Dtype, 4, isCUDA>& diff,
                             const Grid<Dtype, 2, isCUDA>& atom_gradients,
                             const Grid<Dtype, 2, isCUDA>& type_gradients) const {
    const unsigned n = coords.dimension(0), ntypes = type_vector.dimension(1);
    if (n != type_vector.dimension(0)) throw std::invalid_argument("Type dimension doesn't equal number of coordinates.");
    if (ntypes != diff.dimension(0)) throw std::invalid_argument("Channels in diff doesn't equal number of types");
    if (n != atom_gradients.dimension(0)) throw std::invalid_argument("Atom gradient dimension doesn't equal number of coordinates");
    if (n != type_gradients.dimension(0)) throw std::invalid_argument("Type gradient dimension doesn't equal number of coordinates");
    if (type_gradients.dimension(1) != ntypes) throw std::invalid_argument("Type gradient dimension has wrong number of types");
    if (coords.dimension(1) != 3) throw std::invalid_argument("Need x,y,z,r for coord_radius");
    if (p.radii_type_indexed) {
      if (ntypes != radii.size()) throw std::invalid_argument("Radii dimension doesn't equal number of types");
    } else if (n != radii.size()) {
      throw std::invalid_argument("Radii dimension doesn't equal number of coordinates");
    }
    for (unsigned i = 1; i <= 3; ++i)
      if (diff.dimension(i) != p.dim)
        throw std::invalid_argument("diff does not have correct dimension " + itoa(i) + ": " + itoa(diff.dimension(i)) + " vs " + itoa(p.dim));
  }
};

}  // namespace libmolgrid

#endif
