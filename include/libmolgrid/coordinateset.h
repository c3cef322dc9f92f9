// CoordinateSet: the atoms of one molecule as managed arrays -- coords (N x 3), index types (N,
// integers stored as floats) and/or type vectors (N x T), radii (N, or T with type-indexed radii).
// Mirrors the array-based part of libmolgrid's CoordinateSet
// (include/libmolgrid/coordinateset.h:32-165, src/coordinateset.cpp:75-183, 214-229, 263-310);
// construction from molecule files needs a chemistry toolkit and is not part of the gridding path.
#ifndef LIBMOLGRID_COORDINATESET_H_
#define LIBMOLGRID_COORDINATESET_H_

#include <vector>

#include "libmolgrid/managed_grid.h"

namespace libmolgrid {

struct CoordinateSet {
  MGrid2f coords{0, 3};
  MGrid1f type_index{0};
  MGrid2f type_vector{0, 0};
  MGrid1f radii{0};
  unsigned max_type = 0;      ///< number of index types (exclusive maximum)
  const char* src = nullptr;  ///< where the coordinates came from, if known

  CoordinateSet() {}

  /// index types from vectors
  CoordinateSet(const std::vector<float3>& c, const std::vector<float>& t, const std::vector<float>& r,
                unsigned maxt)
      : coords(c.size(), 3), type_index(c.size()), radii(c.size()), max_type(maxt) {
    if (t.size() != c.size()) throw std::invalid_argument("Types and coordinates are of different sizes");
    if (r.size() != c.size()) throw std::invalid_argument("Radii and coordinates are of different sizes");
    for (size_t i = 0; i < c.size(); ++i) {
      coords(i, 0) = c[i].x; coords(i, 1) = c[i].y; coords(i, 2) = c[i].z;
      type_index(i) = t[i];
      radii(i) = r[i];
    }
  }
  CoordinateSet(const std::vector<float3>& c, const std::vector<int>& t, const std::vector<float>& r,
                unsigned maxt)
      : CoordinateSet(c, std::vector<float>(t.begin(), t.end()), r, maxt) {}

  /// vector types from vectors
  CoordinateSet(const std::vector<float3>& c, const std::vector<std::vector<float>>& t,
                const std::vector<float>& r)
      : coords(c.size(), 3), type_vector(c.size(), t.empty() ? 0 : t[0].size()), radii(r.size()) {
    if (t.size() != c.size()) throw std::invalid_argument("Types and coordinates are of different sizes");
    max_type = t.empty() ? 0 : t[0].size();
    for (size_t i = 0; i < c.size(); ++i) {
      coords(i, 0) = c[i].x; coords(i, 1) = c[i].y; coords(i, 2) = c[i].z;
      if (t[i].size() != max_type) throw std::invalid_argument("Type vectors are of different sizes");
      for (size_t k = 0; k < max_type; ++k) type_vector(i, k) = t[i][k];
    }
    for (size_t i = 0; i < r.size(); ++i) radii(i) = r[i];
  }

  /// index types from grids on either side; the data is copied
  template <bool isCUDA>
  CoordinateSet(const Grid<float, 2, isCUDA>& c, const Grid<float, 1, isCUDA>& t,
                const Grid<float, 1, isCUDA>& r, unsigned maxt)
      : coords(c.dimension(0), c.dimension(1)), type_index(t.size()), radii(r.size()), max_type(maxt) {
    if (c.dimension(1) != 3) throw std::invalid_argument("Coordinates need three columns");
    if (t.size() != c.dimension(0)) throw std::invalid_argument("Types and coordinates are of different sizes");
    if (r.size() != c.dimension(0)) throw std::invalid_argument("Radii and coordinates are of different sizes");
    coords.copyFrom(c); type_index.copyFrom(t); radii.copyFrom(r);
  }
  /// vector types from grids on either side; the data is copied
  template <bool isCUDA>
  CoordinateSet(const Grid<float, 2, isCUDA>& c, const Grid<float, 2, isCUDA>& t,
                const Grid<float, 1, isCUDA>& r)
      : coords(c.dimension(0), c.dimension(1)), type_vector(t.dimension(0), t.dimension(1)),
        radii(r.size()), max_type(t.dimension(1)) {
    if (c.dimension(1) != 3) throw std::invalid_argument("Coordinates need three columns");
    if (t.dimension(0) != c.dimension(0)) throw std::invalid_argument("Types and coordinates are of different sizes");
    coords.copyFrom(c); type_vector.copyFrom(t); radii.copyFrom(r);
  }

  /// receptor followed by ligand; with unique_index_types the ligand's type indices are shifted
  /// past the receptor's, and type vectors are laid side by side
  CoordinateSet(const CoordinateSet& rec, const CoordinateSet& lig, bool unique_index_types = true)
      : coords(rec.size() + lig.size(), 3) {
    const unsigned nr = rec.size(), nl = lig.size(), n = nr + nl;
    const bool indexed = rec.has_indexed_types() && lig.has_indexed_types();
    const bool vectored = rec.type_vector.size() > 0 || lig.type_vector.size() > 0;
    max_type = unique_index_types ? rec.max_type + lig.max_type : std::max(rec.max_type, lig.max_type);
    for (unsigned i = 0; i < n; ++i) {
      const CoordinateSet& s = i < nr ? rec : lig;
      const unsigned k = i < nr ? i : i - nr;
      for (unsigned d = 0; d < 3; ++d) coords(i, d) = s.coords(k, d);
    }
    if (indexed && !vectored) {
      type_index = MGrid1f(n);
      radii = MGrid1f(n);
      for (unsigned i = 0; i < n; ++i) {
        const bool r = i < nr;
        const unsigned k = r ? i : i - nr;
        float t = r ? rec.type_index(k) : lig.type_index(k);
        if (!r && unique_index_types && t >= 0) t += rec.max_type;
        type_index(i) = t;
        radii(i) = r ? rec.radii(k) : lig.radii(k);
      }
    } else if (vectored) {
      type_vector = MGrid2f(n, max_type);
      radii = MGrid1f(n);
      for (unsigned i = 0; i < n; ++i) {
        const bool r = i < nr;
        const unsigned k = r ? i : i - nr;
        const CoordinateSet& s = r ? rec : lig;
        const unsigned shift = (!r && unique_index_types) ? rec.max_type : 0;
        for (unsigned t = 0; t < s.max_type && s.type_vector.size() > 0; ++t)
          type_vector(i, shift + t) = s.type_vector(k, t);
        if (s.radii.size() == s.size()) radii(i) = s.radii(k);
      }
    }
  }

  bool has_indexed_types() const { return type_index.size() > 0 || coords.size() == 0; }
  bool has_vector_types() const { return type_vector.size() > 0 || coords.size() == 0; }
  unsigned num_types() const { return max_type; }
  void set_num_types(unsigned maxt) { max_type = maxt; }
  unsigned size() const { return coords.dimension(0); }

  /// mean of the coordinates
  float3 center() const {
    const unsigned n = size();
    if (n == 0) return make_float3(0, 0, 0);
    double s[3] = {0, 0, 0};
    for (unsigned i = 0; i < n; ++i)
      for (unsigned d = 0; d < 3; ++d) s[d] += coords(i, d);
    return make_float3(s[0] / n, s[1] / n, s[2] / n);
  }

  void togpu(bool copy = true) { coords.togpu(copy); type_index.togpu(copy); type_vector.togpu(copy); radii.togpu(copy); }
  void tocpu(bool copy = true) { coords.tocpu(copy); type_index.tocpu(copy); type_vector.tocpu(copy); radii.tocpu(copy); }

  /// deep copy
  CoordinateSet clone() const {
    CoordinateSet out(*this);
    out.coords = coords.clone();
    out.type_index = type_index.clone();
    out.type_vector = type_vector.clone();
    out.radii = radii.clone();
    return out;
  }

  template <bool isCUDA>
  size_t copyTo(Grid<float, 2, isCUDA>& c, Grid<float, 1, isCUDA>& t, Grid<float, 1, isCUDA>& r) const {
    const size_t n = coords.copyTo(c) / 3;
    type_index.copyTo(t);
    radii.copyTo(r);
    return n;
  }
  template <bool isCUDA>
  size_t copyTo(Grid<float, 2, isCUDA>& c, Grid<float, 2, isCUDA>& t, Grid<float, 1, isCUDA>& r) const {
    const size_t n = coords.copyTo(c) / 3;
    type_vector.copyTo(t);
    radii.copyTo(r);
    return n;
  }

  bool operator==(const CoordinateSet& rhs) const {
    return max_type == rhs.max_type && coords == rhs.coords && type_index == rhs.type_index &&
           type_vector == rhs.type_vector && radii == rhs.radii;
  }
};

/// A training example: several coordinate sets (receptor, ligand, ...) plus labels.  Only what
/// the gridding path touches (include/libmolgrid/example.h:60-169, src/example.cpp:198-228).
struct Example {
  std::vector<CoordinateSet> sets;
  std::vector<float> labels;
  int group = -1;
  bool seqcont = false;

  /// all sets as one; index types of later sets are shifted past those of earlier sets
  CoordinateSet merge_coordinates(unsigned start = 0, bool unique_index_types = true) const {
    if (sets.size() <= start) return CoordinateSet();
    CoordinateSet merged = sets[start].clone();
    for (size_t i = start + 1; i < sets.size(); ++i)
      merged = CoordinateSet(merged, sets[i], unique_index_types);
    return merged;
  }
  size_t num_coordinates() const {
    size_t n = 0;
    for (const auto& s : sets) n += s.size();
    return n;
  }
  size_t num_types(bool unique_index_types = true) const {
    size_t n = 0;
    for (const auto& s : sets) n = unique_index_types ? n + s.num_types() : std::max<size_t>(n, s.num_types());
    return n;
  }
};

}  // namespace libmolgrid

#endif
