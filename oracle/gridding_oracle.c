/*
 * CPU oracle for the gridding hot path -- TEST INFRASTRUCTURE ONLY (see the
 * header for what may load it and for the pinning status of each function).
 *
 * Reference paths are relative to the reference checkout.  Where the reference
 * mixes float and double the same widths are used here, and every expression
 * keeps the reference's association order; compile with -ffp-contract=off.
 */
#include "gridding_oracle.h"

#include <math.h>
#include <stddef.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ---- GridMaker set-up ---------------------------------------------------- */

/* src/grid_maker.cpp:15-36 (GridMaker::initialize) and the constructor in
 * include/libmolgrid/grid_maker.h:70-74.  The coefficient formulas use the
 * sign-preserving argument `grm`, while the stored multiple is made positive. */
void orc_gridmaker_init(orc_gridmaker* g, float res, float dimension, int binary,
                        int radii_type_indexed, float radius_scale, float grm) {
  g->resolution = res;
  g->dimension = dimension;
  g->radius_scale = radius_scale;
  g->gaussian_radius_multiple = grm;
  if (grm < 0) {
    g->gaussian_radius_multiple = grm * -1;
    g->final_radius_multiple = g->gaussian_radius_multiple;
  } else {
    g->final_radius_multiple = (1 + 2 * grm * grm) / (2 * grm);
  }
  g->dim = (unsigned)(roundf(dimension / res) + 1);
  g->binary = binary;
  g->radii_type_indexed = radii_type_indexed;

  /* unqualified exp() on a float argument in a host .cpp resolves to the double
   * routine; each product is then carried in double and narrowed on store */
  g->A = (float)(exp(-2 * grm * grm) * 4 * grm * grm);
  g->B = (float)(-exp(-2 * grm * grm) * (4 * grm + 8 * grm * grm * grm));
  g->C = (float)(exp(-2 * grm * grm) * (4 * grm * grm * grm * grm + 4 * grm * grm + 1));
  g->D = (float)(8 * grm * grm * exp(-2.0 * grm * grm));
  g->E = (float)(-(4 * grm + 8 * grm * grm * grm) * exp(-2 * grm * grm));
}

/* src/grid_maker.cpp:100-107 (get_grid_origin): dimension/2.0 is a double
 * quotient narrowed to float before the subtraction. */
static void grid_origin(const orc_gridmaker* g, const float center[3], float origin[3]) {
  float half = (float)(g->dimension / 2.0);
  origin[0] = center[0] - half;
  origin[1] = center[1] - half;
  origin[2] = center[2] - half;
}

/* src/grid_maker.cu:66-79 (get_bounds_1d) */
void orc_bounds_1d(const orc_gridmaker* g, float origin, float coord, float densityrad,
                   unsigned* lo, unsigned* hi) {
  *lo = 0;
  *hi = 0;
  float low = coord - densityrad - origin;
  if (low > 0) *lo = (unsigned)floorf(low / g->resolution);
  float high = coord + densityrad - origin;
  if (high > 0) {
    unsigned top = (unsigned)ceilf(high / g->resolution);
    *hi = top < g->dim ? top : g->dim;
  }
}

/* src/grid_maker.cu:82-92 (sqDistance): ((dx*dx + dy*dy) + dz*dz) with the
 * difference taken as grid point minus atom. */
static inline float sq_distance(float gx, float gy, float gz, float ax, float ay, float az) {
  float t = gx - ax;
  float acc = t * t;
  t = gy - ay;
  acc += t * t;
  t = gz - az;
  acc += t * t;
  return acc;
}

/* src/grid_maker.cu:95-130 (calc_point<false> and calc_point<true>) */
float orc_calc_point(const orc_gridmaker* g, float ax, float ay, float az, float ar,
                     float gx, float gy, float gz) {
  float rsq = sq_distance(gx, gy, gz, ax, ay, az);
  ar *= g->radius_scale;
  if (g->binary) return rsq < ar * ar ? 1.0f : 0.0f;

  float dist = sqrtf(rsq);
  if (dist > ar * g->final_radius_multiple) return 0.0f;
  if (dist <= ar * g->gaussian_radius_multiple) {
    float ex = (float)(-2.0 * dist * dist / (ar * ar));
    return expf(ex);
  }
  float dr = dist / ar;
  float q = (g->A * dr + g->B) * dr + g->C;
  return q > 0 ? q : 0;
}

/* ---- forward ------------------------------------------------------------- */

static size_t grid_points(const orc_gridmaker* g, int64_t ntypes) {
  return (size_t)ntypes * g->dim * g->dim * g->dim;
}

/* src/grid_maker.cpp:153-212 (forward, index types, CPU) */
int orc_forward_index(const orc_gridmaker* g, const float center[3], int64_t natoms,
                      const float* coords, const float* type_index, const float* radii,
                      int64_t ntypes, float* out) {
  memset(out, 0, grid_points(g, ntypes) * sizeof(float));
  if (g->radii_type_indexed) return ORC_ERR_ARGUMENT;
  float origin[3];
  grid_origin(g, center, origin);
  const size_t dim = g->dim;
  const float res = g->resolution;

  for (int64_t a = 0; a < natoms; ++a) {
    int64_t atype = (int64_t)floor(type_index[a]);
    if (atype >= ntypes) return ORC_ERR_TYPE_RANGE;
    if (atype < 0) continue;
    float ax = coords[3 * a], ay = coords[3 * a + 1], az = coords[3 * a + 2];
    float radius = radii[a];
    float densityrad = radius * g->radius_scale * g->final_radius_multiple;
    unsigned lo[3], hi[3];
    orc_bounds_1d(g, origin[0], ax, densityrad, &lo[0], &hi[0]);
    orc_bounds_1d(g, origin[1], ay, densityrad, &lo[1], &hi[1]);
    orc_bounds_1d(g, origin[2], az, densityrad, &lo[2], &hi[2]);
    for (size_t i = lo[0]; i < hi[0]; ++i) {
      for (size_t j = lo[1]; j < hi[1]; ++j) {
        for (size_t k = lo[2]; k < hi[2]; ++k) {
          float gx = origin[0] + i * res;
          float gy = origin[1] + j * res;
          float gz = origin[2] + k * res;
          float val = orc_calc_point(g, ax, ay, az, radius, gx, gy, gz);
          float* cell = out + ((((size_t)atype * dim) + i) * dim + j) * dim + k;
          if (g->binary) {
            if (val != 0) *cell = 1.0f;
          } else {
            *cell += val;
          }
        }
      }
    }
  }
  return ORC_OK;
}

/* src/grid_maker.cpp:214-271 (forward, vector types, CPU) */
int orc_forward_vector(const orc_gridmaker* g, const float center[3], int64_t natoms,
                       const float* coords, const float* type_vector, const float* radii,
                       int64_t ntypes, float* out) {
  memset(out, 0, grid_points(g, ntypes) * sizeof(float));
  float origin[3];
  grid_origin(g, center, origin);
  const size_t dim = g->dim;
  const float res = g->resolution;

  for (int64_t a = 0; a < natoms; ++a) {
    for (int64_t t = 0; t < ntypes; ++t) {
      float tmult = type_vector[a * ntypes + t];
      if (tmult == 0) continue;
      float ax = coords[3 * a], ay = coords[3 * a + 1], az = coords[3 * a + 2];
      float radius = g->radii_type_indexed ? radii[t] : radii[a];
      float densityrad = radius * g->radius_scale * g->final_radius_multiple;
      unsigned lo[3], hi[3];
      orc_bounds_1d(g, origin[0], ax, densityrad, &lo[0], &hi[0]);
      orc_bounds_1d(g, origin[1], ay, densityrad, &lo[1], &hi[1]);
      orc_bounds_1d(g, origin[2], az, densityrad, &lo[2], &hi[2]);
      for (size_t i = lo[0]; i < hi[0]; ++i) {
        for (size_t j = lo[1]; j < hi[1]; ++j) {
          for (size_t k = lo[2]; k < hi[2]; ++k) {
            float gx = origin[0] + i * res;
            float gy = origin[1] + j * res;
            float gz = origin[2] + k * res;
            float val = orc_calc_point(g, ax, ay, az, radius, gx, gy, gz);
            float* cell = out + ((((size_t)t * dim) + i) * dim + j) * dim + k;
            if (g->binary) {
              if (val != 0) *cell += tmult;
            } else {
              *cell += val * tmult;
            }
          }
        }
      }
    }
  }
  return ORC_OK;
}

/* ---- backward ------------------------------------------------------------ */

/* src/grid_maker.cu:881-896 (density_grad_dist); ar already carries radius_scale */
static float density_grad_dist(const orc_gridmaker* g, float dist, float ar) {
  float dist2 = dist * dist;
  if (dist > ar * g->final_radius_multiple) return NAN;
  if (dist <= ar * g->gaussian_radius_multiple) {
    float ex = (float)(-2.0 * dist2 / (ar * ar));
    float coef = (float)(-4.0 * dist / (ar * ar));
    return coef * expf(ex);
  }
  return (g->D * dist / ar + g->E) / ar;
}

/* src/grid_maker.cu:898-919 (accumulate_atom_gradient): the distance is a float
 * square root widened to double, the direction ratio and the product are
 * double, and every update is rounded back into the float accumulator. */
static void accumulate_atom_gradient(const orc_gridmaker* g, float ax, float ay, float az,
                                     float x, float y, float z, float ar, float gridval,
                                     float agrad[3]) {
  float dx = x - ax, dy = y - ay, dz = z - az;
  float dist2 = dx * dx + dy * dy + dz * dz;
  double dist = sqrtf(dist2);
  ar *= g->radius_scale;
  float agrad_dist = density_grad_dist(g, (float)dist, ar);
  if (dist > 0 && isfinite(agrad_dist)) {
    agrad[0] += -(dx / dist) * (agrad_dist * gridval);
    agrad[1] += -(dy / dist) * (agrad_dist * gridval);
    agrad[2] += -(dz / dist) * (agrad_dist * gridval);
  }
}

/* double-accumulating twin of the above, used only by the *_f64 drivers */
static void accumulate_atom_gradient_f64(const orc_gridmaker* g, float ax, float ay, float az,
                                         float x, float y, float z, float ar, float gridval,
                                         double agrad[3]) {
  float dx = x - ax, dy = y - ay, dz = z - az;
  float dist2 = dx * dx + dy * dy + dz * dz;
  double dist = sqrtf(dist2);
  ar *= g->radius_scale;
  float agrad_dist = density_grad_dist(g, (float)dist, ar);
  if (dist > 0 && isfinite(agrad_dist)) {
    agrad[0] += -(dx / dist) * ((double)agrad_dist * gridval);
    agrad[1] += -(dy / dist) * ((double)agrad_dist * gridval);
    agrad[2] += -(dz / dist) * ((double)agrad_dist * gridval);
  }
}

/* src/grid_maker.cpp:325-354 (calc_atom_gradient_cpu): i, j, k sweep of the
 * atom's index box inside one channel of the upstream gradient. */
static void atom_gradient(const orc_gridmaker* g, const float origin[3], const float* xyz,
                          const float* diff_channel, float radius, float agrad[3]) {
  agrad[0] = agrad[1] = agrad[2] = 0;
  float r = radius * g->radius_scale * g->final_radius_multiple;
  unsigned lo[3], hi[3];
  for (int d = 0; d < 3; ++d) orc_bounds_1d(g, origin[d], xyz[d], r, &lo[d], &hi[d]);
  const size_t dim = g->dim;
  for (unsigned i = lo[0]; i < hi[0]; ++i)
    for (unsigned j = lo[1]; j < hi[1]; ++j)
      for (unsigned k = lo[2]; k < hi[2]; ++k) {
        float x = origin[0] + i * g->resolution;
        float y = origin[1] + j * g->resolution;
        float z = origin[2] + k * g->resolution;
        accumulate_atom_gradient(g, xyz[0], xyz[1], xyz[2], x, y, z, radius,
                                 diff_channel[((size_t)i * dim + j) * dim + k], agrad);
      }
}

static void atom_gradient_f64(const orc_gridmaker* g, const float origin[3], const float* xyz,
                              const float* diff_channel, float radius, double agrad[3]) {
  agrad[0] = agrad[1] = agrad[2] = 0;
  float r = radius * g->radius_scale * g->final_radius_multiple;
  unsigned lo[3], hi[3];
  for (int d = 0; d < 3; ++d) orc_bounds_1d(g, origin[d], xyz[d], r, &lo[d], &hi[d]);
  const size_t dim = g->dim;
  for (unsigned i = lo[0]; i < hi[0]; ++i)
    for (unsigned j = lo[1]; j < hi[1]; ++j)
      for (unsigned k = lo[2]; k < hi[2]; ++k) {
        float x = origin[0] + i * g->resolution;
        float y = origin[1] + j * g->resolution;
        float z = origin[2] + k * g->resolution;
        accumulate_atom_gradient_f64(g, xyz[0], xyz[1], xyz[2], x, y, z, radius,
                                     diff_channel[((size_t)i * dim + j) * dim + k], agrad);
      }
}

/* src/grid_maker.cpp:357-389 (calc_type_gradient_cpu) */
static float type_gradient(const orc_gridmaker* g, const float origin[3], const float* xyz,
                           const float* diff_channel, float radius) {
  float r = radius * g->radius_scale * g->final_radius_multiple;
  unsigned lo[3], hi[3];
  for (int d = 0; d < 3; ++d) orc_bounds_1d(g, origin[d], xyz[d], r, &lo[d], &hi[d]);
  const size_t dim = g->dim;
  float ret = 0;
  for (unsigned i = lo[0]; i < hi[0]; ++i)
    for (unsigned j = lo[1]; j < hi[1]; ++j)
      for (unsigned k = lo[2]; k < hi[2]; ++k) {
        float x = origin[0] + i * g->resolution;
        float y = origin[1] + j * g->resolution;
        float z = origin[2] + k * g->resolution;
        float val = orc_calc_point(g, xyz[0], xyz[1], xyz[2], radius, x, y, z);
        ret += val * diff_channel[((size_t)i * dim + j) * dim + k];
      }
  return ret;
}

static double type_gradient_f64(const orc_gridmaker* g, const float origin[3], const float* xyz,
                                const float* diff_channel, float radius) {
  float r = radius * g->radius_scale * g->final_radius_multiple;
  unsigned lo[3], hi[3];
  for (int d = 0; d < 3; ++d) orc_bounds_1d(g, origin[d], xyz[d], r, &lo[d], &hi[d]);
  const size_t dim = g->dim;
  double ret = 0;
  for (unsigned i = lo[0]; i < hi[0]; ++i)
    for (unsigned j = lo[1]; j < hi[1]; ++j)
      for (unsigned k = lo[2]; k < hi[2]; ++k) {
        float x = origin[0] + i * g->resolution;
        float y = origin[1] + j * g->resolution;
        float z = origin[2] + k * g->resolution;
        float val = orc_calc_point(g, xyz[0], xyz[1], xyz[2], radius, x, y, z);
        ret += (double)val * diff_channel[((size_t)i * dim + j) * dim + k];
      }
  return ret;
}

/* src/grid_maker.cpp:436-467 (backward, index types, CPU).  The channel is
 * round(type), not floor as in forward. */
int orc_backward_index(const orc_gridmaker* g, const float center[3], int64_t natoms,
                       const float* coords, const float* type_index, const float* radii,
                       int64_t ntypes, const float* diff, float* atom_gradients) {
  memset(atom_gradients, 0, (size_t)natoms * 3 * sizeof(float));
  if (g->radii_type_indexed) return ORC_ERR_ARGUMENT;
  float origin[3];
  grid_origin(g, center, origin);
  const size_t chan = (size_t)g->dim * g->dim * g->dim;
  for (int64_t a = 0; a < natoms; ++a) {
    int which = (int)round(type_index[a]);
    if (which < 0) continue;
    if (which >= ntypes) return ORC_ERR_TYPE_RANGE;
    atom_gradient(g, origin, coords + 3 * a, diff + which * chan, radii[a],
                  atom_gradients + 3 * a);
  }
  return ORC_OK;
}

int orc_backward_index_f64(const orc_gridmaker* g, const float center[3], int64_t natoms,
                           const float* coords, const float* type_index, const float* radii,
                           int64_t ntypes, const float* diff, double* atom_gradients) {
  memset(atom_gradients, 0, (size_t)natoms * 3 * sizeof(double));
  if (g->radii_type_indexed) return ORC_ERR_ARGUMENT;
  float origin[3];
  grid_origin(g, center, origin);
  const size_t chan = (size_t)g->dim * g->dim * g->dim;
  for (int64_t a = 0; a < natoms; ++a) {
    int which = (int)round(type_index[a]);
    if (which < 0) continue;
    if (which >= ntypes) return ORC_ERR_TYPE_RANGE;
    atom_gradient_f64(g, origin, coords + 3 * a, diff + which * chan, radii[a],
                      atom_gradients + 3 * a);
  }
  return ORC_OK;
}

/* src/grid_maker.cpp:477-519 (backward, vector types, CPU): the atom gradient
 * only takes channels with a non-zero weight, the type gradient takes all. */
int orc_backward_vector(const orc_gridmaker* g, const float center[3], int64_t natoms,
                        const float* coords, const float* type_vector, const float* radii,
                        int64_t ntypes, const float* diff, float* atom_gradients,
                        float* type_gradients) {
  memset(atom_gradients, 0, (size_t)natoms * 3 * sizeof(float));
  memset(type_gradients, 0, (size_t)natoms * ntypes * sizeof(float));
  float origin[3];
  grid_origin(g, center, origin);
  const size_t chan = (size_t)g->dim * g->dim * g->dim;
  for (int64_t a = 0; a < natoms; ++a) {
    float radius = 0;
    if (!g->radii_type_indexed) radius = radii[a];
    for (int64_t t = 0; t < ntypes; ++t) {
      float tmult = type_vector[a * ntypes + t];
      if (g->radii_type_indexed) radius = radii[t];
      if (tmult != 0) {
        float ag[3];
        atom_gradient(g, origin, coords + 3 * a, diff + t * chan, radius, ag);
        atom_gradients[3 * a + 0] += ag[0] * tmult;
        atom_gradients[3 * a + 1] += ag[1] * tmult;
        atom_gradients[3 * a + 2] += ag[2] * tmult;
      }
      type_gradients[a * ntypes + t] =
          type_gradient(g, origin, coords + 3 * a, diff + t * chan, radius);
    }
  }
  return ORC_OK;
}

int orc_backward_vector_f64(const orc_gridmaker* g, const float center[3], int64_t natoms,
                            const float* coords, const float* type_vector, const float* radii,
                            int64_t ntypes, const float* diff, double* atom_gradients,
                            double* type_gradients) {
  memset(atom_gradients, 0, (size_t)natoms * 3 * sizeof(double));
  memset(type_gradients, 0, (size_t)natoms * ntypes * sizeof(double));
  float origin[3];
  grid_origin(g, center, origin);
  const size_t chan = (size_t)g->dim * g->dim * g->dim;
  for (int64_t a = 0; a < natoms; ++a) {
    float radius = 0;
    if (!g->radii_type_indexed) radius = radii[a];
    for (int64_t t = 0; t < ntypes; ++t) {
      float tmult = type_vector[a * ntypes + t];
      if (g->radii_type_indexed) radius = radii[t];
      if (tmult != 0) {
        double ag[3];
        atom_gradient_f64(g, origin, coords + 3 * a, diff + t * chan, radius, ag);
        atom_gradients[3 * a + 0] += ag[0] * tmult;
        atom_gradients[3 * a + 1] += ag[1] * tmult;
        atom_gradients[3 * a + 2] += ag[2] * tmult;
      }
      type_gradients[a * ntypes + t] =
          type_gradient_f64(g, origin, coords + 3 * a, diff + t * chan, radius);
    }
  }
  return ORC_OK;
}

/* ---- relevance and second-order gradients -------------------------------- */

/* src/grid_maker.cpp:392-432 (calc_atom_relevance_cpu) and :680-704 (backward_relevance):
 * every voxel the atom reaches hands the atom the share val/density of its relevance. */
int orc_backward_relevance(const orc_gridmaker* g, const float center[3], int64_t natoms,
                           const float* coords, const float* type_index, const float* radii,
                           int64_t ntypes, const float* density, const float* diff,
                           float* relevance) {
  memset(relevance, 0, (size_t)natoms * sizeof(float));
  float origin[3];
  grid_origin(g, center, origin);
  const size_t chan = (size_t)g->dim * g->dim * g->dim;
  const int64_t dim = g->dim;
  for (int64_t a = 0; a < natoms; ++a) {
    int which = (int)roundf(type_index[a]);
    if (which < 0) continue;
    if (which >= ntypes) return ORC_ERR_TYPE_RANGE;
    const float* dens = density + (size_t)which * chan;
    const float* dif = diff + (size_t)which * chan;
    float ax = coords[3 * a], ay = coords[3 * a + 1], az = coords[3 * a + 2];
    float radius = radii[a];
    float r = radius * g->radius_scale * g->final_radius_multiple;
    unsigned lo[3], hi[3];
    orc_bounds_1d(g, origin[0], ax, r, &lo[0], &hi[0]);
    orc_bounds_1d(g, origin[1], ay, r, &lo[1], &hi[1]);
    orc_bounds_1d(g, origin[2], az, r, &lo[2], &hi[2]);
    float ret = 0;
    for (size_t i = lo[0]; i < hi[0]; ++i)
      for (size_t j = lo[1]; j < hi[1]; ++j)
        for (size_t k = lo[2]; k < hi[2]; ++k) {
          float x = origin[0] + i * g->resolution;
          float y = origin[1] + j * g->resolution;
          float z = origin[2] + k * g->resolution;
          float val = orc_calc_point(g, ax, ay, az, radius, x, y, z);
          if (val > 0) {
            float denseval = dens[(i * dim + j) * dim + k];
            float gridval = dif[(i * dim + j) * dim + k];
            if (denseval > 0) ret += gridval * val / denseval;
          }
        }
    relevance[a] = ret;
  }
  return ORC_OK;
}

/* src/grid_maker.cu:812-855: type_grad_grad and atom_density_grad_grad hold the same
 * expression -- the derivative of -(a-x)/dist * density_grad_dist with respect to a. */
static float density_grad_grad(const orc_gridmaker* g, float a, float x, float dist, float r) {
  float dist2 = dist * dist;
  if (dist > r * g->final_radius_multiple) return 0;
  if (dist <= r * g->gaussian_radius_multiple) {
    float r2 = r * r;
    float ex = (float)(-2.0 * dist2 / r2);
    return 16 * (a - x) * (a - x) * expf(ex) / (r2 * r2) - 4 * expf(ex) / (r2);
  }
  float ax = a - x;
  float ax2 = ax * ax;
  float term1 = (float)(-(g->E + g->D * dist / r) * ax2 / (pow(dist2, 1.5) * r));
  float term2 = g->D * ax2 / (dist2 * r * r);
  float term3 = (g->E + g->D * dist / r) / (dist * r);
  return term1 + term2 + term3;
}

/* src/grid_maker.cu:858-877 (atom_density_grad_grad_other): mixed second derivative */
static float density_grad_grad_other(const orc_gridmaker* g, float a, float x, float b, float y,
                                     float dist, float r) {
  float dist2 = dist * dist;
  if (dist > r * g->final_radius_multiple) return 0;
  if (dist <= r * g->gaussian_radius_multiple) {
    float r2 = r * r;
    float ex = (float)(-2.0 * dist2 / r2);
    return 16 * (a - x) * (b - y) * expf(ex) / (r2 * r2);
  }
  float ax = a - x;
  float by = b - y;
  float term1 = (float)(-(g->E + g->D * dist / r) * ax * by / (pow(dist2, 1.5) * r));
  float term2 = g->D * ax * by / (dist2 * r * r);
  return term1 + term2;
}

/* src/grid_maker.cpp:529-661 (backward_gradients, CPU): gradients of the backward pass
 * (atom_gradients, type_gradients as functions of coords, types and diff) with respect to
 * diff (diffdiff), the coordinates (atom_diffdiff) and the types (type_diffdiff, zero). */
int orc_backward_gradients(const orc_gridmaker* g, const float center[3], int64_t natoms,
                           const float* coords, const float* type_vector, const float* radii,
                           int64_t ntypes, const float* diff, const float* atom_gradients,
                           const float* type_gradients, float* diffdiff, float* atom_diffdiff,
                           float* type_diffdiff) {
  if (g->binary) return ORC_ERR_ARGUMENT;
  const size_t chan = (size_t)g->dim * g->dim * g->dim;
  const int64_t dim = g->dim;
  memset(atom_diffdiff, 0, (size_t)natoms * 3 * sizeof(float));
  memset(type_diffdiff, 0, (size_t)natoms * ntypes * sizeof(float));
  memset(diffdiff, 0, chan * ntypes * sizeof(float));
  float origin[3];
  grid_origin(g, center, origin);
  for (int64_t a = 0; a < natoms; ++a) {
    for (int64_t t = 0; t < ntypes; ++t) {
      float tmult = type_vector[a * ntypes + t];
      if (tmult == 0) continue;
      const float* diffG = diff + (size_t)t * chan;
      float ax = coords[3 * a], ay = coords[3 * a + 1], az = coords[3 * a + 2];
      float gx = atom_gradients[3 * a], gy = atom_gradients[3 * a + 1], gz = atom_gradients[3 * a + 2];
      float tgrad = type_gradients[a * ntypes + t];
      float radius = g->radii_type_indexed ? radii[t] : radii[a];
      float ar = radius * g->radius_scale;
      float densityrad = radius * g->radius_scale * g->final_radius_multiple;
      unsigned lo[3], hi[3];
      orc_bounds_1d(g, origin[0], ax, densityrad, &lo[0], &hi[0]);
      orc_bounds_1d(g, origin[1], ay, densityrad, &lo[1], &hi[1]);
      orc_bounds_1d(g, origin[2], az, densityrad, &lo[2], &hi[2]);
      float dd[3] = {0, 0, 0};
      for (size_t i = lo[0]; i < hi[0]; ++i)
        for (size_t j = lo[1]; j < hi[1]; ++j)
          for (size_t k = lo[2]; k < hi[2]; ++k) {
            float x = origin[0] + i * g->resolution;
            float y = origin[1] + j * g->resolution;
            float z = origin[2] + k * g->resolution;
            size_t off = (size_t)(i * dim + j) * dim + k;
            float G = diffG[off];
            float dist_x = x - ax, dist_y = y - ay, dist_z = z - az;
            float dist2 = dist_x * dist_x + dist_y * dist_y + dist_z * dist_z;
            double dist = sqrtf(dist2);
            float agrad_dist = density_grad_dist(g, (float)dist, ar);
            if (!isfinite(agrad_dist)) continue;
            float gval = 0.0f;
            if (dist > 0) {
              gval += (float)(-(dist_x / dist) * (agrad_dist * gx));
              gval += (float)(-(dist_y / dist) * (agrad_dist * gy));
              gval += (float)(-(dist_z / dist) * (agrad_dist * gz));
              gval *= tmult;
            }
            float val = orc_calc_point(g, ax, ay, az, radius, x, y, z);
            gval += val * tgrad;
            diffdiff[(size_t)t * chan + off] += gval;

            float d = (float)dist;
            dd[0] += density_grad_grad(g, ax, x, d, ar) * G * tmult * gx;
            dd[0] += density_grad_grad_other(g, ax, x, ay, y, d, ar) * G * tmult * gy;
            dd[0] += density_grad_grad_other(g, ax, x, az, z, d, ar) * G * tmult * gz;
            dd[0] += density_grad_grad(g, ax, x, d, ar) * G * tgrad;

            dd[1] += density_grad_grad_other(g, ay, y, ax, x, d, ar) * G * tmult * gx;
            dd[1] += density_grad_grad(g, ay, y, d, ar) * G * tmult * gy;
            dd[1] += density_grad_grad_other(g, ay, y, az, z, d, ar) * G * tmult * gz;
            dd[1] += density_grad_grad(g, ay, y, d, ar) * G * tgrad;

            dd[2] += density_grad_grad_other(g, az, z, ax, x, d, ar) * G * tmult * gx;
            dd[2] += density_grad_grad_other(g, az, z, ay, y, d, ar) * G * tmult * gy;
            dd[2] += density_grad_grad(g, az, z, d, ar) * G * tmult * gz;
            dd[2] += density_grad_grad(g, az, z, d, ar) * G * tgrad;
          }
      atom_diffdiff[3 * a + 0] += dd[0];
      atom_diffdiff[3 * a + 1] += dd[1];
      atom_diffdiff[3 * a + 2] += dd[2];
    }
  }
  return ORC_OK;
}

/* ---- quaternion / transform --------------------------------------------- */

/* include/libmolgrid/quaternion.h:82-91 (Hamilton product, left-to-right sums) */
void orc_quat_mul(const float p[4], const float q[4], float out[4]) {
  float a = p[0], b = p[1], c = p[2], d = p[3];
  float ar = q[0], br = q[1], cr = q[2], dr = q[3];
  float o0 = +a * ar - b * br - c * cr - d * dr;
  float o1 = +a * br + b * ar + c * dr - d * cr;
  float o2 = +a * cr - b * dr + c * ar + d * br;
  float o3 = +a * dr + b * cr - c * br + d * ar;
  out[0] = o0; out[1] = o1; out[2] = o2; out[3] = o3;
}

/* include/libmolgrid/quaternion.h:161-165 (inverse) */
void orc_quat_inverse(const float q[4], float out[4]) {
  float nsq = q[0] * q[0] + q[1] * q[1] + q[2] * q[2] + q[3] * q[3];
  out[0] = q[0] / nsq;
  out[1] = -q[1] / nsq;
  out[2] = -q[2] / nsq;
  out[3] = -q[3] / nsq;
}

/* include/libmolgrid/quaternion.h:145-149 (rotate): q * (0,x,y,z) * (conj(q)/norm(q));
 * the quaternion is not assumed to be of unit length. */
void orc_quat_rotate(const float q[4], float x, float y, float z, float out[3]) {
  float p[4] = {0, x, y, z};
  float n = q[0] * q[0] + q[1] * q[1] + q[2] * q[2] + q[3] * q[3];
  float cj[4] = {q[0] / n, -q[1] / n, -q[2] / n, -q[3] / n};
  float qp[4], r[4];
  orc_quat_mul(q, p, qp);
  orc_quat_mul(qp, cj, r);
  out[0] = r[1];
  out[1] = r[2];
  out[2] = r[3];
}

/* src/transform.cpp:57-79 with quaternion.h:152-158 (Quaternion::transform):
 * rotate about center, add center back, then add the translation (zero when
 * dotranslate is false -- the rotation still happens about center). */
void orc_transform_forward(const float q[4], const float center[3], const float translate[3],
                           int dotranslate, int64_t n, const float* in, float* out) {
  float t[3] = {0, 0, 0};
  if (dotranslate) { t[0] = translate[0]; t[1] = translate[1]; t[2] = translate[2]; }
  for (int64_t i = 0; i < n; ++i) {
    float x = in[3 * i], y = in[3 * i + 1], z = in[3 * i + 2];
    float r[3];
    orc_quat_rotate(q, x - center[0], y - center[1], z - center[2], r);
    out[3 * i + 0] = r[0] + center[0] + t[0];
    out[3 * i + 1] = r[1] + center[1] + t[1];
    out[3 * i + 2] = r[2] + center[2] + t[2];
  }
}

/* src/transform.cpp:85-108 (Transform::backward, CPU) */
void orc_transform_backward(const float q[4], const float center[3], const float translate[3],
                            int dotranslate, int64_t n, const float* in, float* out) {
  float inv[4];
  orc_quat_inverse(q, inv);
  float un[3];
  for (int d = 0; d < 3; ++d)
    un[d] = dotranslate ? -translate[d] - center[d] : -center[d];
  for (int64_t i = 0; i < n; ++i) {
    float x = in[3 * i] + un[0], y = in[3 * i + 1] + un[1], z = in[3 * i + 2] + un[2];
    float r[3];
    orc_quat_rotate(inv, x, y, z, r);
    out[3 * i + 0] = r[0] + center[0];
    out[3 * i + 1] = r[1] + center[1];
    out[3 * i + 2] = r[2] + center[2];
  }
}

/* ---- interpolation ------------------------------------------------------- */

/* src/grid_interpolater.cu:17-23 (get_pt): zero outside the input grid */
static inline float tap(const float* chan, int dim, int x, int y, int z) {
  if (x < 0 || x >= dim || y < 0 || y >= dim || z < 0 || z >= dim) return 0;
  return chan[((size_t)x * dim + y) * dim + z];
}

/* src/grid_interpolater.cu:26-58 (interpolate): floor/ceil taps, weights zero
 * when the coordinate is integral, lerp along x, then y, then z. */
static float trilinear(const float* chan, int dim, float gx, float gy, float gz) {
  int xl = (int)floorf(gx), xh = (int)ceilf(gx);
  int yl = (int)floorf(gy), yh = (int)ceilf(gy);
  int zl = (int)floorf(gz), zh = (int)ceilf(gz);
  float p000 = tap(chan, dim, xl, yl, zl), p001 = tap(chan, dim, xl, yl, zh);
  float p010 = tap(chan, dim, xl, yh, zl), p011 = tap(chan, dim, xl, yh, zh);
  float p100 = tap(chan, dim, xh, yl, zl), p101 = tap(chan, dim, xh, yl, zh);
  float p110 = tap(chan, dim, xh, yh, zl), p111 = tap(chan, dim, xh, yh, zh);
  float xd = xh > xl ? (gx - xl) / (xh - xl) : 0;
  float yd = yh > yl ? (gy - yl) / (yh - yl) : 0;
  float zd = zh > zl ? (gz - zl) / (zh - zl) : 0;
  float c00 = p000 * (1 - xd) + p100 * xd;
  float c01 = p001 * (1 - xd) + p101 * xd;
  float c10 = p010 * (1 - xd) + p110 * xd;
  float c11 = p011 * (1 - xd) + p111 * xd;
  float c0 = c00 * (1 - yd) + c10 * yd;
  float c1 = c01 * (1 - yd) + c11 * yd;
  return c0 * (1 - zd) + c1 * zd;
}

/* src/grid_interpolater.cpp:16-48 (GridInterpolater::forward, CPU) with the
 * index<->Cartesian helpers of include/libmolgrid/grid_interpolater.h:189-198
 * and the point counts of its constructor (:59-64). */
int orc_interpolate(float in_resolution, float in_dimension, float out_resolution,
                    float out_dimension, const float in_center[3], const float* in,
                    int64_t channels, const float q[4], const float rot_center[3],
                    const float translate[3], const float out_center[3], float* out) {
  if (in == out) return ORC_ERR_ARGUMENT;
  const unsigned in_dim = (unsigned)(roundf(in_dimension / in_resolution) + 1);
  const unsigned out_dim = (unsigned)(roundf(out_dimension / out_resolution) + 1);
  float in_radius = (float)(in_dimension / 2.0);
  float out_radius = (float)(out_dimension / 2.0);
  float in_origin[3], out_origin[3], un[3], inv[4];
  for (int d = 0; d < 3; ++d) {
    in_origin[d] = in_center[d] - in_radius;
    out_origin[d] = out_center[d] - out_radius;
    un[d] = -translate[d] - rot_center[d];
  }
  orc_quat_inverse(q, inv);
  const size_t in_chan = (size_t)in_dim * in_dim * in_dim;
  const size_t out_chan = (size_t)out_dim * out_dim * out_dim;
  for (unsigned i = 0; i < out_dim; ++i)
    for (unsigned j = 0; j < out_dim; ++j)
      for (unsigned k = 0; k < out_dim; ++k) {
        float ox = out_origin[0] + i * out_resolution;
        float oy = out_origin[1] + j * out_resolution;
        float oz = out_origin[2] + k * out_resolution;
        float r[3];
        orc_quat_rotate(inv, ox + un[0], oy + un[1], oz + un[2], r);
        float gx = (r[0] + rot_center[0] - in_origin[0]) / in_resolution;
        float gy = (r[1] + rot_center[1] - in_origin[1]) / in_resolution;
        float gz = (r[2] + rot_center[2] - in_origin[2]) / in_resolution;
        size_t o = ((size_t)i * out_dim + j) * out_dim + k;
        for (int64_t c = 0; c < channels; ++c)
          out[c * out_chan + o] = trilinear(in + c * in_chan, (int)in_dim, gx, gy, gz);
      }
  return ORC_OK;
}

/* ---- batched drivers ------------------------------------------------------ */
/* The reference loops over the batch on the host (include/libmolgrid/grid_maker.h:
 * 194-201, 265-301).  Examples are independent, so the loop may be split over
 * threads without changing any value. */

int orc_max_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

#ifdef _OPENMP
#define ORC_PARALLEL_FOR _Pragma("omp parallel for schedule(dynamic, 1) num_threads(nt)")
#else
#define ORC_PARALLEL_FOR
#endif

static int clamp_threads(int nthreads) {
  int nt = nthreads < 1 ? 1 : nthreads;
  int mx = orc_max_threads();
  return nt > mx ? mx : nt;
}

int orc_forward_index_batch(const orc_gridmaker* g, int nbatch, const int64_t* off,
                            const float* centers, const float* coords, const float* type_index,
                            const float* radii, int64_t ntypes, float* out, int nthreads) {
  int nt = clamp_threads(nthreads), status = 0;
  (void)nt;
  const size_t gp = grid_points(g, ntypes);
  ORC_PARALLEL_FOR
  for (int b = 0; b < nbatch; ++b) {
    int s = orc_forward_index(g, centers + 3 * b, off[b + 1] - off[b], coords + 3 * off[b],
                              type_index + off[b], radii + off[b], ntypes, out + gp * b);
    if (s) {
#ifdef _OPENMP
#pragma omp critical
#endif
      if (!status) status = s;
    }
  }
  return status;
}

int orc_forward_vector_batch(const orc_gridmaker* g, int nbatch, const int64_t* off,
                             const float* centers, const float* coords, const float* type_vector,
                             const float* radii, int64_t ntypes, float* out, int nthreads) {
  int nt = clamp_threads(nthreads), status = 0;
  (void)nt;
  const size_t gp = grid_points(g, ntypes);
  ORC_PARALLEL_FOR
  for (int b = 0; b < nbatch; ++b) {
    const float* rad = g->radii_type_indexed ? radii + (size_t)b * ntypes : radii + off[b];
    int s = orc_forward_vector(g, centers + 3 * b, off[b + 1] - off[b], coords + 3 * off[b],
                               type_vector + off[b] * ntypes, rad, ntypes, out + gp * b);
    if (s) {
#ifdef _OPENMP
#pragma omp critical
#endif
      if (!status) status = s;
    }
  }
  return status;
}

int orc_backward_index_batch(const orc_gridmaker* g, int nbatch, const int64_t* off,
                             const float* centers, const float* coords, const float* type_index,
                             const float* radii, int64_t ntypes, const float* diff,
                             float* atom_gradients, int nthreads) {
  int nt = clamp_threads(nthreads), status = 0;
  (void)nt;
  const size_t gp = grid_points(g, ntypes);
  ORC_PARALLEL_FOR
  for (int b = 0; b < nbatch; ++b) {
    int s = orc_backward_index(g, centers + 3 * b, off[b + 1] - off[b], coords + 3 * off[b],
                               type_index + off[b], radii + off[b], ntypes, diff + gp * b,
                               atom_gradients + 3 * off[b]);
    if (s) {
#ifdef _OPENMP
#pragma omp critical
#endif
      if (!status) status = s;
    }
  }
  return status;
}

int orc_backward_vector_batch(const orc_gridmaker* g, int nbatch, const int64_t* off,
                              const float* centers, const float* coords, const float* type_vector,
                              const float* radii, int64_t ntypes, const float* diff,
                              float* atom_gradients, float* type_gradients, int nthreads) {
  int nt = clamp_threads(nthreads), status = 0;
  (void)nt;
  const size_t gp = grid_points(g, ntypes);
  ORC_PARALLEL_FOR
  for (int b = 0; b < nbatch; ++b) {
    const float* rad = g->radii_type_indexed ? radii + (size_t)b * ntypes : radii + off[b];
    int s = orc_backward_vector(g, centers + 3 * b, off[b + 1] - off[b], coords + 3 * off[b],
                                type_vector + off[b] * ntypes, rad, ntypes, diff + gp * b,
                                atom_gradients + 3 * off[b], type_gradients + off[b] * ntypes);
    if (s) {
#ifdef _OPENMP
#pragma omp critical
#endif
      if (!status) status = s;
    }
  }
  return status;
}

void orc_transform_forward_batch(int nbatch, const int64_t* off, const float* quats,
                                 const float* centers, const float* translations, int dotranslate,
                                 const float* in, float* out, int nthreads) {
  int nt = clamp_threads(nthreads);
  (void)nt;
  ORC_PARALLEL_FOR
  for (int b = 0; b < nbatch; ++b)
    orc_transform_forward(quats + 4 * b, centers + 3 * b, translations + 3 * b, dotranslate,
                          off[b + 1] - off[b], in + 3 * off[b], out + 3 * off[b]);
}

void orc_transform_backward_batch(int nbatch, const int64_t* off, const float* quats,
                                  const float* centers, const float* translations, int dotranslate,
                                  const float* in, float* out, int nthreads) {
  int nt = clamp_threads(nthreads);
  (void)nt;
  ORC_PARALLEL_FOR
  for (int b = 0; b < nbatch; ++b)
    orc_transform_backward(quats + 4 * b, centers + 3 * b, translations + 3 * b, dotranslate,
                           off[b + 1] - off[b], in + 3 * off[b], out + 3 * off[b]);
}

int orc_interpolate_batch(float in_resolution, float in_dimension, float out_resolution,
                          float out_dimension, int nbatch, int64_t channels,
                          const float* in_centers, const float* in, const float* quats,
                          const float* rot_centers, const float* translations,
                          const float* out_centers, float* out, int nthreads) {
  int nt = clamp_threads(nthreads), status = 0;
  (void)nt;
  const size_t in_dim = (size_t)(roundf(in_dimension / in_resolution) + 1);
  const size_t out_dim = (size_t)(roundf(out_dimension / out_resolution) + 1);
  const size_t in_sz = (size_t)channels * in_dim * in_dim * in_dim;
  const size_t out_sz = (size_t)channels * out_dim * out_dim * out_dim;
  ORC_PARALLEL_FOR
  for (int b = 0; b < nbatch; ++b) {
    int s = orc_interpolate(in_resolution, in_dimension, out_resolution, out_dimension,
                            in_centers + 3 * b, in + in_sz * b, channels, quats + 4 * b,
                            rot_centers + 3 * b, translations + 3 * b, out_centers + 3 * b,
                            out + out_sz * b);
    if (s) {
#ifdef _OPENMP
#pragma omp critical
#endif
      if (!status) status = s;
    }
  }
  return status;
}
