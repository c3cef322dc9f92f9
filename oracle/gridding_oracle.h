/*
 * CPU oracle for the gridding hot path -- TEST INFRASTRUCTURE ONLY.
 *
 * This is a plain-C restatement of the arithmetic of the reference's CPU
 * overloads (GridMaker::forward / backward on Grid<...,false>, Transform,
 * Quaternion, GridInterpolater::forward).  It exists so that the HIP kernels
 * can be checked against it and so that a CPU timing can be printed beside the
 * GPU numbers.  Nothing that ships may call it: only tests, the smoke check
 * and the benchmark's cpu_baseline leg load this library.
 *
 * Float/double mixing, operation order and loop order follow the reference
 * files cited at each function (paths relative to the reference checkout).
 * Build with -ffp-contract=off and without -ffast-math so that no product is
 * fused into an add.
 *
 * Pinning status (what anchors each function to the reference's behaviour):
 *   orc_gridmaker_init     closed-form constants quoted by the reference's
 *                          tests (test/test_gridmaker.py:131-184)
 *   orc_forward_index      closed-form density profile, brute force over every
 *                          voxel on small inputs, one-hot == index equivalence
 *   orc_forward_vector     linearity in the type vector, type-indexed radii ==
 *                          per-atom radii (test/test_gridmaker.cpp:408-500)
 *   orc_backward_index     known answer (-0.60653067,0,0)
 *                          (test/test_gridmaker.py:186-214), finite difference
 *                          of the forward pass, antisymmetry
 *   orc_backward_vector    type gradient == sum(density*diff) by brute force
 *   orc_quat_*, orc_transform_*  z-90-degree known points
 *                          (test/test_transform.cpp:55-103), forward o backward
 *                          == identity, agreement with a rotation matrix
 *   orc_interpolate        scipy RegularGridInterpolator on a zero padded
 *                          input (test/test_gridinterp.py:112-152), identity
 *                          and pure-translation cases
 * Bit-level rounding of the mixed float/double expressions in
 * orc_calc_point / orc_accumulate_atom_gradient and the inclusive/exclusive
 * edges of orc_bounds_1d cannot be compared against a compiled reference in
 * this environment (the reference needs CUDA, Boost and OpenBabel headers that
 * are absent): at that level they are "parity unpinned".
 */
#ifndef GRIDDING_ORACLE_H_
#define GRIDDING_ORACLE_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct orc_gridmaker {
  float resolution;
  float dimension;
  float radius_scale;
  float gaussian_radius_multiple;
  float final_radius_multiple;
  float A, B, C, D, E;
  int binary;
  int radii_type_indexed;
  unsigned dim;
} orc_gridmaker;

enum {
  ORC_OK = 0,
  ORC_ERR_TYPE_RANGE = 1,   /* reference throws std::out_of_range / invalid_argument */
  ORC_ERR_ARGUMENT = 2
};

void orc_gridmaker_init(orc_gridmaker* g, float res, float dimension, int binary,
                        int radii_type_indexed, float radius_scale, float grm);

float orc_calc_point(const orc_gridmaker* g, float ax, float ay, float az, float ar,
                     float gx, float gy, float gz);

void orc_bounds_1d(const orc_gridmaker* g, float grid_origin, float coord, float densityrad,
                   unsigned* lo, unsigned* hi);

int orc_forward_index(const orc_gridmaker* g, const float center[3], int64_t natoms,
                      const float* coords, const float* type_index, const float* radii,
                      int64_t ntypes, float* out);

int orc_forward_vector(const orc_gridmaker* g, const float center[3], int64_t natoms,
                       const float* coords, const float* type_vector, const float* radii,
                       int64_t ntypes, float* out);

int orc_backward_index(const orc_gridmaker* g, const float center[3], int64_t natoms,
                       const float* coords, const float* type_index, const float* radii,
                       int64_t ntypes, const float* diff, float* atom_gradients);

/* Same sweep as orc_backward_index but every sum is carried in double: what the
 * mathematics fixes, free of the sequential float accumulation noise. */
int orc_backward_index_f64(const orc_gridmaker* g, const float center[3], int64_t natoms,
                           const float* coords, const float* type_index, const float* radii,
                           int64_t ntypes, const float* diff, double* atom_gradients);

int orc_backward_vector(const orc_gridmaker* g, const float center[3], int64_t natoms,
                        const float* coords, const float* type_vector, const float* radii,
                        int64_t ntypes, const float* diff, float* atom_gradients,
                        float* type_gradients);

int orc_backward_vector_f64(const orc_gridmaker* g, const float center[3], int64_t natoms,
                            const float* coords, const float* type_vector, const float* radii,
                            int64_t ntypes, const float* diff, double* atom_gradients,
                            double* type_gradients);

/* relevance of each atom (src/grid_maker.cpp:392-432, 680-704); density is the forward grid */
int orc_backward_relevance(const orc_gridmaker* g, const float center[3], int64_t natoms,
                           const float* coords, const float* type_index, const float* radii,
                           int64_t ntypes, const float* density, const float* diff,
                           float* relevance);

/* gradients of the vector-typed backward pass (src/grid_maker.cpp:529-661); the three outputs
 * are overwritten */
int orc_backward_gradients(const orc_gridmaker* g, const float center[3], int64_t natoms,
                           const float* coords, const float* type_vector, const float* radii,
                           int64_t ntypes, const float* diff, const float* atom_gradients,
                           const float* type_gradients, float* diffdiff, float* atom_diffdiff,
                           float* type_diffdiff);

/* quaternion stored as (a, b, c, d) = real, i, j, k */
void orc_quat_mul(const float p[4], const float q[4], float out[4]);
void orc_quat_inverse(const float q[4], float out[4]);
void orc_quat_rotate(const float q[4], float x, float y, float z, float out[3]);

void orc_transform_forward(const float q[4], const float center[3], const float translate[3],
                           int dotranslate, int64_t n, const float* in, float* out);
void orc_transform_backward(const float q[4], const float center[3], const float translate[3],
                            int dotranslate, int64_t n, const float* in, float* out);

int orc_interpolate(float in_resolution, float in_dimension, float out_resolution,
                    float out_dimension, const float in_center[3], const float* in,
                    int64_t channels, const float q[4], const float rot_center[3],
                    const float translate[3], const float out_center[3], float* out);

/* Batched drivers: examples are independent, so these loop over the batch
 * (optionally with OpenMP threads; nthreads <= 1 means the plain serial loop the
 * reference runs).  atom_offsets has nbatch+1 entries into the packed atom
 * arrays.  Return the first non-zero status of any example. */
int orc_forward_index_batch(const orc_gridmaker* g, int nbatch, const int64_t* atom_offsets,
                            const float* centers, const float* coords, const float* type_index,
                            const float* radii, int64_t ntypes, float* out, int nthreads);
int orc_forward_vector_batch(const orc_gridmaker* g, int nbatch, const int64_t* atom_offsets,
                             const float* centers, const float* coords, const float* type_vector,
                             const float* radii, int64_t ntypes, float* out, int nthreads);
int orc_backward_index_batch(const orc_gridmaker* g, int nbatch, const int64_t* atom_offsets,
                             const float* centers, const float* coords, const float* type_index,
                             const float* radii, int64_t ntypes, const float* diff,
                             float* atom_gradients, int nthreads);
int orc_backward_vector_batch(const orc_gridmaker* g, int nbatch, const int64_t* atom_offsets,
                              const float* centers, const float* coords, const float* type_vector,
                              const float* radii, int64_t ntypes, const float* diff,
                              float* atom_gradients, float* type_gradients, int nthreads);
void orc_transform_forward_batch(int nbatch, const int64_t* atom_offsets, const float* quats,
                                 const float* centers, const float* translations, int dotranslate,
                                 const float* in, float* out, int nthreads);
void orc_transform_backward_batch(int nbatch, const int64_t* atom_offsets, const float* quats,
                                  const float* centers, const float* translations, int dotranslate,
                                  const float* in, float* out, int nthreads);
int orc_interpolate_batch(float in_resolution, float in_dimension, float out_resolution,
                          float out_dimension, int nbatch, int64_t channels,
                          const float* in_centers, const float* in, const float* quats,
                          const float* rot_centers, const float* translations,
                          const float* out_centers, float* out, int nthreads);

int orc_max_threads(void);

#ifdef __cplusplus
}
#endif
#endif
