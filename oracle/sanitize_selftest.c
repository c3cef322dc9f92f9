/* TEST INFRASTRUCTURE.  Runs every entry point of the oracle once on small inputs that sit on the
 * edges the loops have (atoms outside the grid, on its faces and corners, zero and negative radii,
 * ignored types, no atoms, one-voxel grids, rotated resampling with taps outside the input), built
 * with AddressSanitizer and UBSan (`make asan`, host only).  It checks nothing but "the sanitizers
 * stay silent"; values are pinned by tests/test_oracle_pins.py. */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#include "gridding_oracle.h"

static float frand(unsigned* s) {
  *s = *s * 1664525u + 1013904223u;
  return (float)((*s >> 8) & 0xffff) / 65535.0f;
}

static int run(float res, float dimension, int binary, int rti, float scale, float grm, int natoms,
               int ntypes) {
  orc_gridmaker g;
  orc_gridmaker_init(&g, res, dimension, binary, rti, scale, grm);
  const int64_t dim = (int64_t)(roundf(dimension / res) + 1);
  const size_t vox = (size_t)ntypes * dim * dim * dim;
  unsigned seed = 12345u + (unsigned)natoms;
  float* coords = malloc(sizeof(float) * 3 * (natoms + 1));
  float* tindex = malloc(sizeof(float) * (natoms + 1));
  float* tvec = calloc((size_t)(natoms + 1) * ntypes, sizeof(float));
  float* radii = malloc(sizeof(float) * ((rti ? ntypes : natoms) + 1));
  float* grid = malloc(sizeof(float) * vox);
  float* diff = malloc(sizeof(float) * vox);
  float* ag = malloc(sizeof(float) * 3 * (natoms + 1));
  double* ag64 = malloc(sizeof(double) * 3 * (natoms + 1));
  float* tg = malloc(sizeof(float) * (size_t)(natoms + 1) * ntypes);
  double* tg64 = malloc(sizeof(double) * (size_t)(natoms + 1) * ntypes);
  float* rel = malloc(sizeof(float) * (natoms + 1));
  float* dd = malloc(sizeof(float) * vox);
  float* add = malloc(sizeof(float) * 3 * (natoms + 1));
  float* tdd = malloc(sizeof(float) * (size_t)(natoms + 1) * ntypes);
  const float half = dimension / 2;
  const float edge[5] = {-half - 3.f, -half, 0.f, half, half + 3.f};
  for (int a = 0; a < natoms; ++a) {
    for (int d = 0; d < 3; ++d)
      coords[3 * a + d] = a < 15 ? edge[(a / (d == 0 ? 1 : d == 1 ? 5 : 25) + a) % 5]
                                 : (frand(&seed) * 2 - 1) * (half + 2);
    tindex[a] = a % 7 == 0 ? -1.0f : (float)(a % ntypes) + 0.4f * frand(&seed);
    tvec[(size_t)a * ntypes + a % ntypes] = frand(&seed);
    if (!rti) radii[a] = a % 11 == 0 ? 0.f : a % 13 == 0 ? -1.f : 0.8f + 1.2f * frand(&seed);
  }
  if (rti)
    for (int t = 0; t < ntypes; ++t) radii[t] = 0.8f + 1.2f * frand(&seed);
  for (size_t i = 0; i < vox; ++i) diff[i] = frand(&seed) - 0.5f;
  const float c[3] = {0.1f, -0.2f, 0.05f};
  int rc = 0;
  if (!rti) {
    rc |= orc_forward_index(&g, c, natoms, coords, tindex, radii, ntypes, grid);
    rc |= orc_backward_index(&g, c, natoms, coords, tindex, radii, ntypes, diff, ag);
    rc |= orc_backward_index_f64(&g, c, natoms, coords, tindex, radii, ntypes, diff, ag64);
    rc |= orc_backward_relevance(&g, c, natoms, coords, tindex, radii, ntypes, grid, diff, rel);
  }
  rc |= orc_forward_vector(&g, c, natoms, coords, tvec, radii, ntypes, grid);
  rc |= orc_backward_vector(&g, c, natoms, coords, tvec, radii, ntypes, diff, ag, tg);
  rc |= orc_backward_vector_f64(&g, c, natoms, coords, tvec, radii, ntypes, diff, ag64, tg64);
  if (!binary)
    rc |= orc_backward_gradients(&g, c, natoms, coords, tvec, radii, ntypes, diff, ag, tg, dd, add, tdd);
  /* resampling of the grid under a rotation about an off-centre point, shifted by half the box */
  const float q[4] = {0.8f, 0.3f, -0.4f, 0.2f}, rc3[3] = {1.f, -1.f, 0.5f};
  const float tr[3] = {half, -half / 2, 1.f};
  rc |= orc_interpolate(res, dimension, res, dimension, c, grid, ntypes, q, rc3, tr, c, dd);
  float moved[3 * 16], back[3 * 16];
  orc_transform_forward(q, rc3, tr, 1, natoms < 16 ? natoms : 16, coords, moved);
  orc_transform_backward(q, rc3, tr, 0, natoms < 16 ? natoms : 16, moved, back);
  free(coords); free(tindex); free(tvec); free(radii); free(grid); free(diff); free(ag); free(ag64);
  free(tg); free(tg64); free(rel); free(dd); free(add); free(tdd);
  return rc;
}

int main(void) {
  int rc = 0;
  rc |= run(0.5f, 6.0f, 0, 0, 1.0f, 1.0f, 40, 3);
  rc |= run(0.5f, 6.0f, 1, 0, 1.0f, 1.0f, 40, 3);
  rc |= run(0.5f, 6.0f, 0, 1, 1.0f, 1.0f, 40, 3);
  rc |= run(0.5f, 6.0f, 1, 1, 1.0f, 1.0f, 40, 3);
  rc |= run(0.5f, 6.0f, 0, 0, 1.3f, 0.7f, 40, 2);
  rc |= run(0.5f, 6.0f, 0, 0, 1.0f, -1.5f, 40, 2);
  rc |= run(0.5f, 6.0f, 1, 0, 1.0f, -0.5f, 40, 2);
  rc |= run(1.0f, 0.0f, 0, 0, 1.0f, 1.0f, 5, 1);      /* a grid of one voxel */
  rc |= run(0.5f, 6.0f, 0, 0, 1.0f, 1.0f, 0, 2);      /* no atoms */
  printf("oracle sanitize selftest: status %d\n", rc);
  return rc == 0 ? 0 : 1;
}
