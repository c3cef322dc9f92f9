// Exercises the C++ host layer (include/libmolgrid/*.h) the way libmolgrid's own unit tests use
// the reference classes (test/test_gridmaker.cpp, test_transform.cpp, test_gridinterp.cpp,
// test_mgrid.cpp).  `test_api check` only runs what needs no device (argument checks, host-side
// arithmetic); `test_api gpu` runs everything.  Exit status 0 = all passed.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <functional>
#include <string>

#include "libmolgrid/grid_interpolater.h"
#include "libmolgrid/grid_maker.h"

using namespace libmolgrid;

static int failures = 0;
#define CHECK(cond)                                                             \
  do {                                                                          \
    if (!(cond)) { std::printf("FAIL %s:%d: %s\n", __FILE__, __LINE__, #cond); ++failures; } \
  } while (0)
#define CHECK_NEAR(a, b, tol) CHECK(std::fabs((a) - (b)) <= (tol))

template <typename E>
static bool throws(const std::function<void()>& f) {
  try { f(); } catch (const E&) { return true; } catch (...) { return false; }
  return false;
}

static void host_only_tests() {
  // Grid views, slices and element access
  float data[24];
  for (int i = 0; i < 24; ++i) data[i] = i;
  Grid3f g(data, 2, 3, 4);
  CHECK(g.size() == 24 && g.dimension(1) == 3 && g.offset(0) == 12);
  CHECK(g(1, 2, 3) == 23 && g[1][2][3] == 23 && g[1](0, 1) == 13);
  CHECK(throws<std::out_of_range>([&] { g[2]; }));
  CHECK(throws<std::out_of_range>([&] { g.dimension(3); }));
  // ManagedGrid on the host
  MGrid2f m(3, 4);
  CHECK(m.oncpu() && m.size() == 12 && m(2, 3) == 0);
  m(1, 2) = 7;
  MGrid1f row = m[1];
  CHECK(row(2) == 7);
  row(3) = 9;
  CHECK(m(1, 3) == 9);  // shared storage
  MGrid2f copy = m.clone();
  copy(1, 2) = 1;
  CHECK(m(1, 2) == 7);
  // quaternion and transform arithmetic
  const float s = std::sqrt(0.5f);
  Quaternion q(s, 0, 0, s);  // 90 degrees about z
  float3 p = q.rotate(1, 0, 0);
  CHECK_NEAR(p.x, 0, 1e-6); CHECK_NEAR(p.y, 1, 1e-6); CHECK_NEAR(p.z, 0, 1e-6);
  Quaternion one = q * q.inverse();
  CHECK_NEAR(one.R_component_1(), 1, 1e-6);
  CHECK(Transform().is_identity());
  set_random_seed(5);
  Transform r1(make_float3(0, 1, 1), 10.0, true);
  set_random_seed(5);
  Transform r2(make_float3(0, 1, 1), 10.0, true);
  CHECK(r1.get_quaternion() == r2.get_quaternion());
  CHECK_NEAR(r1.get_quaternion().norm(), 1.0, 1e-5);
  // GridMaker set-up and argument checks (thrown before anything touches the device)
  GridMaker gm(0.5, 23.5);
  CHECK(gm.get_first_dim() == 48);
  CHECK_NEAR(gm.get_radiusmultiple(), 1.5, 1e-6);
  GridMaker fine(0.1, 6.0);
  CHECK(fine.get_first_dim() == 61);
  float3 o = gm.get_grid_origin(make_float3(1, 2, 3));
  CHECK_NEAR(o.x, -10.75, 1e-6);
  float c4[12] = {0}, t4[4] = {0}, r4[4] = {1, 1, 1, 1};
  static float big[2 * 16 * 16 * 16];
  GridMaker g16(0.5, 7.5);
  Grid2f C(c4, 4, 3);
  Grid1f T(t4, 4), R(r4, 4), R3(r4, 3);
  Grid4f good(big, 2, 16, 16, 16), bad(big, 2, 16, 16, 15);
  CHECK(throws<std::out_of_range>([&] { g16.forward(make_float3(0, 0, 0), C, T, R, bad); }));
  CHECK(throws<std::out_of_range>([&] { g16.forward(make_float3(0, 0, 0), C, T, R3, good); }));
  t4[0] = 5;
  CHECK(throws<std::out_of_range>([&] { g16.forward(make_float3(0, 0, 0), C, T, R, good); }));
  t4[0] = 0;
  GridMaker rti(0.5, 7.5, false, true);
  CHECK(throws<std::invalid_argument>([&] { rti.forward(make_float3(0, 0, 0), C, T, R, good); }));
  float gr[12];
  Grid2f G(gr, 4, 3), G3(gr, 3, 3);
  CHECK(throws<std::invalid_argument>([&] { g16.backward(make_float3(0, 0, 0), C, T, R, good, G3); }));
  GridInterpolater gi(0.5, 7.5, 0.5, 7.5);
  CHECK(throws<std::invalid_argument>([&] { gi.forward(good, Transform(), good); }));
  Grid2f C2(c4, 3, 3);
  CHECK(throws<std::invalid_argument>([&] { Transform().forward(C, C2); }));
  // coordinate sets
  std::vector<float3> pts = {make_float3(0, 0, 0), make_float3(2, 4, 6)};
  CoordinateSet rec(pts, std::vector<int>{0, 1}, std::vector<float>{1, 1}, 2);
  CoordinateSet lig(pts, std::vector<int>{0, 0}, std::vector<float>{2, 2}, 1);
  CoordinateSet both(rec, lig);
  CHECK(both.size() == 4 && both.max_type == 3 && both.type_index(3) == 2 && both.radii(2) == 2);
  float3 ctr = rec.center();
  CHECK_NEAR(ctr.x, 1, 1e-6); CHECK_NEAR(ctr.z, 3, 1e-6);
}

static void gpu_tests() {
  // density profile of one atom: exp(-2x^2) inside r, quadratic to 1.5r
  GridMaker gm(0.1, 6.0);
  std::vector<float3> pts = {make_float3(0, 0, 0)};
  CoordinateSet one(pts, std::vector<int>{0}, std::vector<float>{1.0f}, 1);
  MGrid4f grid(1, 61, 61, 61);
  gm.forward(make_float3(0, 0, 0), one, grid.gpu());
  CHECK(grid.ongpu());
  CHECK_NEAR(grid(0, 30, 30, 30), 1.0, 1e-6);
  CHECK_NEAR(grid(0, 30, 30, 35), std::exp(-0.5), 1e-6);
  CHECK_NEAR(grid(0, 30, 30, 43), 4 * std::exp(-2.0) * 1.69 - 12 * std::exp(-2.0) * 1.3 + 9 * std::exp(-2.0), 1e-5);
  CHECK(grid(0, 30, 30, 46) == 0);
  // host overload gives the same grid (staged through the device)
  MGrid4f grid2(1, 61, 61, 61);
  gm.forward(make_float3(0, 0, 0), one, grid2.cpu());
  grid.tocpu();
  CHECK(std::memcmp(grid.cpu().data(), grid2.cpu().data(), grid.size() * sizeof(float)) == 0);

  // backward known answer: atom at x=1, r=2, unit gradient at the grid centre -> (-0.60653, 0, 0),
  // also after a random rotation undone by Transform::backward without translation
  std::vector<float3> p1 = {make_float3(1, 0, 0)};
  CoordinateSet atom(p1, std::vector<int>{0}, std::vector<float>{2.0f}, 1);
  MGrid4f diff(1, 61, 61, 61);
  diff(0, 30, 30, 30) = 1.0;
  set_random_seed(3);
  Transform T(make_float3(0, 0, 0), 0, true);
  T.forward(atom, atom);
  MGrid2f cpu_atoms(1, 3), gpu_atoms(1, 3);
  gm.backward(make_float3(0, 0, 0), atom, diff.cpu(), cpu_atoms.cpu());
  gm.backward(make_float3(0, 0, 0), atom, diff.gpu(), gpu_atoms.gpu());
  T.backward(cpu_atoms.cpu(), cpu_atoms.cpu(), false);
  T.backward(gpu_atoms.gpu(), gpu_atoms.gpu(), false);
  CHECK_NEAR(cpu_atoms(0, 0), -0.60653067, 1e-5); CHECK_NEAR(cpu_atoms(0, 1), 0, 1e-5);
  CHECK_NEAR(gpu_atoms(0, 0), -0.60653067, 1e-5); CHECK_NEAR(gpu_atoms(0, 2), 0, 1e-5);

  // transform: z-90 about (0,1,1) then (2,0,-3); forward then backward is the identity
  const float s = std::sqrt(0.5f);
  Transform nr(Quaternion(s, 0, 0, s), make_float3(0, 1, 1), make_float3(2, 0, -3));
  MGrid2f coords(3, 3), moved(3, 3);
  coords(0, 1) = 1; coords(0, 2) = 1;                       // (0,1,1): the centre
  coords(1, 1) = 1;                                          // (0,1,0)
  coords(2, 0) = 1; coords(2, 1) = 1; coords(2, 2) = 1;      // (1,1,1)
  nr.forward(coords.gpu(), moved.gpu());
  CHECK_NEAR(moved(0, 0), 2, 1e-5); CHECK_NEAR(moved(0, 1), 1, 1e-5); CHECK_NEAR(moved(0, 2), -2, 1e-5);
  CHECK_NEAR(moved(1, 0), 2, 1e-5); CHECK_NEAR(moved(1, 1), 1, 1e-5); CHECK_NEAR(moved(1, 2), -3, 1e-5);
  CHECK_NEAR(moved(2, 0), 2, 1e-5); CHECK_NEAR(moved(2, 1), 2, 1e-5); CHECK_NEAR(moved(2, 2), -2, 1e-5);
  nr.backward(moved.gpu(), moved.gpu());
  CHECK_NEAR(moved(2, 0), 1, 1e-5); CHECK_NEAR(moved(1, 2), 0, 1e-5);

  // vector types: one-hot equals index types, half weights halve the density
  GridMaker g1(0.25, 6.0);
  std::vector<float3> two = {make_float3(0, 0, 0), make_float3(2, 0, 0)};
  CoordinateSet idx(two, std::vector<int>{0, 1}, std::vector<float>{1, 1}, 2);
  CoordinateSet hot(two, std::vector<std::vector<float>>{{1, 0}, {0, 1}}, std::vector<float>{1, 1});
  CoordinateSet half(two, std::vector<std::vector<float>>{{0.5f, 0}, {0, 0.5f}}, std::vector<float>{1, 1});
  MGrid4f a(2, 25, 25, 25), b(2, 25, 25, 25), c(2, 25, 25, 25);
  g1.forward(make_float3(0, 0, 0), idx, a.gpu());
  g1.forward(make_float3(0, 0, 0), hot, b.gpu());
  g1.forward(make_float3(0, 0, 0), half, c.gpu());
  double worst = 0, worst2 = 0;
  for (size_t i = 0; i < a.size(); ++i) {
    worst = std::max<double>(worst, std::fabs(a.cpu().data()[i] - b.cpu().data()[i]));
    worst2 = std::max<double>(worst2, std::fabs(a.cpu().data()[i] - 2 * c.cpu().data()[i]));
  }
  CHECK(worst <= 1e-6 && worst2 <= 1e-6);

  // padded batch on the device: one launch, same as per-example calls
  MGrid3f bc(2, 2, 3); MGrid2f bt(2, 2), br(2, 2), cen(2, 3);
  bc(0, 1, 0) = 2; bc(1, 0, 1) = 1; bt(0, 1) = 1; bt(1, 0) = 1;
  for (int i = 0; i < 2; ++i) for (int j = 0; j < 2; ++j) br(i, j) = 1;
  MGrid5f batched(2, 2, 25, 25, 25);
  g1.forward<float, 2, true>(cen.gpu(), bc.gpu(), bt.gpu(), br.gpu(), batched.gpu());
  MGrid4f single(2, 25, 25, 25);
  g1.forward(make_float3(0, 0, 0), bc[1].gpu(), bt[1].gpu(), br[1].gpu(), single.gpu());
  batched.tocpu(); single.tocpu();
  CHECK(std::memcmp(batched[1].cpu().data(), single.cpu().data(), single.size() * sizeof(float)) == 0);

  // interpolation: identity is exact, one-voxel shift moves the data
  MGrid4f src(1, 13, 13, 13), dst(1, 13, 13, 13);
  for (size_t i = 0; i < src.size(); ++i) src.cpu().data()[i] = (float)((i * 7919) % 101) / 101.0f;
  GridInterpolater gi(0.5, 6.0, 0.5, 6.0);
  gi.forward(src.gpu(), Transform(), dst.gpu());
  src.tocpu(); dst.tocpu();
  CHECK(std::memcmp(src.cpu().data(), dst.cpu().data(), src.size() * sizeof(float)) == 0);
  Transform shift(Quaternion(), make_float3(0, 0, 0), make_float3(0.5, 0, 0));
  gi.forward(src.gpu(), shift, dst.gpu());
  CHECK_NEAR(dst(0, 5, 6, 7), src(0, 4, 6, 7), 1e-5);
  CHECK(dst(0, 0, 3, 3) == 0);

  // example -> grid through merge + transform
  Example ex;
  ex.sets.push_back(CoordinateSet(two, std::vector<int>{0, 1}, std::vector<float>{1, 1}, 2));
  ex.sets.push_back(CoordinateSet(p1, std::vector<int>{0}, std::vector<float>{1.5f}, 1));
  MGrid4f eg(3, 25, 25, 25);
  g1.forward(ex, Transform(), eg.gpu());
  CHECK(eg(2, 16, 12, 12) > 0.99f);   // ligand atom at (1,0,0) lands in channel 2
  CHECK(throws<std::out_of_range>([&] { MGrid4f wrong(2, 25, 25, 25); g1.forward(ex, Transform(), wrong.gpu()); }));

  // relevance: test/test_gridmaker.cpp:313-337
  {
    GridMaker gr(0.1, 6.0);
    CoordinateSet cs(std::vector<float3>{make_float3(0, 0, 0)}, std::vector<int>{0}, std::vector<float>{2.0f}, 1);
    const unsigned d = gr.get_grid_dims().x;
    MGrid4f rdiff(1, d, d, d), rdens(1, d, d, d);
    rdiff(0, 31, 30, 30) = 10.0f;
    rdens(0, 31, 30, 30) = 1.0f;
    MGrid1f cpurel(1), gpurel(1);
    gr.backward_relevance(make_float3(0, 0, 0), cs, rdens.cpu(), rdiff.cpu(), cpurel.cpu());
    gr.backward_relevance(make_float3(0, 0, 0), cs, rdens.gpu(), rdiff.gpu(), gpurel.gpu());
    gpurel.tocpu();
    CHECK_NEAR(cpurel(0), gpurel(0), 1e-5);
    CHECK(cpurel(0) > 1.0f && cpurel(0) < 10.0f);
  }
  // second-order pass: zero upstream gradients give zero everywhere; binary is rejected
  {
    GridMaker g2(0.5, 6.0);
    CoordinateSet cs(std::vector<float3>{make_float3(0.2f, 0, 0)}, std::vector<std::vector<float> >{{1.0f, 0.5f}},
                     std::vector<float>{1.5f});
    MGrid4f d4(2, 13, 13, 13), dd4(2, 13, 13, 13);
    for (size_t i = 0; i < d4.size(); ++i) d4.cpu().data()[i] = 1.0f;
    MGrid2f ag(1, 3), tg(1, 2), add(1, 3), tdd(1, 2);
    tg(0, 0) = 1.0f;
    g2.backward_gradients(make_float3(0, 0, 0), cs, d4.gpu(), ag.gpu(), tg.gpu(), dd4.gpu(), add.gpu(), tdd.gpu());
    dd4.tocpu(); add.tocpu(); tdd.tocpu();
    CHECK(tdd(0, 0) == 0 && tdd(0, 1) == 0);
    CHECK(dd4(0, 6, 6, 6) > 0.9f);      // d(type gradient)/d(diff) is the density itself
    CHECK(dd4(1, 6, 6, 6) == 0);
    GridMaker gb(0.5, 6.0, true);
    CHECK(throws<std::invalid_argument>([&] { gb.backward_gradients(make_float3(0, 0, 0), cs, d4.gpu(), ag.gpu(), tg.gpu(), dd4.gpu(), add.gpu(), tdd.gpu()); }));
  }

  // double precision grids (the reference's Grid<double, ...> overloads): the float result, widened
  {
    MGrid4d wide(3, 25, 25, 25), wide_host(3, 25, 25, 25);
    MGrid4f narrow(3, 25, 25, 25);
    CoordinateSet both = ex.merge_coordinates();
    g1.forward(make_float3(0, 0, 0), both, narrow.gpu());
    g1.forward(make_float3(0, 0, 0), both, wide.gpu());
    g1.forward(make_float3(0, 0, 0), both, wide_host.cpu());
    narrow.tocpu();
    wide.tocpu();
    bool same = true;
    for (size_t i = 0; i < narrow.size(); ++i)
      same = same && wide.cpu().data()[i] == (double)narrow.cpu().data()[i] &&
             wide_host.cpu().data()[i] == (double)narrow.cpu().data()[i];
    CHECK(same);
    // backward: double upstream gradient and double atom gradients
    MGrid4d dwide(3, 25, 25, 25);
    MGrid4f dnarrow(3, 25, 25, 25);
    for (size_t i = 0; i < dwide.size(); ++i) {
      const float v = std::sin(0.37f * (float)i);
      dnarrow.cpu().data()[i] = v;
      dwide.cpu().data()[i] = v;
    }
    MGrid2d gwide(both.size(), 3), gwide_host(both.size(), 3);
    MGrid2f gnarrow(both.size(), 3);
    g1.backward(make_float3(0, 0, 0), both, dnarrow.gpu(), gnarrow.gpu());
    g1.backward(make_float3(0, 0, 0), both, dwide.gpu(), gwide.gpu());
    g1.backward(make_float3(0, 0, 0), both, dwide.cpu(), gwide_host.cpu());
    gnarrow.tocpu();
    gwide.tocpu();
    same = true;
    for (size_t i = 0; i < gnarrow.size(); ++i)
      same = same && gwide.cpu().data()[i] == (double)gnarrow.cpu().data()[i] &&
             gwide_host.cpu().data()[i] == (double)gnarrow.cpu().data()[i];
    CHECK(same);
    CHECK(gnarrow.cpu().data()[0] != 0.0f);
    // Transform on double coordinates
    MGrid2d cw(2, 3);
    MGrid2f cn(2, 3);
    for (int i = 0; i < 6; ++i) { cw.cpu().data()[i] = 0.5 * i - 1; cn.cpu().data()[i] = 0.5f * i - 1; }
    Transform tq(Quaternion(std::sqrt(0.5f), 0, 0, std::sqrt(0.5f)), make_float3(0, 1, 0), make_float3(1, 2, 3));
    tq.forward(cn.gpu(), cn.gpu());
    tq.forward(cw.gpu(), cw.gpu());
    cn.tocpu();
    cw.tocpu();
    for (int i = 0; i < 6; ++i) CHECK(cw.cpu().data()[i] == (double)cn.cpu().data()[i]);
  }

  // batch of examples: one packed upload, two launches; equals the per-example calls bit for bit
  Example ex2;
  ex2.sets.push_back(CoordinateSet(p1, std::vector<int>{1}, std::vector<float>{2.0f}, 2));
  ex2.sets.push_back(CoordinateSet(two, std::vector<int>{0, 0}, std::vector<float>{1, 1.5f}, 1));
  Example none;
  none.sets.push_back(CoordinateSet(std::vector<float3>{}, std::vector<int>{}, std::vector<float>{}, 2));
  none.sets.push_back(CoordinateSet(std::vector<float3>{}, std::vector<int>{}, std::vector<float>{}, 1));
  std::vector<Example> batch{ex, ex2, none};
  MGrid5f bg(3, 3, 25, 25, 25), bh(3, 3, 25, 25, 25);
  g1.forward(batch, bg.gpu());
  g1.forward(batch, bh.cpu());
  bg.tocpu();
  CHECK(std::memcmp(bg.cpu().data(), bh.cpu().data(), bg.size() * sizeof(float)) == 0);
  for (int b = 0; b < 3; ++b) {
    MGrid4f one(3, 25, 25, 25);
    g1.forward(batch[b], one.gpu());
    one.tocpu();
    CHECK(std::memcmp(one.cpu().data(), bg.cpu().data() + (size_t)b * one.size(), one.size() * sizeof(float)) == 0);
  }
  CHECK(throws<std::out_of_range>([&] { MGrid5f wrong(2, 3, 25, 25, 25); g1.forward(batch, wrong.gpu()); }));
}

int main(int argc, char** argv) {
  const std::string mode = argc > 1 ? argv[1] : "check";
  host_only_tests();
  if (mode == "gpu") gpu_tests();
  std::printf("%s: %d failure(s)\n", mode.c_str(), failures);
  return failures ? 1 : 0;
}
