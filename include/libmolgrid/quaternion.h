// Single-precision quaternion a + bi + cj + dk used for rigid rotations.  Same members and the
// same float arithmetic, in the same association order, as libmolgrid's Quaternion
// (include/libmolgrid/quaternion.h:17-167): the quaternion is never assumed to be normalised.
#ifndef LIBMOLGRID_QUATERNION_H_
#define LIBMOLGRID_QUATERNION_H_

#include "libmolgrid/common.h"

namespace libmolgrid {

class Quaternion {
 public:
  typedef float fl;

 protected:
  fl a = 1, b = 0, c = 0, d = 0;

 public:
  Quaternion() = default;
  Quaternion(fl A, fl B, fl C, fl D) : a(A), b(B), c(C), d(D) {}

  fl R_component_1() const { return a; }
  fl R_component_2() const { return b; }
  fl R_component_3() const { return c; }
  fl R_component_4() const { return d; }
  float real() const { return a; }

  Quaternion& operator*=(const fl& r) { a *= r; b *= r; c *= r; d *= r; return *this; }
  Quaternion& operator/=(const fl& r) { a /= r; b /= r; c /= r; d /= r; return *this; }
  Quaternion operator/(const fl& r) const { return Quaternion(a / r, b / r, c / r, d / r); }

  /// Hamilton product
  Quaternion operator*(const Quaternion& r) const {
    return Quaternion(+a * r.a - b * r.b - c * r.c - d * r.d,
                      +a * r.b + b * r.a + c * r.d - d * r.c,
                      +a * r.c - b * r.d + c * r.a + d * r.b,
                      +a * r.d + b * r.c - c * r.b + d * r.a);
  }
  Quaternion& operator*=(const Quaternion& r) { *this = *this * r; return *this; }

  /// this * r^-1
  Quaternion operator/(const Quaternion& r) const {
    const fl den = r.a * r.a + r.b * r.b + r.c * r.c + r.d * r.d;
    return Quaternion((+a * r.a + b * r.b + c * r.c + d * r.d) / den,
                      (-a * r.b + b * r.a - c * r.d + d * r.c) / den,
                      (-a * r.c + b * r.d + c * r.a - d * r.b) / den,
                      (-a * r.d - b * r.c + c * r.b + d * r.a) / den);
  }
  Quaternion& operator/=(const Quaternion& r) { *this = *this / r; return *this; }

  /// bit-level equality
  bool operator==(const Quaternion& r) const { return a == r.a && b == r.b && c == r.c && d == r.d; }

  Quaternion conj() const { return Quaternion(+a, -b, -c, -d); }
  /// Cayley norm: the square of the Euclidean length
  float norm() const { return a * a + b * b + c * c + d * d; }
  Quaternion inverse() const {
    const fl nsq = a * a + b * b + c * c + d * d;
    return Quaternion(a / nsq, -b / nsq, -c / nsq, -d / nsq);
  }

  /// rotate the point (x, y, z): q (0,x,y,z) conj(q)/norm(q)
  float3 rotate(fl x, fl y, fl z) const {
    Quaternion p(0, x, y, z);
    p = *this * p * (conj() / norm());
    return make_float3(p.b, p.c, p.d);
  }
  /// rotate about center, then translate
  float3 transform(fl x, fl y, fl z, float3 center, float3 translate) const {
    const float3 pt = rotate(x - center.x, y - center.y, z - center.z);
    return make_float3(pt.x + center.x + translate.x, pt.y + center.y + translate.y,
                       pt.z + center.z + translate.z);
  }
};

}  // namespace libmolgrid

#endif
