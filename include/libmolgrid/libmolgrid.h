// Process-wide state of the host layer: the random engine behind Transform's random constructor
// (reference: include/libmolgrid/libmolgrid.h, src/libmolgrid.cpp:11).
#ifndef LIBMOLGRID_LIBMOLGRID_H_
#define LIBMOLGRID_LIBMOLGRID_H_

#include <random>

namespace libmolgrid {

/// the single engine every random transform draws from
inline std::default_random_engine& random_engine_ref() {
  static std::default_random_engine engine;
  return engine;
}
#define random_engine (::libmolgrid::random_engine_ref())

/// reseed the engine (same sequence of transforms for the same seed)
inline void set_random_seed(int seed) { random_engine_ref().seed(seed); }

}  // namespace libmolgrid

#endif
