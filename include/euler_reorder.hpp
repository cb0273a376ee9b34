// Host-side layout reorders with the signatures of Euler's include/euler_reorder.hpp:
//   reorder<T, dst_format, src_format>(dst, src, dims...)   for T = float, uint8_t.
// Channel tails of the blocked formats are zero-filled on the way in and dropped on the way out.
#pragma once

#include <cassert>
#include <cstdlib>

#include "euler.hpp"

namespace euler {

template <typename Type, const int dst_fmt, const int src_fmt, typename... Args> struct EULER_API reorder {
  reorder(Type *, Type *, Args...)
  {
    assert(!!"reorder not implemented\n");
    abort();
  }
};

#define EULER_DECLARE_REORDER4(DST, SRC, A, B)                                                      \
  template <typename Type> struct EULER_API reorder<Type, DST, SRC> {                               \
    reorder(Type *dst, Type *src, int A, int B, int h, int w);                                      \
  };
#define EULER_DECLARE_REORDER5(DST, SRC)                                                            \
  template <typename Type> struct EULER_API reorder<Type, DST, SRC> {                               \
    reorder(Type *dst, Type *src, int g, int o, int i, int h, int w);                               \
  };

EULER_DECLARE_REORDER4(nchw, nhwc, n, c)
EULER_DECLARE_REORDER4(nhwc, nchw, n, c)
EULER_DECLARE_REORDER4(nchw, nChw16c, n, c)
EULER_DECLARE_REORDER4(nChw16c, nchw, n, c)
EULER_DECLARE_REORDER4(oihw, OIhw16i16o, o, i)
EULER_DECLARE_REORDER4(OIhw16i16o, oihw, o, i)
EULER_DECLARE_REORDER4(oihw, hwio, o, i)
EULER_DECLARE_REORDER4(hwio, oihw, o, i)
EULER_DECLARE_REORDER5(goihw, gOIhw16i16o)
EULER_DECLARE_REORDER5(gOIhw16i16o, goihw)
EULER_DECLARE_REORDER5(goihw, ghwio)
EULER_DECLARE_REORDER5(ghwio, goihw)

#undef EULER_DECLARE_REORDER4
#undef EULER_DECLARE_REORDER5

}  // namespace euler
