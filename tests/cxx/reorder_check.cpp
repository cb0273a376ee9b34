// Every reorder<T, dst, src> the library instantiates (include/euler_reorder.hpp), behind one C entry
// point, so that a Python test can run each of them on host arrays and compare with numpy.
//
//   which: 0 nchw<-nhwc   1 nhwc<-nchw   2 nchw<-nChw16c   3 nChw16c<-nchw
//          4 OIhw16i16o<-oihw   5 oihw<-OIhw16i16o   6 gOIhw16i16o<-goihw   7 goihw<-gOIhw16i16o
//          8 oihw<-hwio   9 hwio<-oihw   10 goihw<-ghwio   11 ghwio<-goihw
//   a, b: (n, c) for the activation formats, (o, i) for the weight formats; g only for the grouped ones
#include <cstdint>

#include "euler.hpp"
#include "euler_reorder.hpp"

using namespace euler;

namespace {
template <typename T> int run(int which, T *dst, T *src, int g, int a, int b, int h, int w)
{
  switch (which) {
  case 0: reorder<T, nchw, nhwc>(dst, src, a, b, h, w); break;
  case 1: reorder<T, nhwc, nchw>(dst, src, a, b, h, w); break;
  case 2: reorder<T, nchw, nChw16c>(dst, src, a, b, h, w); break;
  case 3: reorder<T, nChw16c, nchw>(dst, src, a, b, h, w); break;
  case 4: reorder<T, OIhw16i16o, oihw>(dst, src, a, b, h, w); break;
  case 5: reorder<T, oihw, OIhw16i16o>(dst, src, a, b, h, w); break;
  case 6: reorder<T, gOIhw16i16o, goihw>(dst, src, g, a, b, h, w); break;
  case 7: reorder<T, goihw, gOIhw16i16o>(dst, src, g, a, b, h, w); break;
  case 8: reorder<T, oihw, hwio>(dst, src, a, b, h, w); break;
  case 9: reorder<T, hwio, oihw>(dst, src, a, b, h, w); break;
  case 10: reorder<T, goihw, ghwio>(dst, src, g, a, b, h, w); break;
  case 11: reorder<T, ghwio, goihw>(dst, src, g, a, b, h, w); break;
  default: return -1;
  }
  return 0;
}
}  // namespace

extern "C" __attribute__((visibility("default"))) int reorder_check(int which, int is_u8, void *dst, void *src, int g,
                                                                    int a, int b, int h, int w)
{
  return is_u8 ? run<uint8_t>(which, (uint8_t *)dst, (uint8_t *)src, g, a, b, h, w)
               : run<float>(which, (float *)dst, (float *)src, g, a, b, h, w);
}
