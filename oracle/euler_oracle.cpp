// TEST INFRASTRUCTURE ONLY -- CPU restatement of the reference's int8 convolution arithmetic.
// See euler_oracle.h for conventions, citations and pinning status.
// Build: g++ -O2 -ffp-contract=off -fopenmp (oracle/Makefile).  Scalar C++ that the compiler
// may auto-vectorise; an AVX-512-VNNI inner loop is selected at run time when the host has it
// (integer arithmetic only, so both paths give identical accumulators).
#include "euler_oracle.h"

#include <algorithm>
#include <cfloat>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <vector>
#include <omp.h>
#if defined(__x86_64__)
#include <immintrin.h>
#endif

namespace {

inline int up16(int x) { return (x + 15) / 16 * 16; }

// _mm512_cvt_roundps_epi32(x, nearest): NaN / out of range -> 0x80000000
inline int32_t cvt_s32_rne(float f)
{
  if (!(f >= -2147483648.0f && f < 2147483648.0f)) return INT32_MIN;
  return (int32_t)nearbyintf(f);
}
// _mm512_cvt_roundps_epu32(x, nearest): NaN / out of range -> 0xffffffff
inline uint32_t cvt_u32_rne(float f)
{
  float r = nearbyintf(f);
  if (!(r >= 0.0f && r < 4294967296.0f)) return 0xffffffffu;
  return (uint32_t)r;
}
// _mm512_cvt_roundps_epi32 / _epu32(x, toward -inf): the store of the F(2x2,3x3) output kernel
inline int32_t cvt_s32_floor(float f)
{
  if (!(f >= -2147483648.0f && f < 2147483648.0f)) return INT32_MIN;
  return (int32_t)floorf(f);
}
inline uint32_t cvt_u32_floor(float f)
{
  float r = floorf(f);
  if (!(r >= 0.0f && r < 4294967296.0f)) return 0xffffffffu;
  return (uint32_t)r;
}
inline uint8_t usat8(uint32_t v) { return v > 255u ? 255 : (uint8_t)v; }         // vpmovusdb
inline int8_t ssat8(int32_t v) { return (int8_t)std::min(127, std::max(-128, v)); } // vpmovsdb

// src/kernel/elk_u8s8_gemm.hxx:200-256 (same form in elk_u8s8_conv.hxx:218-242):
//   fout = cvt(acc) * s + z            -> one fused rounding
//   fout += cvt(old) * sum_S           -> one fused rounding
//   fout = min(max(fout, lower), upper)
inline float epilogue_f32(int32_t acc, float scale, float shift, bool with_sum, int old_q,
                          float sum_S, bool relu, float lo, float hi)
{
  float f = fmaf((float)acc, scale, shift);
  if (with_sum) f = fmaf((float)old_q, sum_S, f);
  if (relu) {
    f = f > lo ? f : lo;   // vmaxps(f, lo)
    f = f < hi ? f : hi;   // vminps(f, hi)
  }
  return f;
}

// g++ contracts `a - b * c` where b*c is (iz*wsum)*scale: the last product fuses into the
// subtraction (src/elx_int8_conv_direct_1x1.cpp:337-343, src/elx_int8_conv_direct.cpp:410-414): the
// reference's translation units compiled with its own flags hold vmulps (iz * wsum), vfmadd132ps
// (bias * out_repS + out_z), vfnmadd132ps (that - product * scale) for the 1x1, k x k and depthwise folds.
inline void fold_scale_shift(const orc_conv_params *p, float w_S, float wsum, float bias,
                             float *scale, float *shift)
{
  float s, z;
  if (p->out_type == ORC_F32 || p->out_type == ORC_S32) {
    s = p->in_scale * w_S;
    z = fmaf(-(p->in_z * wsum), s, bias);
  } else {
    const float out_repS = 1.0f / p->out_scale;
    s = p->in_scale * w_S * out_repS;
    z = fmaf(-(p->in_z * wsum), s, fmaf(bias, out_repS, p->out_z));
  }
  // `mmqf -= sum_z * sum_S` (src/elx_int8_conv_direct_1x1.cpp:349-353): both factors are broadcast scalars,
  // g++ multiplies them once as scalars (vmulss), broadcasts and subtracts (vsubps) -- two roundings
  if (p->with_sum) z = z - p->sum_z * p->sum_scale;
  *scale = s;
  *shift = z;
}

inline int8_t quant_w(float w, float absmax)
{
  if (absmax == 0.0f) return 0;  // reference divides 0/0 here; all-zero channels are excluded from tests
  float t = w * 127.0f;
  t = t / absmax;
  return (int8_t)nearbyintf(t);
}

bool cpu_has_vnni()
{
#if defined(__x86_64__)
  static int v = -1;
  if (v < 0) {
    const char *e = getenv("EULER_ORACLE_NO_VNNI");
    v = (e == nullptr || e[0] == '0') && __builtin_cpu_supports("avx512f")
        && __builtin_cpu_supports("avx512bw") && __builtin_cpu_supports("avx512vnni");
  }
  return v == 1;
#else
  return false;
#endif
}

#if defined(__x86_64__)
// acc[16 oc] += sum over `nq` groups of 4 ic: x[4q..4q+3] (u8) * w[q][16 oc][4 ic] (s8)
__attribute__((target("avx512f,avx512bw,avx512vnni")))
inline void dot_vnni(int32_t *acc, const uint8_t *x, const int8_t *w, int nq)
{
  __m512i a = _mm512_loadu_si512(acc);
  for (int q = 0; q < nq; ++q) {
    int32_t xi;
    memcpy(&xi, x + 4 * q, 4);
    a = _mm512_dpbusd_epi32(a, _mm512_set1_epi32(xi), _mm512_loadu_si512(w + 64 * q));
  }
  _mm512_storeu_si512(acc, a);
}

// one 16-oc block, `T` consecutive positions (stride xs bytes between positions), nq ic-quads
template <int T>
__attribute__((target("avx512f,avx512bw,avx512vnni")))
inline void dot_vnni_tile(int32_t *acc /*[T][16]*/, const uint8_t *x, size_t xs,
                          const int8_t *w, int nq)
{
  __m512i a[T];
  for (int t = 0; t < T; ++t) a[t] = _mm512_loadu_si512(acc + 16 * t);
  for (int q = 0; q < nq; ++q) {
    __m512i wv = _mm512_loadu_si512(w + 64 * q);
    for (int t = 0; t < T; ++t) {
      int32_t xi;
      memcpy(&xi, x + t * xs + 4 * q, 4);
      a[t] = _mm512_dpbusd_epi32(a[t], _mm512_set1_epi32(xi), wv);
    }
  }
  for (int t = 0; t < T; ++t) _mm512_storeu_si512(acc + 16 * t, a[t]);
}
#endif

inline void dot_scalar(int32_t *acc, const uint8_t *x, const int8_t *w, int nq)
{
  for (int q = 0; q < nq; ++q)
    for (int o = 0; o < 16; ++o) {
      int32_t s = 0;
      for (int k = 0; k < 4; ++k) s += (int32_t)x[4 * q + k] * (int32_t)w[64 * q + 4 * o + k];
      acc[o] += s;
    }
}

// ---------------------------------------------------------------------------------------
// Winograd F(4x4,3x3) 1-D stages with the fused roundings of the compiled reference kernels
// ---------------------------------------------------------------------------------------
// src/kernel/elk_conv_wino_4x4_3x3_input.hxx:89-145
inline void wino_in_1d(const float f[6], float o[6])
{
  const float z0 = -2.25f, z1 = -0.390625f, z2 = 0.87890625f, z3 = -2.640625f, z4 = 0.625f, z5 = 1.5f;
  float t0 = fmaf(f[2], z0, f[4]);
  float t1 = fmaf(f[1], z0, f[3]);
  float t2 = fmaf(f[2], z1, f[4]);
  float t3 = fmaf(f[1], z1, f[3]);
  float t4 = fmaf(f[0], z2, f[4]);
  float t5 = fmaf(f[1], z2, f[5]);
  o[0] = fmaf(f[2], z3, t4);
  o[1] = fmaf(t1, z4, t0);
  o[2] = fmaf(-t1, z4, t0);
  o[3] = fmaf(t3, z5, t2);
  o[4] = fmaf(-t3, z5, t2);
  o[5] = fmaf(f[3], z3, t5);
}
// The same stage inside the reference's BORDER kernel (is_border = true), where every input is
// the result of a zero-or-load select: g++ 11.4 -O2 hoists the products of those selected
// values out of the block that adds them, so in the first (column) pass every product of a raw
// input is rounded before the add; products of computed temporaries (t1*z4, t3*z5) still fuse.
// In the second (row) pass everything fuses as in the interior kernel, except t4 of the last
// row (f0*z2 + f4), which is also a rounded product.  Observed on the compiled reference
// kernel (oracle/ref_kernels.cpp), not derivable from the source text.
inline void wino_in_1d_border(const float f[6], float o[6], bool raw_unfused, bool t4_unfused)
{
  const float z0 = -2.25f, z1 = -0.390625f, z2 = 0.87890625f, z3 = -2.640625f, z4 = 0.625f, z5 = 1.5f;
  float t0, t1, t2, t3, t4, t5;
  if (raw_unfused) {
    t0 = f[2] * z0 + f[4];
    t1 = f[1] * z0 + f[3];
    t2 = f[2] * z1 + f[4];
    t3 = f[1] * z1 + f[3];
    t4 = f[0] * z2 + f[4];
    t5 = f[1] * z2 + f[5];
    o[0] = f[2] * z3 + t4;
    o[5] = f[3] * z3 + t5;
  } else {
    t0 = fmaf(f[2], z0, f[4]);
    t1 = fmaf(f[1], z0, f[3]);
    t2 = fmaf(f[2], z1, f[4]);
    t3 = fmaf(f[1], z1, f[3]);
    t4 = t4_unfused ? f[0] * z2 + f[4] : fmaf(f[0], z2, f[4]);
    t5 = fmaf(f[1], z2, f[5]);
    o[0] = fmaf(f[2], z3, t4);
    o[5] = fmaf(f[3], z3, t5);
  }
  o[1] = fmaf(t1, z4, t0);
  o[2] = fmaf(-t1, z4, t0);
  o[3] = fmaf(t3, z5, t2);
  o[4] = fmaf(-t3, z5, t2);
}
// src/kernel/elk_conv_wino_4x4_3x3_weights.hxx:25-72.  z0*f2 has two add/sub uses and fuses
// into both; z1*f0 and z2*f0 are therefore rounded products.
inline void wino_w_1d(float f0, float f1, float f2, float o[6])
{
  const float z0 = 0.26890756302521f, z1 = -0.688403361344538f, z2 = 0.119514472455649f,
              z3 = 1.13777777777778f, z4 = 0.430252100840336f, z5 = 0.179271708683473f;
  float p = z1 * f0;
  float q = z2 * f0;
  float t1 = fmaf(-z0, f2, p);
  float t2 = fmaf(z0, f2, q);
  o[0] = z3 * f0;
  o[1] = fmaf(-z4, f1, t1);
  o[2] = fmaf(z4, f1, t1);
  o[3] = fmaf(z5, f1, t2);
  o[4] = fmaf(-z5, f1, t2);
  o[5] = f2;
}
// src/kernel/elk_conv_wino_4x4_3x3_output.hxx:115-152.  In `a*b + c*d` the first product
// fuses, the second is rounded.
inline void wino_out_1d(const float f[6], float o[4])
{
  const float z0 = 1.5f, z1 = 2.25f, z2 = 3.375f, z3 = 0.625f, z4 = 0.390625f, z5 = 0.244140625f;
  float t0 = f[1] + f[2];
  float t1 = f[3] + f[4];
  float t2 = f[1] - f[2];
  float t3 = f[3] - f[4];
  o[0] = t0 + t1 + f[0];
  o[1] = fmaf(t2, z3, t3 * z0);
  o[2] = fmaf(t0, z4, t1 * z1);
  o[3] = fmaf(t2, z5, t3 * z2) + f[5];
}

// ---------------------------------------------------------------------------------------
// F(2x2,3x3), tile size A = 4: additions and exact products only
// ---------------------------------------------------------------------------------------
// src/kernel/elk_conv_wino_2x2_3x3_input.hxx:104-150.  d, v: [4][4] row-major (row = h).
inline void wino4_tile_input(const float d[16], float v[16])
{
#define D(i, j) d[4 * (i) + (j)]
#define V(i, j) v[4 * (i) + (j)]
  float c1, c2;
  c1 = D(1, 2) - D(1, 0);
  c2 = D(2, 0) - D(2, 2);
  V(0, 0) = (D(0, 0) - D(0, 2)) - c2;
  V(1, 0) = c1 + c2;
  V(2, 0) = c2 - c1;
  V(3, 0) = c1 + (D(3, 0) - D(3, 2));
  c1 = D(1, 2) - D(1, 1);
  c2 = D(2, 2) - D(2, 1);
  V(0, 1) = (D(0, 2) - D(0, 1)) - c2;
  V(1, 1) = c2 - c1;
  V(2, 1) = c2 + c1;
  V(3, 1) = (D(3, 2) - D(3, 1)) - c1;
  c1 = D(1, 1) + D(1, 2);
  c2 = D(2, 1) + D(2, 2);
  V(0, 2) = D(0, 1) + D(0, 2) - c2;
  V(1, 2) = c2 - c1;
  V(2, 2) = c2 + c1;
  V(3, 2) = D(3, 1) + D(3, 2) - c1;
  c1 = D(1, 1) - D(1, 3);
  c2 = D(2, 3) - D(2, 1);
  V(0, 3) = (D(0, 3) - D(0, 1)) - c2;
  V(1, 3) = c1 + c2;
  V(2, 3) = c2 - c1;
  V(3, 3) = (c1 - D(3, 1)) + D(3, 3);
#undef D
#undef V
}
// src/kernel/elk_conv_wino_2x2_3x3_weights.hxx:72-107.  g: [3][3] (kh, kw), u: [4][4].
inline void wino4_tile_weights(const float g[9], float u[16])
{
#define G(i, j) g[3 * (i) + (j)]
#define U(i, j) u[4 * (i) + (j)]
  const float r4 = 0.25f, r2 = 0.5f, z2 = 2.0f;
  U(0, 0) = G(0, 0);
  U(1, 0) = r2 * ((G(0, 0) - G(1, 0)) + G(2, 0));
  U(2, 0) = r2 * ((G(0, 0) + G(1, 0)) + G(2, 0));
  U(3, 0) = G(2, 0);
  const float c10 = r4 * ((G(0, 0) - G(0, 1)) + G(0, 2));
  const float c11 = r4 * ((G(1, 0) - G(1, 1)) + G(1, 2));
  const float c12 = r4 * ((G(2, 0) - G(2, 1)) + G(2, 2));
  U(0, 1) = z2 * c10;
  U(1, 1) = c10 - c11 + c12;
  U(2, 1) = c10 + c11 + c12;
  U(3, 1) = z2 * c12;
  const float c20 = r4 * (G(0, 0) + G(0, 1) + G(0, 2));
  const float c21 = r4 * (G(1, 0) + G(1, 1) + G(1, 2));
  const float c22 = r4 * (G(2, 0) + G(2, 1) + G(2, 2));
  U(0, 2) = z2 * c20;
  U(1, 2) = c20 - c21 + c22;
  U(2, 2) = c20 + c21 + c22;
  U(3, 2) = z2 * c22;
  U(0, 3) = G(0, 2);
  U(1, 3) = r2 * (G(0, 2) - G(1, 2) + G(2, 2));
  U(2, 3) = r2 * (G(0, 2) + G(1, 2) + G(2, 2));
  U(3, 3) = G(2, 2);
#undef G
#undef U
}
// src/kernel/elk_conv_wino_2x2_3x3_output.hxx:76-95.  m: [4][4], y: [2][2].
inline void wino4_tile_output(const float m[16], float y[4])
{
#define T(i, j) m[4 * (i) + (j)]
  const float c0 = T(1, 0) + T(1, 1) + T(1, 2);
  const float c1 = T(2, 0) + T(2, 1) + T(2, 2);
  const float c2 = T(1, 2) + T(1, 3) - T(1, 1);
  const float c3 = T(2, 2) + T(2, 3) - T(2, 1);
  y[0] = T(0, 0) + T(0, 1) + T(0, 2) + c0 + c1;            // p00
  y[2] = c1 - c0 + T(3, 0) + T(3, 1) + T(3, 2);            // p10
  y[1] = T(0, 2) - T(0, 1) + T(0, 3) + c2 + c3;            // p01
  y[3] = c3 - c2 - T(3, 1) + T(3, 2) + T(3, 3);            // p11
#undef T
}

// ---------------------------------------------------------------------------------------
// F(3x3,3x3), tile size A = 5.  Products with 0.5 and 2 are exact, so only the products with
// 1.5 (input) and 1/3, 2/3, 4/3 (output) have a fused / unfused question; the compiled
// reference kernels answer it (tests/test_oracle_ref_kernels.py).
// ---------------------------------------------------------------------------------------
// src/kernel/elk_conv_wino_3x3_3x3_input.hxx:91-128.  f2 * 1.5 + f3 is one fused rounding, except in the
// first (column) pass of the BORDER kernel, whose inputs are zero-or-load selects: there the product is
// rounded first -- the same behaviour of the compiled reference as in its F(4x4,3x3) border kernel.
inline void wino5_in_1d(const float f[5], float o[5], bool fuse15)
{
  const float z0 = 0.5f, z1 = 1.5f;
  const float t0 = f[1] * z0;
  const float t1 = f[2] * z0;
  const float t2 = f[3] - f[1];
  o[0] = f[0] * z0 - t1 - t2;
  o[1] = f[3] - t0 - t1;
  o[2] = (fuse15 ? fmaf(f[2], z1, f[3]) : f[2] * z1 + f[3]) + t0;
  o[3] = t2;
  o[4] = f[3] * z0 + f[4] - f[2] - t0;
}
// src/kernel/elk_conv_wino_3x3_3x3_weights.hxx:27-66 (every product exact)
inline void wino5_w_1d(float f0, float f1, float f2, float o[5])
{
  const float t0 = f0 * 2.0f;
  const float t1 = f0 + f2;
  o[0] = t0;
  o[1] = f1 - t1;
  o[2] = f1 + t1;
  o[3] = f2 * 0.5f + t0 - f1;
  o[4] = f2;
}
// src/kernel/elk_conv_wino_3x3_3x3_output.hxx:93-131: f2*z0 fuses into both of its uses, every
// other product into the addition that follows it
inline void wino5_out_1d(const float f[5], float o[3])
{
  const float z0 = 0.3333333333333333f, z1 = 0.6666666666666666f, z2 = 1.3333333333333333f;
  const float t1 = fmaf(f[2], z0, f[1]);
  o[0] = fmaf(f[3], z2, f[0]) + t1;
  o[1] = fmaf(-f[3], z1, fmaf(f[2], z0, -f[1]));
  o[2] = fmaf(f[3], z0, f[4]) + t1;
}

inline int wino_tile_A(const orc_conv_params *p) { return (p->wino_tile == 4 || p->wino_tile == 5) ? p->wino_tile : 6; }

struct WinoGeom {
  int A, M, ht, wt, nt, t, IC2, OC2;
};
inline WinoGeom wino_geom(const orc_conv_params *p)
{
  WinoGeom g;
  g.A = wino_tile_A(p);
  g.M = g.A - 2;
  g.ht = (p->oh + g.M - 1) / g.M;  // (oh + A - K) / (A - K + 1), src/elx_int8_conv_wino.cpp:24-27
  g.wt = (p->ow + g.M - 1) / g.M;
  g.nt = g.ht * g.wt;
  g.t = g.nt * p->n;
  g.IC2 = up16(p->ic) / 16;
  g.OC2 = up16(p->oc) / 16;
  return g;
}

extern "C" void orc_wino_tile_input_a(int A, int border, const float *d, float *v);

// gather one A x A tile of one channel (zero outside the image) and transform it
inline void wino_tile_from_input(const orc_conv_params *p, const float *in_plane /*[ih][iw][16]*/,
                                 int th, int tw, int v, float out[36])
{
  float d[36];
  const int A = wino_tile_A(p), M = A - 2;
  const int h0 = M * th - p->pad_t, w0 = M * tw - p->pad_l;
  bool border = false;  // input_tile_iter::is_border, src/elx_conv_wino_trans_input.hpp:247-249
  for (int i = 0; i < A; ++i)
    for (int j = 0; j < A; ++j) {
      int h = h0 + i, w = w0 + j;
      bool inside = h >= 0 && h < p->ih && w >= 0 && w < p->iw;
      border |= !inside;
      d[A * i + j] = inside ? in_plane[((size_t)h * p->iw + w) * 16 + v] : 0.0f;
    }
  orc_wino_tile_input_a(A, border, d, out);
}

} // namespace

extern "C" {

int orc_num_threads(void) { return omp_get_max_threads(); }
int orc_has_vnni(void) { return cpu_has_vnni() ? 1 : 0; }

// ---------------------------------------------------------------------------------------
// reorders -- src/elx_reorder.cpp:35-93
// ---------------------------------------------------------------------------------------
#define DEF_REORDER_ACT(T, sfx)                                                                  \
  void orc_reorder_nchw_to_blocked_##sfx(T *dst, const T *src, int n, int c, int h, int w)        \
  {                                                                                              \
    const int C2 = up16(c) / 16;                                                                 \
    for (int _n = 0; _n < n; ++_n)                                                               \
      for (int _c = 0; _c < C2; ++_c)                                                            \
        for (int _h = 0; _h < h; ++_h)                                                           \
          for (int _w = 0; _w < w; ++_w)                                                         \
            for (int v = 0; v < 16; ++v) {                                                       \
              int ch = _c * 16 + v;                                                              \
              dst[((((size_t)_n * C2 + _c) * h + _h) * w + _w) * 16 + v] =                        \
                  ch < c ? src[(((size_t)_n * c + ch) * h + _h) * w + _w] : (T)0;                 \
            }                                                                                    \
  }                                                                                              \
  void orc_reorder_blocked_to_nchw_##sfx(T *dst, const T *src, int n, int c, int h, int w)        \
  {                                                                                              \
    const int C2 = up16(c) / 16;                                                                 \
    for (int _n = 0; _n < n; ++_n)                                                               \
      for (int ch = 0; ch < c; ++ch)                                                             \
        for (int _h = 0; _h < h; ++_h)                                                           \
          for (int _w = 0; _w < w; ++_w)                                                         \
            dst[(((size_t)_n * c + ch) * h + _h) * w + _w] =                                      \
                src[((((size_t)_n * C2 + ch / 16) * h + _h) * w + _w) * 16 + ch % 16];            \
  }
DEF_REORDER_ACT(float, f32)
DEF_REORDER_ACT(uint8_t, u8)

void orc_reorder_oihw_to_blocked_f32(float *dst, const float *src, int o, int i, int h, int w)
{
  const int O2 = up16(o) / 16, I2 = up16(i) / 16;
  for (int _o = 0; _o < O2; ++_o)
    for (int _i = 0; _i < I2; ++_i)
      for (int _h = 0; _h < h; ++_h)
        for (int _w = 0; _w < w; ++_w)
          for (int iv = 0; iv < 16; ++iv)
            for (int ov = 0; ov < 16; ++ov) {
              int oc = _o * 16 + ov, ic = _i * 16 + iv;
              dst[(((((size_t)_o * I2 + _i) * h + _h) * w + _w) * 16 + iv) * 16 + ov] =
                  (oc < o && ic < i) ? src[(((size_t)oc * i + ic) * h + _h) * w + _w] : 0.0f;
            }
}

void orc_reorder_blocked_to_oihw_f32(float *dst, const float *src, int o, int i, int h, int w)
{
  const int I2 = up16(i) / 16;
  for (int oc = 0; oc < o; ++oc)
    for (int ic = 0; ic < i; ++ic)
      for (int _h = 0; _h < h; ++_h)
        for (int _w = 0; _w < w; ++_w)
          dst[(((size_t)oc * i + ic) * h + _h) * w + _w] =
              src[(((((size_t)(oc / 16) * I2 + ic / 16) * h + _h) * w + _w) * 16 + ic % 16) * 16 + oc % 16];
}

// ---------------------------------------------------------------------------------------
// harness input quantization -- tests/elt_conv_utils.cpp:354-401: the helper named
// rounding_to_nearest_even truncates, then resolves the fraction against 0.5 with a rule that
// sends exact ties to the ODD neighbour, and the result is narrowed with a plain (uint8_t) cast.
// ---------------------------------------------------------------------------------------
void orc_quantize_input_u8(uint8_t *dst, const float *src, size_t count, float scale, float z)
{
  for (size_t i = 0; i < count; ++i) {
    float f = src[i] / scale + z;
    int32_t i32 = (int32_t)f;
    int32_t r;
    if (i32 >= 0) {
      if (i32 % 2) r = (f - (float)i32 <= 0.5f) ? i32 : i32 + 1;
      else r = (f - (float)i32 >= 0.5f) ? i32 + 1 : i32;
    } else {
      if (i32 % 2) r = ((float)i32 - f <= 0.5f) ? i32 : i32 - 1;
      else r = ((float)i32 - f >= 0.5f) ? i32 - 1 : i32;
    }
    dst[i] = (uint8_t)r;
  }
}

// ---------------------------------------------------------------------------------------
// harness fp32 reference convolution -- tests/elt_conv_utils.cpp:666-750.  The accumulation
// `out[...] += in[...] * w[...]` is one vfmadd in the compiled harness (g++ -O2 contracts it).
// ---------------------------------------------------------------------------------------
int orc_ref_conv_f32(const orc_conv_params *p, float *output, const float *input, const float *weights, const float *bias)
{
  if (p->g < 1 || p->ic % p->g || p->oc % p->g) return -1;
  const int icg = p->ic / p->g, ocg = p->oc / p->g;
#pragma omp parallel for collapse(2)
  for (int n = 0; n < p->n; ++n)
    for (int oc = 0; oc < p->oc; ++oc) {
      const int grp = oc / ocg;
      for (int oh = 0; oh < p->oh; ++oh)
        for (int ow = 0; ow < p->ow; ++ow) {
          float *o = &output[(((size_t)n * p->oc + oc) * p->oh + oh) * p->ow + ow];
          const float b = p->with_bias ? bias[oc] : 0.0f;
          float acc = p->with_sum ? *o + b : b;
          for (int i = 0; i < icg; ++i)
            for (int kh = 0; kh < p->kh; ++kh) {
              const int ih = oh * p->stride_h - p->pad_t + kh;
              if (ih < 0 || ih >= p->ih) continue;
              for (int kw = 0; kw < p->kw; ++kw) {
                const int iw = ow * p->stride_w - p->pad_l + kw;
                if (iw < 0 || iw >= p->iw) continue;
                acc = fmaf(input[(((size_t)n * p->ic + grp * icg + i) * p->ih + ih) * p->iw + iw],
                           weights[(((size_t)oc * icg + i) * p->kh + kh) * p->kw + kw], acc);
              }
            }
          *o = (p->with_relu && acc < 0.0f) ? 0.0f : acc;
        }
    }
  return 0;
}

// tests/elt_conv_utils.cpp:306-346; `diff` is a double there (the 0.000001 literal promotes it), so the
// asymmetric scale and zero point are double quotients narrowed on assignment
void orc_calibrate_output_quant(int with_relu, int out_type, int with_sum, float out_min, float out_max, float sum_absmax,
                                float representation, float *output_scale, float *output_z, float *sum_scale)
{
  const float abs_cur = out_min > 0 ? out_min : -out_min;
  const float abs_max = out_max > abs_cur ? out_max : abs_cur;
  if (with_relu || out_type == ORC_S8) {
    *output_scale = abs_max / representation;
    *output_z = 0.0f;
  } else {
    const double diff = (double)(out_max - out_min) + 0.000001;
    *output_scale = (float)(diff / representation);
    *output_z = (float)((double)(-out_min * representation) / diff);
  }
  if (with_sum) {
    const float sum_operand_scale = sum_absmax / representation;
    *sum_scale = sum_operand_scale / *output_scale;
  }
}

int orc_epilogue(int out_kind, int32_t acc, float scale, float shift, int with_sum, int old_q,
                 float sum_scale, int with_relu, float lo, float hi, float *fout)
{
  float f = epilogue_f32(acc, scale, shift, with_sum, old_q, sum_scale, with_relu, lo, hi);
  if (fout) *fout = f;
  if (out_kind == ORC_U8) return usat8((uint32_t)cvt_s32_rne(f));
  if (out_kind == ORC_S8) return ssat8(cvt_s32_rne(f));
  return 0;
}

// ---------------------------------------------------------------------------------------
// direct 1x1 / KxK
// ---------------------------------------------------------------------------------------
int orc_direct_prepare(const orc_conv_params *p, const float *w, const float *bias, int8_t *wq,
                       float *scale, float *shift, int32_t *wsum)
{
  const int OCp = up16(p->oc), ICp = up16(p->ic), I2 = ICp / 16, KH = p->kh, KW = p->kw;
  auto widx = [&](int oc, int ic, int kh, int kw) {
    return (((((size_t)(oc / 16) * I2 + ic / 16) * KH + kh) * KW + kw) * 16 + ic % 16) * 16 + oc % 16;
  };
#pragma omp parallel for
  for (int oc = 0; oc < OCp; ++oc) {
    float absmax = 0.0f;
    for (int ic = 0; ic < p->ic; ++ic)
      for (int kh = 0; kh < KH; ++kh)
        for (int kw = 0; kw < KW; ++kw) absmax = std::max(absmax, std::fabs(w[widx(oc, ic, kh, kw)]));
    int32_t acc = 0;
    for (int ic = 0; ic < ICp; ++ic)
      for (int kh = 0; kh < KH; ++kh)
        for (int kw = 0; kw < KW; ++kw) {
          int8_t q = ic < p->ic ? quant_w(w[widx(oc, ic, kh, kw)], absmax) : 0;
          wq[(((size_t)oc * ICp + ic) * KH + kh) * KW + kw] = q;
          acc += q;
        }
    wsum[oc] = acc;
    const float w_S = absmax / 127.0f;
    const float b = p->with_bias ? bias[oc] : 0.0f;
    fold_scale_shift(p, w_S, (float)acc, b, &scale[oc], &shift[oc]);
  }
  return 0;
}

// shift_px_stride == 0: shift is [OCp]; otherwise a per-pixel map [oh][ow][OCp] (shift_px_stride = OCp)
static int direct_execute_impl(const orc_conv_params *p, const uint8_t *input, const int8_t *wq,
                               const float *scale, const float *shift, size_t shift_px_stride, void *output,
                               int32_t *acc_out)
{
  const int OCp = up16(p->oc), ICp = up16(p->ic), I2 = ICp / 16, O2 = OCp / 16;
  const int KH = p->kh, KW = p->kw, IH = p->ih, IW = p->iw, OH = p->oh, OW = p->ow;
  if (p->g != 1) return -1;
  // repack to [oc2][kh][kw][ic/4][16 oc][4 ic] (the reference's V1/V/Vx inner order,
  // src/elx_int8_conv_direct.cpp:425-426)
  std::vector<int8_t> wt((size_t)O2 * KH * KW * ICp * 16);
  for (int oc = 0; oc < OCp; ++oc)
    for (int ic = 0; ic < ICp; ++ic)
      for (int kh = 0; kh < KH; ++kh)
        for (int kw = 0; kw < KW; ++kw)
          wt[((((size_t)(oc / 16) * KH + kh) * KW + kw) * (ICp / 4) + ic / 4) * 64 + (oc % 16) * 4 + ic % 4] =
              wq[(((size_t)oc * ICp + ic) * KH + kh) * KW + kw];
  const bool vnni = cpu_has_vnni();
  const bool relu = p->with_relu != 0, with_sum = p->with_sum != 0;

#pragma omp parallel for collapse(3) schedule(static)
  for (int n = 0; n < p->n; ++n)
    for (int o2 = 0; o2 < O2; ++o2)
      for (int oh = 0; oh < OH; ++oh) {
        std::vector<int32_t> rowacc((size_t)OW * 16, 0);
        for (int kh = 0; kh < KH; ++kh) {
          const int ih = oh * p->stride_h + kh - p->pad_t;
          if (ih < 0 || ih >= IH) continue;  // padded taps are skipped (src/elx_int8_conv_direct.cpp:512-520)
          for (int kw = 0; kw < KW; ++kw)
            for (int i2 = 0; i2 < I2; ++i2) {
              const int8_t *wp = &wt[((((size_t)o2 * KH + kh) * KW + kw) * (ICp / 4) + i2 * 4) * 64];
              const uint8_t *xrow = input + (((size_t)n * I2 + i2) * IH + ih) * IW * 16;
              int ow = 0;
#if defined(__x86_64__)
              if (vnni && p->stride_w == 1) {
                // positions whose tap falls inside the image: ow + kw - pad_l in [0, IW)
                int lo = std::max(0, p->pad_l - kw), hi = std::min(OW, IW + p->pad_l - kw);
                ow = lo;
                for (; ow + 14 <= hi; ow += 14)
                  dot_vnni_tile<14>(&rowacc[(size_t)ow * 16], xrow + (size_t)(ow + kw - p->pad_l) * 16, 16, wp, 4);
                for (; ow < hi; ++ow)
                  dot_vnni(&rowacc[(size_t)ow * 16], xrow + (size_t)(ow + kw - p->pad_l) * 16, wp, 4);
                continue;
              }
#endif
              for (ow = 0; ow < OW; ++ow) {
                const int iw = ow * p->stride_w + kw - p->pad_l;
                if (iw < 0 || iw >= IW) continue;
#if defined(__x86_64__)
                if (vnni) dot_vnni(&rowacc[(size_t)ow * 16], xrow + (size_t)iw * 16, wp, 4);
                else
#endif
                  dot_scalar(&rowacc[(size_t)ow * 16], xrow + (size_t)iw * 16, wp, 4);
              }
            }
        }
        const size_t obase = (((size_t)n * O2 + o2) * OH + oh) * OW * 16;
        for (int ow = 0; ow < OW; ++ow)
          for (int v = 0; v < 16; ++v) {
            const size_t oi = obase + (size_t)ow * 16 + v;
            const int oc = o2 * 16 + v;
            const int32_t a = rowacc[(size_t)ow * 16 + v];
            if (acc_out) acc_out[oi] = a;
            if (p->out_type == ORC_S32) { ((int32_t *)output)[oi] = a; continue; }
            int old_q = 0;
            if (with_sum) old_q = p->out_type == ORC_U8 ? (int)((uint8_t *)output)[oi]
                                 : p->out_type == ORC_S8 ? (int)((int8_t *)output)[oi] : 0;
            // the f32-output path of the reference has no sum fusion
            // (src/elx_int8_conv_direct.cpp:656-716, src/kernel/elk_u8s8_gemm.hxx:234-236)
            const float sh = shift[((size_t)oh * OW + ow) * shift_px_stride + oc];
            float f = epilogue_f32(a, scale[oc], sh, with_sum && p->out_type != ORC_F32, old_q,
                                   p->sum_scale, relu, p->relu_lo, p->relu_hi);
            if (p->out_type == ORC_F32) ((float *)output)[oi] = f;
            else if (p->out_type == ORC_U8) ((uint8_t *)output)[oi] = usat8((uint32_t)cvt_s32_rne(f));
            else ((int8_t *)output)[oi] = ssat8(cvt_s32_rne(f));
          }
      }
  return 0;
}

int orc_direct_execute(const orc_conv_params *p, const uint8_t *input, const int8_t *wq,
                       const float *scale, const float *shift, void *output, int32_t *acc_out)
{
  return direct_execute_impl(p, input, wq, scale, shift, 0, output, acc_out);
}

// Non-zero input zero point with padding (src/elx_int8_conv_direct.cpp:227-423): a padded tap is
// skipped, so it must not take part in the "- in_z * sum(w) * scale" term either.  The reference
// keeps one sum of weights per range of valid kernel rows and columns (wacc_h_ranges_ /
// wacc_w_ranges_) and one shift per (row class, width block, position in the block); what it
// encodes is: the shift of an output pixel folds the sum of the weights of the taps that fall
// inside the image for THAT pixel.  shift_map is [oh][ow][OCp].
int orc_direct_border_shifts(const orc_conv_params *p, const float *w, const float *bias, float *shift_map)
{
  const int OCp = up16(p->oc), ICp = up16(p->ic), I2 = ICp / 16, KH = p->kh, KW = p->kw;
  auto widx = [&](int oc, int ic, int kh, int kw) {
    return (((((size_t)(oc / 16) * I2 + ic / 16) * KH + kh) * KW + kw) * 16 + ic % 16) * 16 + oc % 16;
  };
#pragma omp parallel for
  for (int oc = 0; oc < OCp; ++oc) {
    float absmax = 0.0f;
    for (int ic = 0; ic < p->ic; ++ic)
      for (int kh = 0; kh < KH; ++kh)
        for (int kw = 0; kw < KW; ++kw) absmax = std::max(absmax, std::fabs(w[widx(oc, ic, kh, kw)]));
    std::vector<int32_t> tapsum((size_t)KH * KW, 0);   // sum over input channels per tap
    for (int kh = 0; kh < KH; ++kh)
      for (int kw = 0; kw < KW; ++kw)
        for (int ic = 0; ic < p->ic; ++ic) tapsum[(size_t)kh * KW + kw] += quant_w(w[widx(oc, ic, kh, kw)], absmax);
    const float w_S = absmax / 127.0f;
    const float b = p->with_bias ? bias[oc] : 0.0f;
    for (int oh = 0; oh < p->oh; ++oh)
      for (int ow = 0; ow < p->ow; ++ow) {
        int32_t acc = 0;
        for (int kh = 0; kh < KH; ++kh) {
          const int ih = oh * p->stride_h + kh - p->pad_t;
          if (ih < 0 || ih >= p->ih) continue;
          for (int kw = 0; kw < KW; ++kw) {
            const int iw = ow * p->stride_w + kw - p->pad_l;
            if (iw < 0 || iw >= p->iw) continue;
            acc += tapsum[(size_t)kh * KW + kw];
          }
        }
        float sc, sh;
        fold_scale_shift(p, w_S, (float)acc, b, &sc, &sh);
        shift_map[((size_t)oh * p->ow + ow) * OCp + oc] = sh;
      }
  }
  return 0;
}

int orc_direct_execute_border(const orc_conv_params *p, const uint8_t *input, const int8_t *wq,
                              const float *scale, const float *shift_map, void *output, int32_t *acc_out)
{
  return direct_execute_impl(p, input, wq, scale, shift_map, (size_t)up16(p->oc), output, acc_out);
}

// ---------------------------------------------------------------------------------------
// depthwise 3x3
// ---------------------------------------------------------------------------------------
int orc_depthwise_prepare(const orc_conv_params *p, const float *w, const float *bias, int8_t *wq,
                          float *scale, float *shift, int32_t *wsum)
{
  const int G = up16(p->g);
  for (int g = 0; g < G; ++g) {
    if (g >= p->g) {
      for (int k = 0; k < 9; ++k) wq[(size_t)g * 9 + k] = 0;
      scale[g] = 0.0f; shift[g] = 0.0f; wsum[g] = 0;
      continue;
    }
    float absmax = 0.0f;
    for (int k = 0; k < 9; ++k) absmax = std::max(std::fabs(w[(size_t)g * 9 + k]), absmax);
    int32_t acc = 0;
    for (int k = 0; k < 9; ++k) {
      // t0 = t0 * EL_INT8_MAX / absmax; (int8_t)std::rint(t0)
      // (src/elx_int8_conv_direct_depthwise.cpp:222-233)
      int8_t q = quant_w(w[(size_t)g * 9 + k], absmax);
      wq[(size_t)g * 9 + k] = q;
      acc += q;
    }
    wsum[g] = acc;
    orc_conv_params q = *p;
    q.with_sum = 0;  // no sum term in the depthwise folding (src/elx_int8_conv_direct_depthwise.cpp:261-291)
    fold_scale_shift(&q, absmax / 127.0f, (float)acc, p->with_bias ? bias[g] : 0.0f, &scale[g], &shift[g]);
  }
  return 0;
}

int orc_depthwise_execute(const orc_conv_params *p, const uint8_t *input, const int8_t *wq,
                          const float *scale, const float *shift, void *output, int32_t *acc_out)
{
  const int G2 = up16(p->g) / 16, IH = p->ih, IW = p->iw, OH = p->oh, OW = p->ow;
  // stride 1 and 2 share everything but the input index (the kernel's S template parameter,
  // src/kernel/elk_u8s8_depthwise_conv.hxx:153,176-178,371-403)
  if (p->kh != 3 || p->kw != 3 || p->stride_h < 1 || p->stride_h > 2 || p->stride_w != p->stride_h) return -1;
  if (p->out_type != ORC_U8 && p->out_type != ORC_S8) return -1;
  const int T = p->T > 0 ? std::min(p->T, OW) : 1;
  const int wt = (OW + T - 1) / T;
  const int Tr = OW % T ? OW % T : T;
  const bool relu = p->with_relu != 0;
#pragma omp parallel for collapse(2) schedule(static)
  for (int n = 0; n < p->n; ++n)
    for (int g2 = 0; g2 < G2; ++g2) {
      const uint8_t *in = input + ((size_t)n * G2 + g2) * IH * IW * 16;
      const size_t obase = ((size_t)n * G2 + g2) * OH * OW * 16;
      for (int oh = 0; oh < OH; ++oh)
        for (int _wt = 0; _wt < wt; ++_wt) {
          const int Tz = _wt == wt - 1 ? Tr : T;
          for (int _T = 0; _T < Tz; ++_T) {
            const int ow = _wt * T + _T;
            for (int v = 0; v < 16; ++v) {
              const int g = g2 * 16 + v;
              int32_t a = 0;
              for (int kh = 0; kh < 3; ++kh) {
                int ih = oh * p->stride_h + kh - p->pad_t;
                if (ih < 0 || ih >= IH) continue;
                for (int kw = 0; kw < 3; ++kw) {
                  int iw = ow * p->stride_w + kw - p->pad_l;
                  if (iw < 0 || iw >= IW) continue;
                  a += (int32_t)in[((size_t)ih * IW + iw) * 16 + v] * (int32_t)wq[(size_t)g * 9 + kh * 3 + kw];
                }
              }
              const size_t oi = obase + ((size_t)oh * OW + ow) * 16 + v;
              if (acc_out) acc_out[oi] = a;
              float f = epilogue_f32(a, scale[g], shift[g], false, 0, 0.0f, relu, p->relu_lo, p->relu_hi);
              if (p->out_type == ORC_U8) {
                if (_T < 4 * (Tz / 4)) {
                  // groups of four columns: round toward -inf, bytes merged by shift-and-add
                  // with no saturation (src/kernel/elk_u8s8_depthwise_conv.hxx:257-286,406-454).
                  // The byte is exact whenever the value lies in [0,255]; outside that range the
                  // reference's carries spill into neighbouring bytes, which callers must avoid.
                  int32_t fl = (!(f >= -2147483648.0f && f < 2147483648.0f)) ? INT32_MIN : (int32_t)floorf(f);
                  ((uint8_t *)output)[oi] = (uint8_t)fl;
                } else {
                  ((uint8_t *)output)[oi] = usat8((uint32_t)cvt_s32_rne(f));
                }
              } else {
                ((int8_t *)output)[oi] = ssat8(cvt_s32_rne(f));
              }
            }
          }
        }
    }
  return 0;
}

// ---------------------------------------------------------------------------------------
// Winograd F(4x4,3x3)
// ---------------------------------------------------------------------------------------
void orc_wino_tile_input(const float d[36], float v[36])
{
  float m[36];
  for (int j = 0; j < 6; ++j) {  // along h for every column j
    float f[6], o[6];
    for (int i = 0; i < 6; ++i) f[i] = d[6 * i + j];
    wino_in_1d(f, o);
    for (int i = 0; i < 6; ++i) m[6 * i + j] = o[i];
  }
  for (int i = 0; i < 6; ++i) wino_in_1d(&m[6 * i], &v[6 * i]);  // along w for every row i
}

void orc_wino_tile_input_border(const float d[36], float v[36])
{
  float m[36];
  for (int j = 0; j < 6; ++j) {
    float f[6], o[6];
    for (int i = 0; i < 6; ++i) f[i] = d[6 * i + j];
    wino_in_1d_border(f, o, true, false);
    for (int i = 0; i < 6; ++i) m[6 * i + j] = o[i];
  }
  for (int i = 0; i < 6; ++i) wino_in_1d_border(&m[6 * i], &v[6 * i], false, i == 5);
}

void orc_wino_tile_weights(const float g[9], float u[36])
{
  float M[6][3];
  for (int i = 0; i < 3; ++i) {  // along kh for every kw = i
    float o[6];
    wino_w_1d(g[0 * 3 + i], g[1 * 3 + i], g[2 * 3 + i], o);
    for (int k = 0; k < 6; ++k) M[k][i] = o[k];
  }
  for (int i = 0; i < 6; ++i) wino_w_1d(M[i][0], M[i][1], M[i][2], &u[6 * i]);
}

void orc_wino_tile_output(const float m[36], float y[16])
{
  float M[4][6];
  for (int i = 0; i < 6; ++i) {  // along hA for every column i
    float f[6], o[4];
    for (int k = 0; k < 6; ++k) f[k] = m[6 * k + i];
    wino_out_1d(f, o);
    for (int k = 0; k < 4; ++k) M[k][i] = o[k];
  }
  for (int i = 0; i < 4; ++i) wino_out_1d(M[i], &y[4 * i]);
}

// any tile size: A = 6 as above, A = 4 F(2x2,3x3), A = 5 F(3x3,3x3); arrays are [A][A] row-major
void orc_wino_tile_input_a(int A, int border, const float *d, float *v)
{
  if (A == 4) {
    wino4_tile_input(d, v);
  } else if (A == 5) {
    float m[25];
    for (int j = 0; j < 5; ++j) {
      float f[5], o[5];
      for (int i = 0; i < 5; ++i) f[i] = d[5 * i + j];
      wino5_in_1d(f, o, !border);
      for (int i = 0; i < 5; ++i) m[5 * i + j] = o[i];
    }
    for (int i = 0; i < 5; ++i) wino5_in_1d(&m[5 * i], &v[5 * i], true);
  } else if (border) {
    orc_wino_tile_input_border(d, v);
  } else {
    orc_wino_tile_input(d, v);
  }
}

void orc_wino_tile_weights_a(int A, const float g[9], float *u)
{
  if (A == 4) {
    wino4_tile_weights(g, u);
  } else if (A == 5) {
    float M[5][3];
    for (int i = 0; i < 3; ++i) {
      float o[5];
      wino5_w_1d(g[0 * 3 + i], g[1 * 3 + i], g[2 * 3 + i], o);
      for (int k = 0; k < 5; ++k) M[k][i] = o[k];
    }
    for (int i = 0; i < 5; ++i) wino5_w_1d(M[i][0], M[i][1], M[i][2], &u[5 * i]);
  } else {
    orc_wino_tile_weights(g, u);
  }
}

// y: [A - 2][A - 2] row-major
void orc_wino_tile_output_a(int A, const float *m, float *y)
{
  if (A == 4) {
    wino4_tile_output(m, y);
  } else if (A == 5) {
    float M[3][5];
    for (int i = 0; i < 5; ++i) {
      float f[5], o[3];
      for (int k = 0; k < 5; ++k) f[k] = m[5 * k + i];
      wino5_out_1d(f, o);
      for (int k = 0; k < 3; ++k) M[k][i] = o[k];
    }
    for (int i = 0; i < 3; ++i) wino5_out_1d(M[i], &y[3 * i]);
  } else {
    orc_wino_tile_output(m, y);
  }
}

int orc_wino_tiles(const orc_conv_params *p) { return wino_geom(p).t; }

int orc_wino_tinput_range(const orc_conv_params *p, const float *input, float *min_out, float *max_out)
{
  const WinoGeom g = wino_geom(p);
  float mn = FLT_MAX, mx = -FLT_MAX;
#pragma omp parallel for collapse(2) reduction(min : mn) reduction(max : mx)
  for (int n = 0; n < p->n; ++n)
    for (int c2 = 0; c2 < g.IC2; ++c2) {
      const float *plane = input + ((size_t)n * g.IC2 + c2) * p->ih * p->iw * 16;
      for (int th = 0; th < g.ht; ++th)
        for (int tw = 0; tw < g.wt; ++tw)
          for (int v = 0; v < 16; ++v) {
            if (c2 * 16 + v >= p->ic) continue;
            float o[36];
            wino_tile_from_input(p, plane, th, tw, v, o);
            for (int k = 0; k < g.A * g.A; ++k) { mn = std::min(mn, o[k]); mx = std::max(mx, o[k]); }
          }
    }
  *min_out = mn; *max_out = mx;
  return 0;
}

int orc_wino_prepare(const orc_conv_params *p, const float *w, int8_t *twq, float *tscale, float *tshift)
{
  const int OCp = up16(p->oc), ICp = up16(p->ic), I2 = ICp / 16;
  const int A = wino_tile_A(p), AA = A * A;
  const float tin_S = p->tin_scale, tin_z = std::ceil(p->tin_z);  // src/elx_int8_conv_wino.cpp:270-276
  std::vector<float> U((size_t)AA * OCp * ICp);
#pragma omp parallel for collapse(2)
  for (int oc = 0; oc < OCp; ++oc)
    for (int ic = 0; ic < ICp; ++ic) {
      float g[9], u[36];
      for (int k = 0; k < 9; ++k)
        g[k] = w[((((size_t)(oc / 16) * I2 + ic / 16) * 9 + k) * 16 + ic % 16) * 16 + oc % 16];
      orc_wino_tile_weights_a(A, g, u);
      for (int a = 0; a < AA; ++a) U[((size_t)a * OCp + oc) * ICp + ic] = u[a];
    }
  // src/elx_conv_wino_trans_weights.cpp:437-535
#pragma omp parallel for collapse(2)
  for (int a = 0; a < AA; ++a)
    for (int oc = 0; oc < OCp; ++oc) {
      const float *u = &U[((size_t)a * OCp + oc) * ICp];
      float absmax = 0.0f;
      for (int ic = 0; ic < ICp; ++ic) absmax = std::max(absmax, std::fabs(u[ic]));
      float acc = 0.0f;
      for (int ic = 0; ic < ICp; ++ic) {
        int8_t q = quant_w(u[ic], absmax);
        twq[((size_t)a * OCp + oc) * ICp + ic] = q;
        acc += (float)q;
      }
      float Sw = absmax;
      Sw /= 127.0f;
      Sw = Sw * tin_S;
      float Zw = -acc * Sw * tin_z;
      tscale[(size_t)a * OCp + oc] = Sw;
      tshift[(size_t)a * OCp + oc] = Zw;
    }
  return 0;
}

int orc_wino_trans_input(const orc_conv_params *p, const float *input, uint8_t *tinput)
{
  const WinoGeom g = wino_geom(p);
  const float tin_repS = 1.0f / p->tin_scale;
  const float mrepS = p->in_scale * tin_repS;   // src/elx_conv_wino_trans_input.cpp:617-618
  const float mz = std::ceil(p->tin_z);
#pragma omp parallel for collapse(2)
  for (int n = 0; n < p->n; ++n)
    for (int c2 = 0; c2 < g.IC2; ++c2) {
      const float *plane = input + ((size_t)n * g.IC2 + c2) * p->ih * p->iw * 16;
      for (int th = 0; th < g.ht; ++th)
        for (int tw = 0; tw < g.wt; ++tw) {
          const size_t t = (size_t)n * g.nt + (size_t)th * g.wt + tw;
          for (int v = 0; v < 16; ++v) {
            float o[36];
            wino_tile_from_input(p, plane, th, tw, v, o);
            for (int a = 0; a < g.A * g.A; ++a) {
              float f = fmaf(o[a], mrepS, mz);
              tinput[(((size_t)a * g.IC2 + c2) * g.t + t) * 16 + v] = usat8(cvt_u32_rne(f));
            }
          }
        }
    }
  return 0;
}

int orc_wino_gemm(const orc_conv_params *p, const uint8_t *tinput, const int8_t *twq, const float *tscale,
                  const float *tshift, float *toutput, int32_t *acc_out)
{
  const WinoGeom g = wino_geom(p);
  const int OCp = g.OC2 * 16, ICp = g.IC2 * 16;
  const bool vnni = cpu_has_vnni();
#pragma omp parallel for collapse(2) schedule(static)
  for (int a = 0; a < g.A * g.A; ++a)
    for (int o2 = 0; o2 < g.OC2; ++o2) {
      // [ic/4][16 oc][4 ic]
      std::vector<int8_t> wt((size_t)ICp * 16);
      for (int v = 0; v < 16; ++v)
        for (int ic = 0; ic < ICp; ++ic)
          wt[(size_t)(ic / 4) * 64 + v * 4 + ic % 4] = twq[((size_t)a * OCp + o2 * 16 + v) * ICp + ic];
      for (int t = 0; t < g.t; ++t) {
        int32_t acc[16] = {0};
        for (int c2 = 0; c2 < g.IC2; ++c2) {
          const uint8_t *x = tinput + (((size_t)a * g.IC2 + c2) * g.t + t) * 16;
#if defined(__x86_64__)
          if (vnni) dot_vnni(acc, x, &wt[(size_t)c2 * 256], 4);
          else
#endif
            dot_scalar(acc, x, &wt[(size_t)c2 * 256], 4);
        }
        const size_t oi = (((size_t)a * g.OC2 + o2) * g.t + t) * 16;
        for (int v = 0; v < 16; ++v) {
          if (acc_out) acc_out[oi + v] = acc[v];
          toutput[oi + v] = fmaf((float)acc[v], tscale[(size_t)a * OCp + o2 * 16 + v],
                                 tshift[(size_t)a * OCp + o2 * 16 + v]);
        }
      }
    }
  return 0;
}

// One output value after the tile transform: bias, [u8 / s8 output: * (1 / out_S) + ceil(out_z),
// one rounding], ReLU as max(., 0) only, then round-to-nearest-even and saturate
// (src/kernel/elk_conv_wino_4x4_3x3_output.hxx:94-111,159-195; src/elx_int8_conv_wino.cpp:272-276).
// The u8 conversion goes through an UNSIGNED 32-bit integer: anything below -0.5 becomes 0xffffffff
// and saturates to 255.  Returns the code for u8 / s8, the float through *f32_out.
int orc_wino_output_value(float y, int with_bias, float bias, int out_type, float out_scale, float out_z,
                          int with_relu, float *f32_out)
{
  return orc_wino_output_value_a(6, y, with_bias, bias, out_type, out_scale, out_z, with_relu, f32_out);
}

// The same for any tile size.  The F(2x2,3x3) kernel converts toward minus infinity in its u8 / s8
// store (src/kernel/elk_conv_wino_2x2_3x3_output.hxx:142-151), the others to nearest even
// (src/kernel/elk_conv_wino_3x3_3x3_output.hxx:74-86).
int orc_wino_output_value_a(int A, float y, int with_bias, float bias, int out_type, float out_scale, float out_z,
                            int with_relu, float *f32_out)
{
  return orc_wino_output_value_sum(A, y, with_bias, bias, out_type, out_scale, out_z, with_relu, 0, 0.0f, f32_out);
}

// ... and with the in-place sum (with_ip_sum): the old output -- an f32, or the u8 / s8 code as a float,
// no scale -- is added after the output quantization and before the ReLU
// (src/kernel/elk_conv_wino_4x4_3x3_output.hxx:168-187)
int orc_wino_output_value_sum(int A, float y, int with_bias, float bias, int out_type, float out_scale, float out_z,
                              int with_relu, int with_sum, float old, float *f32_out)
{
  float r = y;
  if (with_bias) r += bias;
  if (out_type == ORC_U8 || out_type == ORC_S8) r = fmaf(r, 1.0f / out_scale, std::ceil(out_z));
  if (with_sum) r += old;
  if (with_relu) r = r > 0.0f ? r : 0.0f;  // vmaxps(p, 0): no upper bound here
  if (f32_out) *f32_out = r;
  if (out_type == ORC_U8) return usat8(A == 4 ? cvt_u32_floor(r) : cvt_u32_rne(r));
  if (out_type == ORC_S8) return ssat8(A == 4 ? cvt_s32_floor(r) : cvt_s32_rne(r));
  return 0;
}

// output: f32, u8 or s8 nChw16c according to p->out_type
int orc_wino_trans_output(const orc_conv_params *p, const float *toutput, const float *bias, void *output)
{
  const WinoGeom g = wino_geom(p);
#pragma omp parallel for collapse(2)
  for (int n = 0; n < p->n; ++n)
    for (int o2 = 0; o2 < g.OC2; ++o2)
      for (int th = 0; th < g.ht; ++th)
        for (int tw = 0; tw < g.wt; ++tw) {
          const size_t t = (size_t)n * g.nt + (size_t)th * g.wt + tw;
          for (int v = 0; v < 16; ++v) {
            float m[36], y[16];
            for (int a = 0; a < g.A * g.A; ++a) m[a] = toutput[(((size_t)a * g.OC2 + o2) * g.t + t) * 16 + v];
            orc_wino_tile_output_a(g.A, m, y);
            for (int i = 0; i < g.M; ++i)
              for (int j = 0; j < g.M; ++j) {
                int oh = g.M * th + i, ow = g.M * tw + j;
                if (oh >= p->oh || ow >= p->ow) continue;
                float r;
                const size_t oi = ((((size_t)n * g.OC2 + o2) * p->oh + oh) * p->ow + ow) * 16 + v;
                float old = 0.0f;
                if (p->with_sum)
                  old = p->out_type == ORC_U8 ? (float)((uint8_t *)output)[oi]
                      : (p->out_type == ORC_S8 ? (float)((int8_t *)output)[oi] : ((float *)output)[oi]);
                const int q = orc_wino_output_value_sum(g.A, y[g.M * i + j], p->with_bias,
                                                        p->with_bias ? bias[o2 * 16 + v] : 0.0f, p->out_type,
                                                        p->out_scale, p->out_z, p->with_relu, p->with_sum, old, &r);
                if (p->out_type == ORC_U8) ((uint8_t *)output)[oi] = (uint8_t)q;
                else if (p->out_type == ORC_S8) ((int8_t *)output)[oi] = (int8_t)q;
                else ((float *)output)[oi] = r;
              }
          }
        }
  return 0;
}

} // extern "C"
