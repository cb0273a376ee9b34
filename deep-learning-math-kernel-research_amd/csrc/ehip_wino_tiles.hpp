// Winograd tile transforms for the three tile sizes of the reference's int8 executor
// (src/eld_conv.cpp:257-270): A = 6 F(4x4,3x3), A = 4 F(2x2,3x3), A = 5 F(3x3,3x3).
// The float arithmetic follows the reference's COMPILED kernels operation for operation: which
// multiply-adds are one rounding is spelled out with __builtin_fmaf, and the sources that include
// this header are compiled with -ffp-contract=off.  Arrays are [A][A] row-major (row = h).
#ifndef EHIP_WINO_TILES_HPP
#define EHIP_WINO_TILES_HPP

namespace ehip {
namespace wino {

// ---- A = 6: src/kernel/elk_conv_wino_4x4_3x3_{input,weights,output}.hxx --------------------------
// Tiles that touch the zero frame go through the reference's "border" kernel, whose compiled form
// rounds the products of raw inputs in the column pass (and one product of the last row pass)
// separately.
__device__ __forceinline__ void in6_1d(const float f[6], float o[6], bool raw_unfused, bool t4_unfused)
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
    t0 = __builtin_fmaf(f[2], z0, f[4]);
    t1 = __builtin_fmaf(f[1], z0, f[3]);
    t2 = __builtin_fmaf(f[2], z1, f[4]);
    t3 = __builtin_fmaf(f[1], z1, f[3]);
    t4 = t4_unfused ? f[0] * z2 + f[4] : __builtin_fmaf(f[0], z2, f[4]);
    t5 = __builtin_fmaf(f[1], z2, f[5]);
    o[0] = __builtin_fmaf(f[2], z3, t4);
    o[5] = __builtin_fmaf(f[3], z3, t5);
  }
  o[1] = __builtin_fmaf(t1, z4, t0);
  o[2] = __builtin_fmaf(-t1, z4, t0);
  o[3] = __builtin_fmaf(t3, z5, t2);
  o[4] = __builtin_fmaf(-t3, z5, t2);
}
// The same with the choice made per LANE and without a branch, for waves that hold tiles of both kinds:
// fma(p, 1, g) with p = f * z already rounded IS the rounded sum p + g, so a term is
// fma(unfused ? p : f, unfused ? 1 : z, g) -- one multiply and one select more than the plain form
// instead of running the whole transform twice under complementary masks.
__device__ __forceinline__ float fma_or_mul_add(float f, float z, float g, bool unfused)
{
  const float p = f * z;
  return __builtin_fmaf(unfused ? p : f, unfused ? 1.0f : z, g);
}
__device__ __forceinline__ void in6_1d_lanes(const float f[6], float o[6], bool raw_unfused, bool t4_unfused)
{
  const float z0 = -2.25f, z1 = -0.390625f, z2 = 0.87890625f, z3 = -2.640625f, z4 = 0.625f, z5 = 1.5f;
  const float t0 = fma_or_mul_add(f[2], z0, f[4], raw_unfused);
  const float t1 = fma_or_mul_add(f[1], z0, f[3], raw_unfused);
  const float t2 = fma_or_mul_add(f[2], z1, f[4], raw_unfused);
  const float t3 = fma_or_mul_add(f[1], z1, f[3], raw_unfused);
  const float t4 = fma_or_mul_add(f[0], z2, f[4], raw_unfused || t4_unfused);
  const float t5 = fma_or_mul_add(f[1], z2, f[5], raw_unfused);
  o[0] = fma_or_mul_add(f[2], z3, t4, raw_unfused);
  o[5] = fma_or_mul_add(f[3], z3, t5, raw_unfused);
  o[1] = __builtin_fmaf(t1, z4, t0);
  o[2] = __builtin_fmaf(-t1, z4, t0);
  o[3] = __builtin_fmaf(t3, z5, t2);
  o[4] = __builtin_fmaf(-t3, z5, t2);
}
__device__ __forceinline__ void out6_1d(const float f[6], float o[4])
{
  const float z0 = 1.5f, z1 = 2.25f, z2 = 3.375f, z3 = 0.625f, z4 = 0.390625f, z5 = 0.244140625f;
  const float t0 = f[1] + f[2];
  const float t1 = f[3] + f[4];
  const float t2 = f[1] - f[2];
  const float t3 = f[3] - f[4];
  o[0] = t0 + t1 + f[0];
  o[1] = __builtin_fmaf(t2, z3, t3 * z0);
  o[2] = __builtin_fmaf(t0, z4, t1 * z1);
  o[3] = __builtin_fmaf(t2, z5, t3 * z2) + f[5];
}
// z0*f2 feeds two adds and fuses into both, z1*f0 and z2*f0 are rounded products
__device__ __forceinline__ void w6_1d(float f0, float f1, float f2, float o[6])
{
  const float z0 = 0.26890756302521f, z1 = -0.688403361344538f, z2 = 0.119514472455649f,
              z3 = 1.13777777777778f, z4 = 0.430252100840336f, z5 = 0.179271708683473f;
  const float pq = z1 * f0;
  const float qq = z2 * f0;
  const float t1 = __builtin_fmaf(-z0, f2, pq);
  const float t2 = __builtin_fmaf(z0, f2, qq);
  o[0] = z3 * f0;
  o[1] = __builtin_fmaf(-z4, f1, t1);
  o[2] = __builtin_fmaf(z4, f1, t1);
  o[3] = __builtin_fmaf(z5, f1, t2);
  o[4] = __builtin_fmaf(-z5, f1, t2);
  o[5] = f2;
}

// ---- A = 5: src/kernel/elk_conv_wino_3x3_3x3_{input,weights,output}.hxx --------------------------
// Products with 0.5 and 2 are exact; f2 * 1.5 + f3 is one rounding except in the column pass of the
// border kernel (`fuse15` false); in the output stage f2 / 3 fuses into both of its uses and every
// other product into the addition behind it.
__device__ __forceinline__ void in5_1d(const float f[5], float o[5], bool fuse15)
{
  const float z0 = 0.5f, z1 = 1.5f;
  const float t0 = f[1] * z0;
  const float t1 = f[2] * z0;
  const float t2 = f[3] - f[1];
  o[0] = f[0] * z0 - t1 - t2;
  o[1] = f[3] - t0 - t1;
  o[2] = (fuse15 ? __builtin_fmaf(f[2], z1, f[3]) : f[2] * z1 + f[3]) + t0;
  o[3] = t2;
  o[4] = f[3] * z0 + f[4] - f[2] - t0;
}
__device__ __forceinline__ void in5_1d_lanes(const float f[5], float o[5], bool unfused15)
{
  const float z0 = 0.5f, z1 = 1.5f;
  const float t0 = f[1] * z0;
  const float t1 = f[2] * z0;
  const float t2 = f[3] - f[1];
  o[0] = f[0] * z0 - t1 - t2;
  o[1] = f[3] - t0 - t1;
  o[2] = fma_or_mul_add(f[2], z1, f[3], unfused15) + t0;
  o[3] = t2;
  o[4] = f[3] * z0 + f[4] - f[2] - t0;
}
__device__ __forceinline__ void w5_1d(float f0, float f1, float f2, float o[5])
{
  const float t0 = f0 * 2.0f;
  const float t1 = f0 + f2;
  o[0] = t0;
  o[1] = f1 - t1;
  o[2] = f1 + t1;
  o[3] = f2 * 0.5f + t0 - f1;
  o[4] = f2;
}
__device__ __forceinline__ void out5_1d(const float f[5], float o[3])
{
  const float z0 = 0.3333333333333333f, z1 = 0.6666666666666666f, z2 = 1.3333333333333333f;
  const float t1 = __builtin_fmaf(f[2], z0, f[1]);
  o[0] = __builtin_fmaf(f[3], z2, f[0]) + t1;
  o[1] = __builtin_fmaf(-f[3], z1, __builtin_fmaf(f[2], z0, -f[1]));
  o[2] = __builtin_fmaf(f[3], z0, f[4]) + t1;
}

// ---- any A ------------------------------------------------------------------------------------------
template <int A>
__device__ __forceinline__ void tile_input(const float *d, float *v, bool border);
template <>
__device__ __forceinline__ void tile_input<6>(const float *d, float *v, bool border)
{
  float m[36];
#pragma unroll
  for (int j = 0; j < 6; ++j) {
    float f[6], o[6];
#pragma unroll
    for (int i = 0; i < 6; ++i) f[i] = d[6 * i + j];
    in6_1d(f, o, border, false);
#pragma unroll
    for (int i = 0; i < 6; ++i) m[6 * i + j] = o[i];
  }
#pragma unroll
  for (int i = 0; i < 6; ++i) in6_1d(&m[6 * i], &v[6 * i], false, border && i == 5);
}
template <>
__device__ __forceinline__ void tile_input<5>(const float *d, float *v, bool border)
{
  float m[25];
#pragma unroll
  for (int j = 0; j < 5; ++j) {
    float f[5], o[5];
#pragma unroll
    for (int i = 0; i < 5; ++i) f[i] = d[5 * i + j];
    in5_1d(f, o, !border);
#pragma unroll
    for (int i = 0; i < 5; ++i) m[5 * i + j] = o[i];
  }
#pragma unroll
  for (int i = 0; i < 5; ++i) in5_1d(&m[5 * i], &v[5 * i], true);
}
// A = 4 (src/kernel/elk_conv_wino_2x2_3x3_input.hxx:104-150): additions only, written out in two
// dimensions with the reference's association order
template <>
__device__ __forceinline__ void tile_input<4>(const float *d, float *v, bool)
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

// tile_input with the border flag per lane (see fma_or_mul_add): what a wave with both kinds of tile runs
template <int A>
__device__ __forceinline__ void tile_input_lanes(const float *d, float *v, bool border);
template <>
__device__ __forceinline__ void tile_input_lanes<6>(const float *d, float *v, bool border)
{
  float m[36];
#pragma unroll
  for (int j = 0; j < 6; ++j) {
    float f[6], o[6];
#pragma unroll
    for (int i = 0; i < 6; ++i) f[i] = d[6 * i + j];
    in6_1d_lanes(f, o, border, false);
#pragma unroll
    for (int i = 0; i < 6; ++i) m[6 * i + j] = o[i];
  }
#pragma unroll
  for (int i = 0; i < 5; ++i) in6_1d(&m[6 * i], &v[6 * i], false, false);
  in6_1d_lanes(&m[30], &v[30], false, border);
}
template <>
__device__ __forceinline__ void tile_input_lanes<5>(const float *d, float *v, bool border)
{
  float m[25];
#pragma unroll
  for (int j = 0; j < 5; ++j) {
    float f[5], o[5];
#pragma unroll
    for (int i = 0; i < 5; ++i) f[i] = d[5 * i + j];
    in5_1d_lanes(f, o, border);
#pragma unroll
    for (int i = 0; i < 5; ++i) m[5 * i + j] = o[i];
  }
#pragma unroll
  for (int i = 0; i < 5; ++i) in5_1d(&m[5 * i], &v[5 * i], true);
}
template <>
__device__ __forceinline__ void tile_input_lanes<4>(const float *d, float *v, bool border)
{
  tile_input<4>(d, v, border);
}

// g: [3][3] (kh, kw)
template <int A>
__device__ __forceinline__ void tile_weights(const float g[9], float *u);
template <>
__device__ __forceinline__ void tile_weights<6>(const float g[9], float *u)
{
  float M[6][3];
#pragma unroll
  for (int i = 0; i < 3; ++i) {
    float o[6];
    w6_1d(g[i], g[3 + i], g[6 + i], o);
#pragma unroll
    for (int k = 0; k < 6; ++k) M[k][i] = o[k];
  }
#pragma unroll
  for (int i = 0; i < 6; ++i) w6_1d(M[i][0], M[i][1], M[i][2], &u[6 * i]);
}
template <>
__device__ __forceinline__ void tile_weights<5>(const float g[9], float *u)
{
  float M[5][3];
#pragma unroll
  for (int i = 0; i < 3; ++i) {
    float o[5];
    w5_1d(g[i], g[3 + i], g[6 + i], o);
#pragma unroll
    for (int k = 0; k < 5; ++k) M[k][i] = o[k];
  }
#pragma unroll
  for (int i = 0; i < 5; ++i) w5_1d(M[i][0], M[i][1], M[i][2], &u[5 * i]);
}
// src/kernel/elk_conv_wino_2x2_3x3_weights.hxx:72-107
template <>
__device__ __forceinline__ void tile_weights<4>(const float g[9], float *u)
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

// m: [A][A], y: [A - 2][A - 2]
template <int A>
__device__ __forceinline__ void tile_output(const float *m, float *y);
template <>
__device__ __forceinline__ void tile_output<6>(const float *m, float *y)
{
  float M[4][6];
#pragma unroll
  for (int i = 0; i < 6; ++i) {
    float f[6], o[4];
#pragma unroll
    for (int r = 0; r < 6; ++r) f[r] = m[6 * r + i];
    out6_1d(f, o);
#pragma unroll
    for (int r = 0; r < 4; ++r) M[r][i] = o[r];
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) out6_1d(M[i], &y[4 * i]);
}
template <>
__device__ __forceinline__ void tile_output<5>(const float *m, float *y)
{
  float M[3][5];
#pragma unroll
  for (int i = 0; i < 5; ++i) {
    float f[5], o[3];
#pragma unroll
    for (int r = 0; r < 5; ++r) f[r] = m[5 * r + i];
    out5_1d(f, o);
#pragma unroll
    for (int r = 0; r < 3; ++r) M[r][i] = o[r];
  }
#pragma unroll
  for (int i = 0; i < 3; ++i) out5_1d(M[i], &y[3 * i]);
}
// src/kernel/elk_conv_wino_2x2_3x3_output.hxx:76-95
template <>
__device__ __forceinline__ void tile_output<4>(const float *m, float *y)
{
#define T(i, j) m[4 * (i) + (j)]
  const float c0 = T(1, 0) + T(1, 1) + T(1, 2);
  const float c1 = T(2, 0) + T(2, 1) + T(2, 2);
  const float c2 = T(1, 2) + T(1, 3) - T(1, 1);
  const float c3 = T(2, 2) + T(2, 3) - T(2, 1);
  y[0] = T(0, 0) + T(0, 1) + T(0, 2) + c0 + c1;
  y[2] = c1 - c0 + T(3, 0) + T(3, 1) + T(3, 2);
  y[1] = T(0, 2) - T(0, 1) + T(0, 3) + c2 + c3;
  y[3] = c3 - c2 - T(3, 1) + T(3, 2) + T(3, 3);
#undef T
}

}  // namespace wino
}  // namespace ehip
#endif
