// One-time weight preparation on the device (the reference's "first run" work), the fp32 -> u8
// activation quantizer and the layout reorders.
//
//   direct 1x1 / KxK : src/elx_int8_conv_direct_1x1.cpp:234-355, src/elx_int8_conv_direct.cpp:311-500
//   depthwise        : src/elx_int8_conv_direct_depthwise.cpp:200-292
//   Winograd         : src/kernel/elk_conv_wino_4x4_3x3_weights.hxx:18-72,
//                      src/elx_conv_wino_trans_weights.cpp:437-535
//   input quantizer  : tests/elt_conv_utils.cpp:354-401
//   reorders         : src/elx_reorder.cpp:35-93
//
// Arithmetic order is the reference's: q = rint((w * 127) / absmax) with a rounded product and a
// correctly rounded division; scale = in_S * (absmax / 127) [* 1/out_S]; shift folds bias, zero
// points and the sum operand's zero point with the single-rounding multiply-adds of the
// reference's compiled code.  Packed weights are laid out [tap][unit][oc][16 ic] so that one lane
// of an MFMA A-operand is 16 contiguous bytes and a wave's operand load is one contiguous KiB.
#include "ehip_internal.hpp"
#include "ehip_wino_tiles.hpp"

namespace ehip {

namespace {

__device__ __forceinline__ int quant_w(float w, float absmax)
{
  if (absmax == 0.0f) return 0;
  float t = w * 127.0f;
  t = __fdiv_rn(t, absmax);
  return (int)__builtin_rintf(t);
}

struct FoldParams {
  float in_S, in_z, out_repS, out_z, sum_S, sum_z;
  int f32_out, with_sum, with_bias;
};

__device__ __forceinline__ void fold(const FoldParams &p, float absmax, float wsum, float bias, float *scale,
                                     float *shift)
{
  const float w_S = __fdiv_rn(absmax, 127.0f);
  float s, z;
  if (p.f32_out) {
    s = p.in_S * w_S;
    z = __builtin_fmaf(-(p.in_z * wsum), s, bias);
  } else {
    s = p.in_S * w_S * p.out_repS;
    z = __builtin_fmaf(-(p.in_z * wsum), s, __builtin_fmaf(bias, p.out_repS, p.out_z));
  }
  // sum_z * sum_S is a product of two scalars that the reference's compiled code rounds on its own and
  // then subtracts (src/elx_int8_conv_direct_1x1.cpp:349-353: vmulss, broadcast, vsubps) -- two roundings
  if (p.with_sum) z = z - p.sum_z * p.sum_S;
  *scale = s;
  *shift = z;
}

FoldParams make_fold(const ehip_conv_desc_t &d, bool allow_sum)
{
  FoldParams p;
  p.in_S = d.input_scale;
  p.in_z = d.input_z;
  p.out_repS = 1.0f / d.output_scale;
  p.out_z = d.output_z;
  p.sum_S = d.sum_scale;
  p.sum_z = d.sum_z;
  p.f32_out = d.output_type == EHIP_F32 || d.output_type == EHIP_S32;
  p.with_sum = allow_sum && d.with_ip_sum;
  p.with_bias = d.with_bias;
  return p;
}

// one block per 16-wide oc block; w is OIhw16i16o f32: [o2][i2][tap][16 i][16 o]
__global__ __launch_bounds__(kBlock) void k_absmax_direct(const float *w, int i2n, int taps, float *absmax)
{
  __shared__ float red[16][16];
  const int o2 = blockIdx.x, ov = threadIdx.x & 15, r = threadIdx.x >> 4;
  const float *base = w + (size_t)o2 * i2n * taps * 256;
  const int rows = i2n * taps * 16;
  float m = 0.0f;
  for (int e = r; e < rows; e += 16) {
    const float v = __builtin_fabsf(base[(size_t)e * 16 + ov]);
    m = v > m ? v : m;
  }
  red[r][ov] = m;
  __syncthreads();
  if (r == 0) {
#pragma unroll
    for (int k = 1; k < 16; ++k) m = red[k][ov] > m ? red[k][ov] : m;
    absmax[o2 * 16 + ov] = m;
  }
}

// one thread per packed dword: (tap, unit, oc row, quad of 4 ic)
__global__ __launch_bounds__(kBlock) void k_quant_pack_direct(const float *w, const float *absmax, int oc2n,
                                                              int i2n, int ic_real, int taps, int units_pad,
                                                              int ocpp, unsigned *wpacked)
{
  const long long total = (long long)taps * units_pad * ocpp * 4;
  const long long idx = (long long)blockIdx.x * kBlock + threadIdx.x;
  if (idx >= total) return;
  const int q = (int)(idx & 3);
  long long rest = idx >> 2;
  const int oc = oc_of_packed_row((int)(rest % ocpp));   // the channel this packed row holds
  rest /= ocpp;
  const int u = (int)(rest % units_pad);
  const int tap = (int)(rest / units_pad);
  unsigned packed = 0u;
  if (u < i2n && oc < oc2n * 16) {
    const float am = absmax[oc];
    const float *src = w + (((size_t)(oc >> 4) * i2n + u) * taps + tap) * 256 + (oc & 15);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int iv = 4 * q + k;
      int v = 0;
      if (u * 16 + iv < ic_real) v = quant_w(src[iv * 16], am);
      packed |= ((unsigned)v & 0xffu) << (8 * k);
    }
  }
  wpacked[idx] = packed;
}

// Layers with at most four input channels (first layers, k_conv_fewch_u8s8): a 16-byte cell
// holds ppc = 16 / icl horizontally adjacent pixels of icl bytes each (icl = ic, or 4 for three channels: see
// conv_fewch_icl), so one kernel row is nu = ceil(kw / ppc) cells instead of kw.  Packed weights:
// [kh * nu + j][OCpp rows][16], byte b of unit j = tap kw = j * ppc + b / icl, channel b % icl (zero where
// kw >= KW, b >= ppc * icl or the channel is the pad byte).  One thread per packed dword.
__global__ __launch_bounds__(kBlock) void k_quant_pack_direct_px(const float *w, const float *absmax, int oc2n,
                                                                 int ic, int icl, int KH, int KW, int ppc, int nu,
                                                                 int ocpp, unsigned *wpacked)
{
  const long long total = (long long)KH * nu * ocpp * 4;
  const long long idx = (long long)blockIdx.x * kBlock + threadIdx.x;
  if (idx >= total) return;
  const int q = (int)(idx & 3);
  long long rest = idx >> 2;
  const int oc = oc_of_packed_row((int)(rest % ocpp));
  const int t = (int)(rest / ocpp);
  const int kh = t / nu, j = t - kh * nu;
  unsigned packed = 0u;
  if (oc < oc2n * 16) {
    const float am = absmax[oc];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int b = 4 * q + k;
      const int jj = b / icl, c = b - jj * icl, kw = j * ppc + jj;
      int v = 0;
      if (jj < ppc && kw < KW && c < ic) v = quant_w(w[((size_t)(oc >> 4) * KH * KW + kh * KW + kw) * 256 + c * 16 + (oc & 15)], am);
      packed |= ((unsigned)v & 0xffu) << (8 * k);
    }
  }
  wpacked[idx] = packed;
}

// pixel-packed counterpart of k_fold_direct_border: one thread per (class, channel); ic = bytes per pixel of a
// cell (pad bytes hold zero weights)
__global__ __launch_bounds__(kBlock) void k_fold_direct_border_px(const unsigned *wpacked, const float *absmax,
                                                                  const float *bias, int oc_rows, int ic, int ppc,
                                                                  int nu, int ocpp, FoldParams p, const int4 *rects,
                                                                  int nclass, float *shift_tab)
{
  const int idx = blockIdx.x * kBlock + threadIdx.x;
  if (idx >= nclass * ocpp) return;
  const int c = idx / ocpp, oc = idx - c * ocpp;
  float sh = 0.0f;
  if (oc < oc_rows) {
    const int4 r = rects[c];
    int s = 0;
    for (int kh = r.x; kh <= r.y; ++kh)
      for (int j = 0; j < nu; ++j) {
        const uint4 cell = *reinterpret_cast<const uint4 *>(wpacked + ((size_t)(kh * nu + j) * ocpp + packed_row_of_oc(oc)) * 4);
        const unsigned d[4] = {cell.x, cell.y, cell.z, cell.w};
        for (int b = 0; b < ppc * ic; ++b) {
          const int kw = j * ppc + b / ic;
          if (kw >= r.z && kw <= r.w) s += (int)(signed char)((d[b >> 2] >> (8 * (b & 3))) & 0xffu);
        }
      }
    float sc;
    fold(p, absmax[oc], (float)s, p.with_bias ? bias[oc] : 0.0f, &sc, &sh);
  }
  shift_tab[idx] = sh;
}

// one thread per oc row: sum of the packed weights, compensation, scale/shift
__global__ __launch_bounds__(kBlock) void k_fold_direct(const unsigned *wpacked, const float *absmax,
                                                        const float *bias, int oc_rows, int taps, int units_pad,
                                                        int ocpp, FoldParams p, float *scale, float *shift,
                                                        int *wsum, int *comp)
{
  const int oc = blockIdx.x * kBlock + threadIdx.x;
  if (oc >= ocpp) return;
  int s = 0;
  if (oc < oc_rows) {
    for (int tu = 0; tu < taps * units_pad; ++tu) {
      const uint4 c = *reinterpret_cast<const uint4 *>(wpacked + ((size_t)tu * ocpp + packed_row_of_oc(oc)) * 4);
      const unsigned d[4] = {c.x, c.y, c.z, c.w};
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int k = 0; k < 4; ++k) s += (int)(signed char)((d[j] >> (8 * k)) & 0xffu);
    }
  }
  wsum[oc] = s;
  comp[oc] = 128 * s;
  float sc = 0.0f, sh = 0.0f;
  if (oc < oc_rows) fold(p, absmax[oc], (float)s, p.with_bias ? bias[oc] : 0.0f, &sc, &sh);
  scale[oc] = sc;
  shift[oc] = sh;
}

// Shift rows for a non-zero input zero point with padding (src/elx_int8_conv_direct.cpp:311-423):
// class c covers the output pixels whose valid taps are the rectangle rects[c] = {kh_lo, kh_hi,
// kw_lo, kw_hi} (inclusive); its shift folds the sum of the weights of those taps only.
// One thread per (class, channel).
__global__ __launch_bounds__(kBlock) void k_fold_direct_border(const unsigned *wpacked, const float *absmax,
                                                               const float *bias, int oc_rows, int kw, int units_pad,
                                                               int ocpp, FoldParams p, const int4 *rects, int nclass,
                                                               float *shift_tab)
{
  const int idx = blockIdx.x * kBlock + threadIdx.x;
  if (idx >= nclass * ocpp) return;
  const int c = idx / ocpp, oc = idx - c * ocpp;
  float sh = 0.0f;
  if (oc < oc_rows) {
    const int4 r = rects[c];
    int s = 0;
    for (int kh = r.x; kh <= r.y; ++kh)
      for (int kwi = r.z; kwi <= r.w; ++kwi)
        for (int u = 0; u < units_pad; ++u) {
          const size_t tu = (size_t)(kh * kw + kwi) * units_pad + u;
          const uint4 cell = *reinterpret_cast<const uint4 *>(wpacked + (tu * ocpp + packed_row_of_oc(oc)) * 4);
          const unsigned d[4] = {cell.x, cell.y, cell.z, cell.w};
#pragma unroll
          for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int k = 0; k < 4; ++k) s += (int)(signed char)((d[j] >> (8 * k)) & 0xffu);
        }
    float sc;
    fold(p, absmax[oc], (float)s, p.with_bias ? bias[oc] : 0.0f, &sc, &sh);
  }
  shift_tab[idx] = sh;
}

// depthwise: one thread per channel; w is goihw f32 [g][3][3]; packed [g2][kh][16][kw0 kw1 kw2 0]
__global__ __launch_bounds__(kBlock) void k_prepare_depthwise(const float *w, const float *bias, int g, int G,
                                                              FoldParams p, int8_t *wpacked, float *scale,
                                                              float *shift, int *wsum)
{
  const int c = blockIdx.x * kBlock + threadIdx.x;
  if (c >= G) return;
  float am = 0.0f;
  if (c < g)
    for (int k = 0; k < 9; ++k) {
      const float v = __builtin_fabsf(w[(size_t)c * 9 + k]);
      am = v > am ? v : am;
    }
  int s = 0;
  for (int k = 0; k < 9; ++k) {
    const int q = c < g ? quant_w(w[(size_t)c * 9 + k], am) : 0;
    wpacked[(((size_t)(c >> 4) * 3 + k / 3) * 16 + (c & 15)) * 4 + k % 3] = (int8_t)q;
    s += q;
  }
  for (int kh = 0; kh < 3; ++kh) wpacked[(((size_t)(c >> 4) * 3 + kh) * 16 + (c & 15)) * 4 + 3] = 0;
  wsum[c] = s;
  float sc = 0.0f, sh = 0.0f;
  if (c < g) fold(p, am, (float)s, p.with_bias ? bias[c] : 0.0f, &sc, &sh);
  scale[c] = sc;
  shift[c] = sh;
}

// ---- Winograd weights --------------------------------------------------------------------------
// U = G g Gt (tile arithmetic in ehip_wino_tiles.hpp); one thread per (oc, ic): U[pos][oc][ic] f32
template <int A>
__global__ __launch_bounds__(kBlock) void k_wino_weights_u(const float *w, int ocp, int icp, float *U)
{
  const long long idx = (long long)blockIdx.x * kBlock + threadIdx.x;
  if (idx >= (long long)ocp * icp) return;
  const int oc = (int)(idx % ocp), ic = (int)(idx / ocp);  // oc fastest: coalesced reads of the 16o axis
  const float *src = w + (((size_t)(oc >> 4) * (icp >> 4) + (ic >> 4)) * 9) * 256 + (ic & 15) * 16 + (oc & 15);
  float g[9];
#pragma unroll
  for (int k = 0; k < 9; ++k) g[k] = src[(size_t)k * 256];
  float u[A * A];
  wino::tile_weights<A>(g, u);
#pragma unroll
  for (int e = 0; e < A * A; ++e) U[((size_t)e * ocp + oc) * icp + ic] = u[e];
}

// one thread per (pos, oc): abs-max over ic, quantize, pack, fold
__global__ __launch_bounds__(kBlock) void k_wino_quant(const float *U, int npos, int ocp, int icp, int units_pad, int ocpp,
                                                       float tin_S, float tin_z, int8_t *wpacked, float *scale,
                                                       float *shift, int *wsum, int *comp)
{
  const int idx = blockIdx.x * kBlock + threadIdx.x;
  if (idx >= npos * ocp) return;
  const int pos = idx / ocp, oc = idx - pos * ocp;
  const float *u = U + ((size_t)pos * ocp + oc) * icp;
  float am = 0.0f;
  for (int ic = 0; ic < icp; ++ic) {
    const float v = __builtin_fabsf(u[ic]);
    am = v > am ? v : am;
  }
  int s = 0;
  for (int ic = 0; ic < icp; ++ic) {
    const int q = quant_w(u[ic], am);
    wpacked[(((size_t)pos * units_pad + (ic >> 4)) * ocpp + packed_row_of_oc(oc)) * 16 + (ic & 15)] = (int8_t)q;
    s += q;
  }
  // Sw = absmax / 127; Sw = Sw * tin_S; Zw = -acc * Sw * tin_z  (trans_weights.cpp:523-533)
  float Sw = __fdiv_rn(am, 127.0f);
  Sw = Sw * tin_S;
  const float Zw = -(float)s * Sw * tin_z;
  scale[(size_t)pos * ocpp + oc] = Sw;
  shift[(size_t)pos * ocpp + oc] = Zw;
  wsum[(size_t)pos * ocpp + oc] = s;
  comp[(size_t)pos * ocpp + oc] = 128 * s;
}

// ---- activation quantizer ----------------------------------------------------------------------
// The reference harness' helper truncates, then compares the fraction with 0.5 so that exact ties
// go to the odd neighbour, and narrows with a plain (uint8_t) cast.
__device__ __forceinline__ unsigned quant_in(float x, float scale, float z)
{
  const float f = __fdiv_rn(x, scale) + z;
  const int i = (int)f;
  int r;
  if (i >= 0) {
    if (i % 2) r = (f - (float)i <= 0.5f) ? i : i + 1;
    else r = (f - (float)i >= 0.5f) ? i + 1 : i;
  } else {
    if (i % 2) r = ((float)i - f <= 0.5f) ? i : i - 1;
    else r = ((float)i - f >= 0.5f) ? i - 1 : i;
  }
  return (unsigned)r & 0xffu;
}

__global__ __launch_bounds__(kBlock) void k_quantize_input_u8(unsigned *dst, const float4 *src, size_t quads,
                                                              const float *src_tail, uint8_t *dst_tail,
                                                              int tail, float scale, float z)
{
  const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
  if (i < quads) {
    const float4 v = src[i];
    dst[i] = quant_in(v.x, scale, z) | (quant_in(v.y, scale, z) << 8) | (quant_in(v.z, scale, z) << 16) |
        (quant_in(v.w, scale, z) << 24);
  }
  if (i < (size_t)tail) dst_tail[i] = (uint8_t)quant_in(src_tail[i], scale, z);
}

// ---- reorders -----------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(kBlock) void k_nchw_to_blocked(T *dst, const T *src, int n, int c, int h, int w)
{
  const int C2 = (c + 15) / 16;
  const size_t total = (size_t)n * C2 * h * w * 16;
  const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= total) return;
  const int v = (int)(i & 15);
  size_t r = i >> 4;
  const int _w = (int)(r % w); r /= w;
  const int _h = (int)(r % h); r /= h;
  const int _c = (int)(r % C2);
  const int _n = (int)(r / C2);
  const int ch = _c * 16 + v;
  dst[i] = ch < c ? src[(((size_t)_n * c + ch) * h + _h) * w + _w] : (T)0;
}

template <typename T>
__global__ __launch_bounds__(kBlock) void k_blocked_to_nchw(T *dst, const T *src, int n, int c, int h, int w)
{
  const int C2 = (c + 15) / 16;
  const size_t total = (size_t)n * c * h * w;
  const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= total) return;
  size_t r = i;
  const int _w = (int)(r % w); r /= w;
  const int _h = (int)(r % h); r /= h;
  const int ch = (int)(r % c);
  const int _n = (int)(r / c);
  dst[i] = src[((((size_t)_n * C2 + ch / 16) * h + _h) * w + _w) * 16 + ch % 16];
}

__global__ __launch_bounds__(kBlock) void k_oihw_to_blocked(float *dst, const float *src, int o, int i, int h, int w)
{
  const int O2 = (o + 15) / 16, I2 = (i + 15) / 16;
  const size_t total = (size_t)O2 * I2 * h * w * 256;
  const size_t idx = (size_t)blockIdx.x * kBlock + threadIdx.x;
  if (idx >= total) return;
  const int ov = (int)(idx & 15), iv = (int)((idx >> 4) & 15);
  size_t r = idx >> 8;
  const int _w = (int)(r % w); r /= w;
  const int _h = (int)(r % h); r /= h;
  const int _i = (int)(r % I2);
  const int _o = (int)(r / I2);
  const int oc = _o * 16 + ov, ic = _i * 16 + iv;
  dst[idx] = (oc < o && ic < i) ? src[(((size_t)oc * i + ic) * h + _h) * w + _w] : 0.0f;
}

inline dim3 grid_for(size_t total) { return dim3((unsigned)((total + kBlock - 1) / kBlock)); }

}  // namespace

hipError_t launch_prepare_direct(const float *w, const float *bias, int oc, int ic, int kh, int kw, int units_pad,
                                 int ocpp, const ehip_conv_desc_t &d, float *absmax, int8_t *wpacked, float *scale,
                                 float *shift, int *wsum, int *comp, hipStream_t s)
{
  const int oc2 = up(oc, 16) / 16, i2 = up(ic, 16) / 16, taps = kh * kw;
  hipLaunchKernelGGL(k_absmax_direct, dim3(oc2), dim3(kBlock), 0, s, w, i2, taps, absmax);
  const size_t dwords = (size_t)taps * units_pad * ocpp * 4;
  hipLaunchKernelGGL(k_quant_pack_direct, grid_for(dwords), dim3(kBlock), 0, s, w, absmax, oc2, i2, ic, taps,
                     units_pad, ocpp, reinterpret_cast<unsigned *>(wpacked));
  const FoldParams fp = make_fold(d, d.algorithm == EHIP_CONV_DIRECT_1X1);
  hipLaunchKernelGGL(k_fold_direct, grid_for(ocpp), dim3(kBlock), 0, s, reinterpret_cast<const unsigned *>(wpacked),
                     absmax, bias, oc2 * 16, taps, units_pad, ocpp, fp, scale, shift, wsum, comp);
  return hipGetLastError();
}

// weight side of the pixel-packed form (see k_quant_pack_direct_px): taps = kh * nu units of one cell
hipError_t launch_prepare_direct_px(const float *w, const float *bias, int oc, int ic, int icl, int kh, int kw, int ppc, int nu,
                                    int ocpp, const ehip_conv_desc_t &d, float *absmax, int8_t *wpacked, float *scale,
                                    float *shift, int *wsum, int *comp, hipStream_t s)
{
  const int oc2 = up(oc, 16) / 16;
  hipLaunchKernelGGL(k_absmax_direct, dim3(oc2), dim3(kBlock), 0, s, w, 1, kh * kw, absmax);
  const size_t dwords = (size_t)kh * nu * ocpp * 4;
  hipLaunchKernelGGL(k_quant_pack_direct_px, grid_for(dwords), dim3(kBlock), 0, s, w, absmax, oc2, ic, icl, kh, kw, ppc,
                     nu, ocpp, reinterpret_cast<unsigned *>(wpacked));
  const FoldParams fp = make_fold(d, false);
  hipLaunchKernelGGL(k_fold_direct, grid_for(ocpp), dim3(kBlock), 0, s, reinterpret_cast<const unsigned *>(wpacked),
                     absmax, bias, oc2 * 16, kh * nu, 1, ocpp, fp, scale, shift, wsum, comp);
  return hipGetLastError();
}

hipError_t launch_fold_direct_border_px(const int8_t *wpacked, const float *absmax, const float *bias, int oc, int ic,
                                        int ppc, int nu, int ocpp, const ehip_conv_desc_t &d, const int *rects,
                                        int nclass, float *shift_tab, hipStream_t s)
{
  const FoldParams fp = make_fold(d, false);
  hipLaunchKernelGGL(k_fold_direct_border_px, grid_for((size_t)nclass * ocpp), dim3(kBlock), 0, s,
                     reinterpret_cast<const unsigned *>(wpacked), absmax, bias, up(oc, 16), ic, ppc, nu, ocpp, fp,
                     reinterpret_cast<const int4 *>(rects), nclass, shift_tab);
  return hipGetLastError();
}

hipError_t launch_fold_direct_border(const int8_t *wpacked, const float *absmax, const float *bias, int oc, int kw,
                                     int units_pad, int ocpp, const ehip_conv_desc_t &d, const int *rects, int nclass,
                                     float *shift_tab, hipStream_t s)
{
  const FoldParams fp = make_fold(d, d.with_ip_sum != 0 && d.algorithm == EHIP_CONV_DIRECT_1X1);
  hipLaunchKernelGGL(k_fold_direct_border, grid_for((size_t)nclass * ocpp), dim3(kBlock), 0, s,
                     reinterpret_cast<const unsigned *>(wpacked), absmax, bias, up(oc, 16), kw, units_pad, ocpp, fp,
                     reinterpret_cast<const int4 *>(rects), nclass, shift_tab);
  return hipGetLastError();
}

hipError_t launch_prepare_depthwise(const float *w, const float *bias, int g, const ehip_conv_desc_t &d,
                                    int8_t *wpacked, float *scale, float *shift, int *wsum, hipStream_t s)
{
  const int G = up(g, 16);
  const FoldParams fp = make_fold(d, false);
  hipLaunchKernelGGL(k_prepare_depthwise, grid_for(G), dim3(kBlock), 0, s, w, bias, g, G, fp, wpacked, scale, shift,
                     wsum);
  return hipGetLastError();
}

// tile: the Winograd tile size A (4, 5 or 6); u_tmp holds A * A * ocp * icp floats
hipError_t launch_prepare_wino(const float *w, int oc, int ic, int tile, int units_pad, int ocpp, const ehip_conv_desc_t &d,
                               float *u_tmp, int8_t *wpacked, float *scale, float *shift, int *wsum, int *comp,
                               hipStream_t s)
{
  const int ocp = up(oc, 16), icp = up(ic, 16);
  void (*kern)(const float *, int, int, float *) = tile == 4 ? k_wino_weights_u<4> : (tile == 5 ? k_wino_weights_u<5> : k_wino_weights_u<6>);
  const int npos = tile == 4 ? 16 : (tile == 5 ? 25 : 36);
  hipLaunchKernelGGL(kern, grid_for((size_t)ocp * icp), dim3(kBlock), 0, s, w, ocp, icp, u_tmp);
  hipLaunchKernelGGL(k_wino_quant, grid_for((size_t)npos * ocp), dim3(kBlock), 0, s, u_tmp, npos, ocp, icp, units_pad, ocpp,
                     d.tinput_scale, ceilf(d.tinput_z), wpacked, scale, shift, wsum, comp);
  return hipGetLastError();
}

hipError_t launch_quantize_input(uint8_t *dst, const float *src, size_t count, float scale, float z, hipStream_t s)
{
  const size_t quads = count / 4;
  const int tail = (int)(count - quads * 4);
  const size_t threads = quads > (size_t)tail ? quads : (size_t)tail;
  if (threads == 0) return hipSuccess;
  hipLaunchKernelGGL(k_quantize_input_u8, grid_for(threads), dim3(kBlock), 0, s, reinterpret_cast<unsigned *>(dst),
                     reinterpret_cast<const float4 *>(src), quads, src + quads * 4, dst + quads * 4, tail, scale, z);
  return hipGetLastError();
}

hipError_t launch_reorder_nchw_to_blocked(void *dst, const void *src, int es, int n, int c, int h, int w,
                                          hipStream_t s)
{
  const size_t total = (size_t)n * up(c, 16) * h * w;
  if (es == 4)
    hipLaunchKernelGGL(k_nchw_to_blocked<float>, grid_for(total), dim3(kBlock), 0, s, (float *)dst,
                       (const float *)src, n, c, h, w);
  else
    hipLaunchKernelGGL(k_nchw_to_blocked<uint8_t>, grid_for(total), dim3(kBlock), 0, s, (uint8_t *)dst,
                       (const uint8_t *)src, n, c, h, w);
  return hipGetLastError();
}

hipError_t launch_reorder_blocked_to_nchw(void *dst, const void *src, int es, int n, int c, int h, int w,
                                          hipStream_t s)
{
  const size_t total = (size_t)n * c * h * w;
  if (es == 4)
    hipLaunchKernelGGL(k_blocked_to_nchw<float>, grid_for(total), dim3(kBlock), 0, s, (float *)dst,
                       (const float *)src, n, c, h, w);
  else
    hipLaunchKernelGGL(k_blocked_to_nchw<uint8_t>, grid_for(total), dim3(kBlock), 0, s, (uint8_t *)dst,
                       (const uint8_t *)src, n, c, h, w);
  return hipGetLastError();
}

hipError_t launch_reorder_oihw_to_blocked(float *dst, const float *src, int o, int i, int h, int w, hipStream_t s)
{
  const size_t total = (size_t)up(o, 16) * up(i, 16) * h * w;
  hipLaunchKernelGGL(k_oihw_to_blocked, grid_for(total), dim3(kBlock), 0, s, dst, src, o, i, h, w);
  return hipGetLastError();
}

}  // namespace ehip
