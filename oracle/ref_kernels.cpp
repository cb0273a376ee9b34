// TEST INFRASTRUCTURE ONLY -- never linked into, imported by, or called from the product path.
//
// Thin C-ABI driver around the reference's own AVX-512 micro-kernel templates.  It is
// compiled (by oracle/Makefile, target `ref`) against the header files where they lie under
// /root/reference with the GNU flags of the reference's cmake/flags.cmake:77-87
// (-std=c++11 -O2 -DNDEBUG -mavx512f -mavx512dq -mavx512bw -mfma -mavx512vl, WITH_VNNI),
// so that the float glue of the reference (which a*b+c become one fused rounding, the
// floor/round-to-nearest split of the depthwise store, the unsigned saturation) is pinned by
// the reference's compiled code and not by a reading of it.  Nothing of the reference is
// copied: the templates are instantiated straight from
//   src/kernel/elk_u8s8_gemm.hxx, elk_u8s8_conv.hxx, elk_u8s8_depthwise_conv.hxx,
//   src/kernel/elk_conv_wino_{4x4,2x2,3x3}_3x3_{input,weights,output}.hxx.
// The executor classes (src/elx_int8_conv_*.cpp) are NOT built: they bind kernels through
// tables that the reference's build generates with shell scripts at configure time.
//
// The only accommodation: the reference uses the "aligned" 512-bit integer load/store
// intrinsics on addresses that are only 16-byte aligned (depthwise kernel); the intrinsic
// headers are included first and those two names are redirected to the unaligned forms.
// This changes no arithmetic.
#include <immintrin.h>
#include <x86intrin.h>
#define _mm512_load_epi32(p) _mm512_loadu_si512(p)
#define _mm512_store_epi32(p, v) _mm512_storeu_si512(p, v)

#include <cstdint>
#include <cstring>
#include <string>
#include <cfloat>

#include "euler.hpp"
#include "el_def.hpp"
#include "elk_def.hpp"
#include "elx_conv.hpp"
#include "elk_u8s8_gemm.hxx"
#include "elk_u8s8_conv.hxx"
#include "elk_u8s8_depthwise_conv.hxx"
#include "elk_conv_wino.hpp"
#include "elk_conv_wino_4x4_3x3_input.hxx"
#include "elk_conv_wino_4x4_3x3_weights.hxx"
#include "elk_conv_wino_4x4_3x3_output.hxx"
#include "elk_conv_wino_2x2_3x3_input.hxx"
#include "elk_conv_wino_2x2_3x3_weights.hxx"
#include "elk_conv_wino_2x2_3x3_output.hxx"
#include "elk_conv_wino_3x3_3x3_input.hxx"
#include "elk_conv_wino_3x3_3x3_weights.hxx"
#include "elk_conv_wino_3x3_3x3_output.hxx"

using namespace euler;

namespace {

void fill_common(elx_param_t &ep, float relu_lo, float relu_hi, float sum_S)
{
  ep.V1 = 4; ep.Vx = 4;
  ep.O = 1; ep.O1 = 1; ep.O2 = 1; ep.O3 = 1; ep.O4 = 1;
  ep.I2 = 1; ep.I3 = 1; ep.I4 = 1;
  ep.Ir = 4; ep.Or = 16;
  ep.hs = ep.ws = 1; ep.hd = ep.wd = 1;
  ep.lp = ep.rp = ep.tp = ep.bp = 0;
  ep.kh = ep.kw = 1;
  ep.g = 1; ep.G2 = 1; ep.G3 = 1;
  ep.streaming_input = ep.streaming_output = 0;
  ep.sampling_kind = CALIBRATED;
  ep.relu_bound_lower = relu_lo;
  ep.relu_bound_upper = relu_hi;
  ep.sum_quant_S = sum_S;
  for (int i = 0; i < 16; ++i) {
    ep.relu_bound_lower_vec[i] = relu_lo;
    ep.relu_bound_upper_vec[i] = relu_hi;
    ep.sum_quant_S_vec[i] = sum_S;
  }
}

template <typename OT, int O, int T>
void run_gemm_ccc(elx_param_t &ep, float *toutput, void *ooutput, uint8_t *input,
    int8_t *weights, int attr, float *wscale, float *wshift)
{
  using ker = u8s8_gemm_kernel<conv_impl::INT8_F32, OT, 16, 4, ISA_AVX512,
      estl::integer_sequence<1, GKF_CCC, O, T, 1>>;
  ker::gemm(ep, toutput, (OT *)ooutput, input, weights, nullptr, attr,
      nullptr, nullptr, wscale, wshift);
}

template <typename OT, int T, int S = 1>
void run_dw(elx_param_t &ep, void *routput, uint8_t *input, int8_t *weights,
    float *wscale, float *wshift, int khs, int khe, int pad_l, int pad_r, int attr)
{
  using ker = u8s8_depthwise_conv_kernel<conv_impl::INT8_F32, OT, 16, 4, ISA_AVX512,
      estl::integer_sequence<S, GKF_DCD, 1, T, 3>>;
  ker::conv(ep, nullptr, (OT *)routput, input, weights, nullptr, nullptr, nullptr,
      wscale, wshift, khs, khe, 0, 3, pad_l, pad_r, attr);
}

template <typename OT, int T, int S = 1, int K = 3>
void run_conv3(elx_param_t &ep, float *toutput, void *routput, uint8_t *input,
    int8_t *weights, float *wscale, float *wshift, int khs, int khe, int kws,
    int kwe, int pad_l, int pad_r, int attr)
{
  using ker = u8s8_conv_kernel<conv_impl::INT8_F32, OT, 16, 4, ISA_AVX512,
      estl::integer_sequence<S, GKF_DCD, 1, T, K>>;
  ker::conv(ep, toutput, (OT *)routput, input, weights, nullptr, nullptr, nullptr,
      wscale, wshift, khs, khe, kws, kwe, pad_l, pad_r, attr);
}

} // namespace

extern "C" {

// u8s8 GEMM micro-kernel, compact layout (GKF_CCC, src/kernel/elk_def.hpp:36-41):
//   input   [I2][T][16]  u8,   weights [I2][4][O][16 oc][4 ic] s8  (O1 = 1),
//   toutput [O][T][16]   f32-typed (holds s32 partials or the f32 result),
//   ooutput [O][T][16]   u8/s8 (out_kind 1/2; also the in-place sum operand).
// out_kind: 0 = f32, 1 = u8, 2 = s8.  (O,T) in {(1,4),(2,6)}.
int ref_u8s8_gemm(int out_kind, int O, int T, int I2, int attr, float relu_lo,
    float relu_hi, float sum_S, float *toutput, void *ooutput, uint8_t *input,
    int8_t *weights, float *wscale, float *wshift)
{
  elx_param_t ep;
  fill_common(ep, relu_lo, relu_hi, sum_S);
  ep.I2 = I2; ep.O = O; ep.O2 = O; ep.T = T;
  ep.IC = I2 * 16; ep.ic = ep.IC; ep.OC = O * 16; ep.oc = ep.OC;
  ep.ic2 = I2; ep.ic34 = 1;
  ep.oh = 1; ep.ow = T; ep.ih = 1; ep.iw = T;
#define GEMM_CASE(k, OT, o, t)                                                  \
  if (out_kind == k && O == o && T == t) {                                      \
    run_gemm_ccc<OT, o, t>(ep, toutput, ooutput, input, weights, attr, wscale,  \
        wshift);                                                                \
    return 0;                                                                   \
  }
  GEMM_CASE(0, float, 1, 4) GEMM_CASE(0, float, 2, 6)
  GEMM_CASE(1, uint8_t, 1, 4) GEMM_CASE(1, uint8_t, 2, 6)
  GEMM_CASE(2, int8_t, 1, 4) GEMM_CASE(2, int8_t, 2, 6)
#undef GEMM_CASE
  return -1;
}

// Depthwise 3x3 stride-1 micro-kernel (src/kernel/elk_u8s8_depthwise_conv.hxx:288-474) on
// one width block of T outputs of one output row, all G2 channel groups:
//   input   [G2][ih][iw][16] u8 (whole plane; the kernel is handed the pointer of the
//           block's first centre pixel, as conv_c160 does,
//           src/elx_int8_conv_direct_depthwise.cpp:294-319),
//   weights [G2][3][16][4] s8, wscale/wshift [G2][16], routput [G2][oh*ow][16].
// out_kind: 1 = u8, 2 = s8.  T is the layer's width-block size, Tz the size of THIS block
// (T, or ow % T for the last one); the kernel is instantiated for Tz in {4,5,6,7,8,11,14}.
int ref_u8s8_depthwise(int out_kind, int T, int Tz, int G2, int ih, int iw, int oh, int ow,
    int _ht, int _wt, int tp, int lp, int rp, int with_relu, float relu_lo,
    float relu_hi, void *routput, uint8_t *input, int8_t *weights, float *wscale,
    float *wshift)
{
  elx_param_t ep;
  fill_common(ep, relu_lo, relu_hi, 0.f);
  ep.kh = ep.kw = 3; ep.G2 = G2; ep.ic2 = G2; ep.oc2 = G2; ep.I2 = G2;
  ep.ih = ih; ep.iw = iw; ep.oh = oh; ep.ow = ow; ep.T = T;
  ep.tp = tp; ep.lp = lp; ep.rp = rp;
  const int wt = (ow + T - 1) / T;
  int khs = tp - _ht > 0 ? tp - _ht : 0;
  int khe = 3 < ih + tp - _ht ? 3 : ih + tp - _ht;
  int pad_l = (_wt == 0) && lp > 0;
  int pad_r = (_wt == wt - 1) && rp > 0;
  int cih = _ht + 1 - tp, ciw = _wt * T + 1 - lp;
  uint8_t *in = input + ((size_t)cih * iw + ciw) * 16;
  char *out = (char *)routput + ((size_t)_ht * ow + _wt * T) * 16;
  int attr = with_relu ? (int)AT_RELU_MASK : 0;
#define DW_CASE(k, OT, t)                                                       \
  if (out_kind == k && Tz == t) {                                                \
    run_dw<OT, t>(ep, out, in, weights, wscale, wshift, khs, khe, pad_l, pad_r, \
        attr);                                                                  \
    return 0;                                                                   \
  }
  DW_CASE(1, uint8_t, 4) DW_CASE(1, uint8_t, 5) DW_CASE(1, uint8_t, 6)
  DW_CASE(1, uint8_t, 7) DW_CASE(1, uint8_t, 8) DW_CASE(1, uint8_t, 11)
  DW_CASE(1, uint8_t, 14)
  DW_CASE(2, int8_t, 7) DW_CASE(2, int8_t, 14)
#undef DW_CASE
  return -1;
}

// Direct 3x3 stride-1 micro-kernel (src/kernel/elk_u8s8_conv.hxx:679-901), O = O1 = 1, one
// width block of T outputs of one output row, one 16-wide OC block:
//   input   [I2][ih][iw][16] u8,  weights [3][3][I2][4][16 oc][4 ic] s8,
//   wscale [16], wshift [T][16], routput [oh*ow][16] (u8/s8) or toutput (f32).
// out_kind: 0 = f32 (toutput), 1 = u8, 2 = s8.  T in {7, 14}.
int ref_u8s8_conv3x3(int out_kind, int T, int I2, int ih, int iw, int oh, int ow,
    int _ht, int _wt, int pad, int with_relu, float relu_lo, float relu_hi,
    float *toutput, void *routput, uint8_t *input, int8_t *weights, float *wscale,
    float *wshift)
{
  elx_param_t ep;
  fill_common(ep, relu_lo, relu_hi, 0.f);
  ep.kh = ep.kw = 3; ep.I2 = I2; ep.ic2 = I2; ep.IC = ep.ic = 16 * I2;
  ep.OC = ep.oc = 16; ep.oc2 = 1;
  ep.ih = ih; ep.iw = iw; ep.oh = oh; ep.ow = ow; ep.T = T;
  ep.tp = ep.lp = ep.rp = ep.bp = pad;
  const int wt = (ow + T - 1) / T;
  int khs = pad - _ht > 0 ? pad - _ht : 0;
  int khe = 3 < ih + pad - _ht ? 3 : ih + pad - _ht;
  int kws = _wt == 0 ? pad : 0;
  int kwe = _wt == wt - 1 ? 3 - pad : 3;
  int pad_l = _wt == 0 ? pad : 0;
  int pad_r = _wt == wt - 1 ? pad : 0;
  int cih = _ht + 1 - pad, ciw = _wt * T + 1 - pad;
  uint8_t *in = input + ((size_t)cih * iw + ciw) * 16;
  size_t ooff = ((size_t)_ht * ow + _wt * T) * 16;
  int attr = AT_CLEAR_OUTPUT_MASK | AT_RESTORE_OUTPUT_MASK
      | (with_relu ? (int)AT_RELU_MASK : 0);
#define CV_CASE(k, OT, t)                                                       \
  if (out_kind == k && T == t) {                                                \
    run_conv3<OT, t>(ep, toutput ? toutput + ooff : nullptr,                    \
        routput ? (char *)routput + ooff * sizeof(OT) : nullptr, in, weights,   \
        wscale, wshift, khs, khe, kws, kwe, pad_l, pad_r, attr);                \
    return 0;                                                                   \
  }
  CV_CASE(0, float, 7) CV_CASE(0, float, 14)
  CV_CASE(1, uint8_t, 7) CV_CASE(1, uint8_t, 14)
  CV_CASE(2, int8_t, 7) CV_CASE(2, int8_t, 14)
#undef CV_CASE
  return -1;
}

// The same 3x3 micro-kernel at stride 2 with independent left / right / top pads (0 or 1), set up
// as conv_c160 does (src/elx_int8_conv_direct.cpp:502-571) and bound as the executor binds it:
// the "lean left padding" instantiation S2_LLP when lp > rp, plain 2 otherwise
// (src/elx_int8_conv_direct_bind.hpp:108-117).  T = 7.
// Note for rp = 1: this 3x3-specialised template applies the kw = 2 tap to all T positions at
// stride 2 (unroll_for(_T, T - 1 + S - 1), src/kernel/elk_u8s8_conv.hxx:829-884), i.e. it reads the
// pixel behind the row's end for the last output column, where the template for other kernel
// sizes (:341-347) skips that position.  The golden cases therefore keep rp = 0.
int ref_u8s8_conv3x3_s2(int out_kind, int T, int I2, int ih, int iw, int oh, int ow,
    int _ht, int _wt, int tp, int lp, int rp, int with_relu, float relu_lo, float relu_hi,
    float *toutput, void *routput, uint8_t *input, int8_t *weights, float *wscale,
    float *wshift)
{
  elx_param_t ep;
  fill_common(ep, relu_lo, relu_hi, 0.f);
  ep.kh = ep.kw = 3; ep.I2 = I2; ep.ic2 = I2; ep.IC = ep.ic = 16 * I2;
  ep.OC = ep.oc = 16; ep.oc2 = 1;
  ep.ih = ih; ep.iw = iw; ep.oh = oh; ep.ow = ow; ep.T = T;
  ep.hs = ep.ws = 2;
  ep.tp = tp; ep.lp = lp; ep.rp = rp; ep.bp = 0;
  const int wt = (ow + T - 1) / T;
  int khs = tp - 2 * _ht > 0 ? tp - 2 * _ht : 0;
  int khe = 3 < ih + tp - 2 * _ht ? 3 : ih + tp - 2 * _ht;
  int kws = _wt == 0 ? lp : 0;
  int kwe = _wt == wt - 1 ? 3 - rp : 3;
  int pad_l = _wt == 0 ? lp : 0;
  int pad_r = _wt == wt - 1 ? rp : 0;
  int cih = 2 * _ht + 1 - tp, ciw = 2 * _wt * T + 1 - lp;
  uint8_t *in = input + ((long)cih * iw + ciw) * 16;
  size_t ooff = ((size_t)_ht * ow + _wt * T) * 16;
  int attr = AT_CLEAR_OUTPUT_MASK | AT_RESTORE_OUTPUT_MASK
      | (with_relu ? (int)AT_RELU_MASK : 0);
#define CV_CASE(k, OT, t)                                                       \
  if (out_kind == k && T == t) {                                                \
    if (lp > rp)                                                                \
      run_conv3<OT, t, S2_LLP>(ep, toutput ? toutput + ooff : nullptr,          \
          routput ? (char *)routput + ooff * sizeof(OT) : nullptr, in, weights, \
          wscale, wshift, khs, khe, kws, kwe, pad_l, pad_r, attr);              \
    else                                                                        \
      run_conv3<OT, t, 2>(ep, toutput ? toutput + ooff : nullptr,               \
          routput ? (char *)routput + ooff * sizeof(OT) : nullptr, in, weights, \
          wscale, wshift, khs, khe, kws, kwe, pad_l, pad_r, attr);              \
    return 0;                                                                   \
  }
  CV_CASE(0, float, 7) CV_CASE(1, uint8_t, 7) CV_CASE(2, int8_t, 7)
#undef CV_CASE
  return -1;
}

// The micro-kernel template for the other kernel sizes (5x5 and 7x7: the generic branch,
// src/kernel/elk_u8s8_conv.hxx:254-677), stride 1 or 2, set up and bound as above for any K
// (src/elx_int8_conv_direct.cpp:502-571, src/elx_int8_conv_direct_bind.hpp:108-117).  T = 7, one
// width block (_wt = 0, wt = 1): pads lp on the left and rp on the right of that block.
int ref_u8s8_convk(int K, int S, int out_kind, int I2, int ih, int iw, int oh, int ow, int _ht,
    int tp, int lp, int rp, int with_relu, float relu_lo, float relu_hi, float *toutput,
    void *routput, uint8_t *input, int8_t *weights, float *wscale, float *wshift)
{
  const int T = 7;
  if (ow != T) return -2;
  elx_param_t ep;
  fill_common(ep, relu_lo, relu_hi, 0.f);
  ep.kh = ep.kw = K; ep.I2 = I2; ep.ic2 = I2; ep.IC = ep.ic = 16 * I2;
  ep.OC = ep.oc = 16; ep.oc2 = 1;
  ep.ih = ih; ep.iw = iw; ep.oh = oh; ep.ow = ow; ep.T = T;
  ep.hs = ep.ws = S;
  ep.tp = tp; ep.lp = lp; ep.rp = rp; ep.bp = 0;
  int khs = tp - S * _ht > 0 ? tp - S * _ht : 0;
  int khe = K < ih + tp - S * _ht ? K : ih + tp - S * _ht;
  int kws = lp, kwe = K - rp;
  int cih = S * _ht + K / 2 - tp, ciw = K / 2 - lp;
  uint8_t *in = input + ((long)cih * iw + ciw) * 16;
  size_t ooff = (size_t)_ht * ow * 16;
  int attr = AT_CLEAR_OUTPUT_MASK | AT_RESTORE_OUTPUT_MASK
      | (with_relu ? (int)AT_RELU_MASK : 0);
#define CV_CASE(kk, ss, k, OT)                                                  \
  if (K == kk && S == ss && out_kind == k) {                                    \
    if (ss == 2 && lp > rp)                                                     \
      run_conv3<OT, 7, (ss == 2 ? S2_LLP : 1), kk>(ep, toutput ? toutput + ooff : nullptr, \
          routput ? (char *)routput + ooff * sizeof(OT) : nullptr, in, weights, \
          wscale, wshift, khs, khe, kws, kwe, lp, rp, attr);                    \
    else                                                                        \
      run_conv3<OT, 7, ss, kk>(ep, toutput ? toutput + ooff : nullptr,          \
          routput ? (char *)routput + ooff * sizeof(OT) : nullptr, in, weights, \
          wscale, wshift, khs, khe, kws, kwe, lp, rp, attr);                    \
    return 0;                                                                   \
  }
  CV_CASE(5, 1, 0, float) CV_CASE(5, 1, 1, uint8_t) CV_CASE(5, 1, 2, int8_t)
  CV_CASE(7, 2, 0, float) CV_CASE(7, 2, 1, uint8_t) CV_CASE(7, 2, 2, int8_t)
  CV_CASE(5, 2, 0, float) CV_CASE(5, 2, 1, uint8_t) CV_CASE(5, 2, 2, int8_t)
  CV_CASE(7, 1, 0, float) CV_CASE(7, 1, 1, uint8_t) CV_CASE(7, 1, 2, int8_t)
#undef CV_CASE
  return -1;
}

// The depthwise micro-kernel at stride 2 (its S != 1 branch,
// src/kernel/elk_u8s8_depthwise_conv.hxx:371-403), set up as conv_c160 of the depthwise executor
// does (src/elx_int8_conv_direct_depthwise.cpp:294-319).  Tz in {4, 7}.
int ref_u8s8_depthwise_s2(int out_kind, int T, int Tz, int G2, int ih, int iw, int oh, int ow,
    int _ht, int _wt, int tp, int lp, int rp, int with_relu, float relu_lo,
    float relu_hi, void *routput, uint8_t *input, int8_t *weights, float *wscale,
    float *wshift)
{
  elx_param_t ep;
  fill_common(ep, relu_lo, relu_hi, 0.f);
  ep.kh = ep.kw = 3; ep.G2 = G2; ep.ic2 = G2; ep.oc2 = G2; ep.I2 = G2;
  ep.ih = ih; ep.iw = iw; ep.oh = oh; ep.ow = ow; ep.T = T;
  ep.hs = ep.ws = 2;
  ep.tp = tp; ep.lp = lp; ep.rp = rp;
  const int wt = (ow + T - 1) / T;
  int khs = tp - 2 * _ht > 0 ? tp - 2 * _ht : 0;
  int khe = 3 < ih + tp - 2 * _ht ? 3 : ih + tp - 2 * _ht;
  int pad_l = (_wt == 0) && lp > 0;
  int pad_r = (_wt == wt - 1) && rp > 0;
  int cih = 2 * _ht + 1 - tp, ciw = 2 * _wt * T + 1 - lp;
  uint8_t *in = input + ((long)cih * iw + ciw) * 16;
  char *out = (char *)routput + ((size_t)_ht * ow + _wt * T) * 16;
  int attr = with_relu ? (int)AT_RELU_MASK : 0;
#define DW_CASE(k, OT, t)                                                       \
  if (out_kind == k && Tz == t) {                                                \
    run_dw<OT, t, 2>(ep, out, in, weights, wscale, wshift, khs, khe, pad_l,     \
        pad_r, attr);                                                           \
    return 0;                                                                   \
  }
  DW_CASE(1, uint8_t, 4) DW_CASE(1, uint8_t, 7) DW_CASE(2, int8_t, 7)
#undef DW_CASE
  return -1;
}

// Winograd F(4x4,3x3) input transform of one 6x6 tile of 16 channels
// (src/kernel/elk_conv_wino_4x4_3x3_input.hxx:13-352).  `tile` points at element (0,0) of
// the tile inside an [ih][iw][16] f32 plane; rows/cols outside [hs,he]x[ws,we] read as zero
// when border != 0.  tinput is [6][6][16] f32.
void ref_wino_trans_input(int border, int ih, int iw, float *tinput, float *tile,
    int hs, int he, int ws, int we)
{
  elx_param_t ep;
  fill_common(ep, 0.f, FLT_MAX, 0.f);
  ep.ih = ih; ep.iw = iw;
  if (border)
    elk_conv_wino_trans_input<float, float, TKF_BLOCKED, true, ISA_AVX512, 6,
        16>::execute(ep, tinput, tile, hs, he, ws, we);
  else
    elk_conv_wino_trans_input<float, float, TKF_BLOCKED, false, ISA_AVX512, 6,
        16>::execute(ep, tinput, tile, 0, 5, 0, 5);
}

// Winograd F(4x4,3x3) weights transform of one 16ic x 16oc block
// (src/kernel/elk_conv_wino_4x4_3x3_weights.hxx:18-72): in [3][3][16 ic][16 oc],
// out [6][6][16 ic][16 oc], both f32, 64-byte aligned.
void ref_wino_trans_weights(float *tweights, float *weights)
{
  elk_conv_wino_trans_weights<float, float, ISA_AVX512, 6, 3, 16>::execute(
      *(float(*)[6][6][16][16])tweights, *(float(*)[3][3][16][16])weights);
}

// Winograd F(4x4,3x3) output transform of one tile of 16 channels
// (src/kernel/elk_conv_wino_4x4_3x3_output.hxx:19-201), f32 output in an [oh][ow][16] plane.
// `out` points at the tile's first output element, toutput is [6][6][16] f32, rows > h_end or
// cols > w_end are not written when border != 0.
void ref_wino_trans_output(int border, int with_bias, int with_relu, int oh, int ow,
    float *out, float *toutput, float *bias, int h_end, int w_end)
{
  elx_param_t ep;
  fill_common(ep, 0.f, FLT_MAX, 0.f);
  ep.oh = oh; ep.ow = ow;
#define WO_CASE(b, wb, wr)                                                      \
  if (!!border == b && !!with_bias == wb && !!with_relu == wr) {                \
    elk_conv_wino_trans_output<float, float, float, TKF_BLOCKED, b, wb, wr,     \
        false, ISA_AVX512, 6, 3, 16>::execute(ep, out, toutput, bias, h_end,    \
        w_end);                                                                 \
    return;                                                                     \
  }
  WO_CASE(false, false, false) WO_CASE(false, true, false)
  WO_CASE(false, true, true) WO_CASE(false, false, true)
  WO_CASE(true, false, false) WO_CASE(true, true, false)
  WO_CASE(true, true, true) WO_CASE(true, false, true)
#undef WO_CASE
}

// The same output transform storing u8 (out_kind 1) or s8 (2): * output_quant_repS + output_quant_z
// before the ReLU, round-to-nearest and saturate in the store
// (src/kernel/elk_conv_wino_4x4_3x3_output.hxx:94-111,165-171).  `out` is an [oh][ow][16] byte plane.
void ref_wino_trans_output_q(int out_kind, int border, int with_bias, int with_relu, int oh, int ow,
    void *out, float *toutput, float *bias, int h_end, int w_end, float repS, float z)
{
  elx_param_t ep;
  fill_common(ep, 0.f, FLT_MAX, 0.f);
  ep.oh = oh; ep.ow = ow;
  ep.output_quant_repS = repS;
  ep.output_quant_z = z;
#define WQ_CASE(k, OT, b, wb, wr)                                               \
  if (out_kind == k && !!border == b && !!with_bias == wb && !!with_relu == wr) { \
    elk_conv_wino_trans_output<float, OT, float, TKF_BLOCKED, b, wb, wr,        \
        false, ISA_AVX512, 6, 3, 16>::execute(ep, (OT *)out, toutput, bias,     \
        h_end, w_end);                                                          \
    return;                                                                     \
  }
  WQ_CASE(1, uint8_t, false, true, true) WQ_CASE(1, uint8_t, false, true, false)
  WQ_CASE(1, uint8_t, true, true, true) WQ_CASE(1, uint8_t, true, false, false)
  WQ_CASE(2, int8_t, false, true, true) WQ_CASE(2, int8_t, false, false, false)
  WQ_CASE(2, int8_t, true, true, false) WQ_CASE(2, int8_t, true, true, true)
#undef WQ_CASE
}

// The other tile sizes: A = 4 is F(2x2,3x3) (src/kernel/elk_conv_wino_2x2_3x3_*.hxx), A = 5 is
// F(3x3,3x3) (src/kernel/elk_conv_wino_3x3_3x3_*.hxx).  Same conventions as the A = 6 drivers above;
// tinput / toutput are [A][A][16] f32, the f32 or u8 input tile lies in an [ih][iw][16] plane.
int ref_wino_trans_input_a(int A, int border, int ih, int iw, float *tinput, float *tile,
    int hs, int he, int ws, int we)
{
  elx_param_t ep;
  fill_common(ep, 0.f, FLT_MAX, 0.f);
  ep.ih = ih; ep.iw = iw;
#define WI_CASE(a)                                                              \
  if (A == a) {                                                                 \
    if (border)                                                                 \
      elk_conv_wino_trans_input<float, float, TKF_BLOCKED, true, ISA_AVX512, a, \
          16>::execute(ep, tinput, tile, hs, he, ws, we);                       \
    else                                                                        \
      elk_conv_wino_trans_input<float, float, TKF_BLOCKED, false, ISA_AVX512,   \
          a, 16>::execute(ep, tinput, tile, 0, a - 1, 0, a - 1);                \
    return 0;                                                                   \
  }
  WI_CASE(4) WI_CASE(5)
#undef WI_CASE
  return -1;
}

// in [3][3][16 ic][16 oc], out [A][A][16 ic][16 oc], f32, 64-byte aligned
int ref_wino_trans_weights_a(int A, float *tweights, float *weights)
{
  if (A == 4) {
    elk_conv_wino_trans_weights<float, float, ISA_AVX512, 4, 3, 16>::execute(
        *(float(*)[4][4][16][16])tweights, *(float(*)[3][3][16][16])weights);
    return 0;
  }
  if (A == 5) {
    elk_conv_wino_trans_weights<float, float, ISA_AVX512, 5, 3, 16>::execute(
        *(float(*)[5][5][16][16])tweights, *(float(*)[3][3][16][16])weights);
    return 0;
  }
  return -1;
}

// out_kind 0: f32, 1: u8, 2: s8 output plane [oh][ow][16]; rows > h_end / cols > w_end are not
// written when border != 0
int ref_wino_trans_output_a(int A, int out_kind, int border, int with_bias, int with_relu, int oh,
    int ow, void *out, float *toutput, float *bias, int h_end, int w_end, float repS, float z)
{
  elx_param_t ep;
  fill_common(ep, 0.f, FLT_MAX, 0.f);
  ep.oh = oh; ep.ow = ow;
  ep.output_quant_repS = repS;
  ep.output_quant_z = z;
#define WA_CASE(a, k, OT, b, wb, wr)                                            \
  if (A == a && out_kind == k && !!border == b && !!with_bias == wb && !!with_relu == wr) { \
    elk_conv_wino_trans_output<float, OT, float, TKF_BLOCKED, b, wb, wr,        \
        false, ISA_AVX512, a, 3, 16>::execute(ep, (OT *)out, toutput, bias,     \
        h_end, w_end);                                                          \
    return 0;                                                                   \
  }
#define WA_ALL(a, k, OT)                                                        \
  WA_CASE(a, k, OT, false, false, false) WA_CASE(a, k, OT, false, true, false)  \
  WA_CASE(a, k, OT, false, true, true) WA_CASE(a, k, OT, true, false, false)    \
  WA_CASE(a, k, OT, true, true, false) WA_CASE(a, k, OT, true, true, true)
  WA_ALL(4, 0, float) WA_ALL(4, 1, uint8_t) WA_ALL(4, 2, int8_t)
  WA_ALL(5, 0, float) WA_ALL(5, 1, uint8_t) WA_ALL(5, 2, int8_t)
#undef WA_ALL
#undef WA_CASE
  return -1;
}

// The output transform with the in-place sum fused (with_ip_sum = true): the old output value -- an
// f32, or a u8 / s8 code converted to float -- is added after the output quantization and before the
// ReLU (src/kernel/elk_conv_wino_4x4_3x3_output.hxx:112-131 and the same lines of the other tile sizes).
int ref_wino_trans_output_sum(int A, int out_kind, int border, int with_bias, int with_relu, int oh,
    int ow, void *out, float *toutput, float *bias, int h_end, int w_end, float repS, float z)
{
  elx_param_t ep;
  fill_common(ep, 0.f, FLT_MAX, 0.f);
  ep.oh = oh; ep.ow = ow;
  ep.output_quant_repS = repS;
  ep.output_quant_z = z;
#define WS_CASE(a, k, OT, b, wb, wr)                                            \
  if (A == a && out_kind == k && !!border == b && !!with_bias == wb && !!with_relu == wr) { \
    elk_conv_wino_trans_output<float, OT, float, TKF_BLOCKED, b, wb, wr,        \
        true, ISA_AVX512, a, 3, 16>::execute(ep, (OT *)out, toutput, bias,      \
        h_end, w_end);                                                          \
    return 0;                                                                   \
  }
#define WS_ALL(a, k, OT)                                                        \
  WS_CASE(a, k, OT, false, true, true) WS_CASE(a, k, OT, false, false, false)   \
  WS_CASE(a, k, OT, true, true, true) WS_CASE(a, k, OT, true, true, false)
  WS_ALL(6, 0, float) WS_ALL(6, 1, uint8_t) WS_ALL(6, 2, int8_t)
  WS_ALL(4, 0, float) WS_ALL(4, 1, uint8_t) WS_ALL(4, 2, int8_t)
  WS_ALL(5, 0, float) WS_ALL(5, 1, uint8_t) WS_ALL(5, 2, int8_t)
#undef WS_ALL
#undef WS_CASE
  return -1;
}

} // extern "C"
