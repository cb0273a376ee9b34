// Internal declarations shared by the gfx950 kernels and the C-ABI layer.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <string>

#include "euler_hip.h"

namespace ehip {

typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int kWave = 64;
constexpr int kBlock = 256;      // 4 waves per workgroup everywhere
constexpr int kOcTile = 256;     // packed weights are zero-padded to a multiple of this many rows

inline int up(int x, int m) { return (x + m - 1) / m * m; }

enum Family { FAM_GEMM_1X1 = 1, FAM_CONV_3X3 = 2, FAM_DEPTHWISE = 3, FAM_WINOGRAD = 4 };

// requantization epilogue parameters, by value in kernel arguments
struct Epilogue {
  const float *scale;   // [batch][OCpp]
  const float *shift;   // [batch][OCpp]
  const int *comp;      // [batch][OCpp]  128 * sum of the packed weights (u8 -> s8 remap)
  float sum_scale, lo, hi;
  int out_type;         // EHIP_F32 / U8 / S8 / S32
  int with_sum, with_relu;
};

// D[oc][pixel] = W[oc][k] * X[k][pixel] on MFMA; one "unit" is 16 input channels of one tap.
struct GemmArgs {
  const uint8_t *in;    // [batch][n][ic2][ih*iw][16] u8
  const int8_t *w;      // [batch][units_pad][OCpp][16] s8
  void *out;            // [batch][n][oc2][ohw][16]
  Epilogue ep;
  int p_total;          // pixels per batch entry (n * oh * ow)
  int ohw, ow;          // output plane
  int ihw, iw;          // input plane
  int stride_h, stride_w;
  int ic2;              // real input units
  int units_pad;        // units in the packed weights (multiple of the kernel's chunk)
  int oc2;              // real 16-wide output blocks
  int ocpp;             // padded rows in the packed weights
  long long in_batch_stride;   // bytes
  long long out_batch_stride;  // elements
};

struct Conv3x3Args {
  const uint8_t *in;    // [n][ic2][ih][iw][16]
  const int8_t *w;      // [9][units_pad][OCpp][16]
  void *out;            // [n][oc2][oh][ow][16]
  Epilogue ep;
  int ih, iw, oh, ow;
  int pad_t, pad_l;
  int ic2, units_pad, oc2, ocpp;
  int halo_rows;        // input rows staged per tile
  int chunk_units;      // ic2 units staged per LDS fill (multiple of 4)
};

struct DepthwiseArgs {
  const uint8_t *in;    // [n][g2][ih][iw][16]
  const int8_t *w;      // [g2][9][16]
  void *out;            // [n][g2][oh][ow][16]
  const float *scale, *shift;  // [G]
  int n, g2, ih, iw, oh, ow, pad_t, pad_l;
  int T, Tr, wt;        // width blocking of the reference kernel (decides floor vs round per column)
  int out_type, with_relu;
  float lo, hi;
};

struct WinoArgs {
  const float *in;      // [n][ic2][ih][iw][16] f32
  uint8_t *tin;         // [36][ic2][t][16]
  const float *tout;    // [36][oc2][t][16]
  float *out;           // [n][oc2][oh][ow][16]
  const float *bias;
  int n, ic2, oc2, ih, iw, oh, ow, ht, wt, nt, t, pad_t, pad_l;
  float mrepS, mz;      // input_S / tinput_S, ceil(tinput_z)
  int with_bias, with_relu;
};

// ---- launchers (implemented next to their kernels) ------------------------------------------
hipError_t launch_gemm(const GemmArgs &a, int nbatch, int variant, hipStream_t s);
int gemm_pick_variant(int p_total, int oc2, int ic2, int nbatch);
int gemm_variant_chunk(int variant);
const char *gemm_variant_name(int variant);

hipError_t launch_conv3x3(const Conv3x3Args &a, int n, int variant, size_t lds_bytes, hipStream_t s);
int conv3x3_pick_variant(int oh, int ow, int oc2);
int conv3x3_variant_pixels(int variant);
const char *conv3x3_variant_name(int variant);

hipError_t launch_depthwise(const DepthwiseArgs &a, hipStream_t s);
hipError_t launch_wino_trans_input(const WinoArgs &a, hipStream_t s);
hipError_t launch_wino_trans_output(const WinoArgs &a, hipStream_t s);
hipError_t launch_wino_range(const WinoArgs &a, int ic_real, unsigned *minmax_dev, hipStream_t s);

// weight preparation
hipError_t launch_prepare_direct(const float *w_blocked, const float *bias, int oc, int ic, int kh, int kw,
                                 int units_pad, int ocpp, const ehip_conv_desc_t &d, float *absmax_scratch,
                                 int8_t *wpacked, float *scale, float *shift, int *wsum, int *comp, hipStream_t s);
hipError_t launch_prepare_depthwise(const float *w_goihw, const float *bias, int g, const ehip_conv_desc_t &d,
                                    int8_t *wpacked, float *scale, float *shift, int *wsum, hipStream_t s);
hipError_t launch_prepare_wino(const float *w_blocked, int oc, int ic, int units_pad, int ocpp,
                               const ehip_conv_desc_t &d, float *u_tmp, int8_t *wpacked, float *scale,
                               float *shift, int *wsum, int *comp, hipStream_t s);
hipError_t launch_quantize_input(uint8_t *dst, const float *src, size_t count, float scale, float z,
                                 hipStream_t s);
hipError_t launch_reorder_nchw_to_blocked(void *dst, const void *src, int es, int n, int c, int h, int w,
                                          hipStream_t s);
hipError_t launch_reorder_blocked_to_nchw(void *dst, const void *src, int es, int n, int c, int h, int w,
                                          hipStream_t s);
hipError_t launch_reorder_oihw_to_blocked(float *dst, const float *src, int o, int i, int h, int w,
                                          hipStream_t s);

void set_error(const std::string &msg);

}  // namespace ehip

// ---- device helpers -----------------------------------------------------------------------------
#if defined(__HIPCC__)
namespace ehip {

// round-to-nearest-even float -> s32 with the x86 "integer indefinite" for NaN / out of range
__device__ __forceinline__ int cvt_s32_rne(float f)
{
  if (!(f >= -2147483648.0f && f < 2147483648.0f)) return (int)0x80000000;
  return (int)__builtin_rintf(f);
}
// float -> u32, round-to-nearest-even; NaN / negative / too large -> 0xffffffff
__device__ __forceinline__ unsigned cvt_u32_rne(float f)
{
  float r = __builtin_rintf(f);
  if (!(r >= 0.0f && r < 4294967296.0f)) return 0xffffffffu;
  return (unsigned)r;
}
__device__ __forceinline__ unsigned usat8(unsigned v) { return v > 255u ? 255u : v; }
__device__ __forceinline__ int ssat8(int v) { return v < -128 ? -128 : (v > 127 ? 127 : v); }

// acc * scale + shift (one rounding), [+ old * sum_scale (one rounding)], clamp
__device__ __forceinline__ float requant(int acc, float scale, float shift, bool with_sum, int old_q,
                                         float sum_scale, bool relu, float lo, float hi)
{
  float f = __builtin_fmaf((float)acc, scale, shift);
  if (with_sum) f = __builtin_fmaf((float)old_q, sum_scale, f);
  if (relu) {
    f = f > lo ? f : lo;
    f = f < hi ? f : hi;
  }
  return f;
}

// Epilogue for one lane's 4 consecutive output channels of one pixel.
//   acc      the four s32 accumulators (compensation already added)
//   oc       first of the four channels (multiple of 4)
//   out_elem element index of channel `oc` of this pixel in the output tensor
__device__ __forceinline__ void store_quad(const Epilogue &ep, const float *scale, const float *shift,
                                           v4i acc, int oc, void *out, size_t out_elem)
{
  if (ep.out_type == EHIP_S32) {
    *reinterpret_cast<v4i *>(static_cast<int *>(out) + out_elem) = acc;
    return;
  }
  const float4 sc = *reinterpret_cast<const float4 *>(scale + oc);
  const float4 sh = *reinterpret_cast<const float4 *>(shift + oc);
  const bool relu = ep.with_relu != 0;
  if (ep.out_type == EHIP_F32) {
    float4 r;
    r.x = requant(acc.x, sc.x, sh.x, false, 0, 0.f, relu, ep.lo, ep.hi);
    r.y = requant(acc.y, sc.y, sh.y, false, 0, 0.f, relu, ep.lo, ep.hi);
    r.z = requant(acc.z, sc.z, sh.z, false, 0, 0.f, relu, ep.lo, ep.hi);
    r.w = requant(acc.w, sc.w, sh.w, false, 0, 0.f, relu, ep.lo, ep.hi);
    *reinterpret_cast<float4 *>(static_cast<float *>(out) + out_elem) = r;
    return;
  }
  unsigned *dst = reinterpret_cast<unsigned *>(static_cast<uint8_t *>(out) + out_elem);
  const bool with_sum = ep.with_sum != 0;
  unsigned old = with_sum ? *dst : 0u;
  int o0, o1, o2, o3;
  if (ep.out_type == EHIP_U8) {
    o0 = old & 0xff; o1 = (old >> 8) & 0xff; o2 = (old >> 16) & 0xff; o3 = old >> 24;
  } else {
    o0 = (int)(signed char)(old & 0xff); o1 = (int)(signed char)((old >> 8) & 0xff);
    o2 = (int)(signed char)((old >> 16) & 0xff); o3 = (int)(signed char)(old >> 24);
  }
  float f0 = requant(acc.x, sc.x, sh.x, with_sum, o0, ep.sum_scale, relu, ep.lo, ep.hi);
  float f1 = requant(acc.y, sc.y, sh.y, with_sum, o1, ep.sum_scale, relu, ep.lo, ep.hi);
  float f2 = requant(acc.z, sc.z, sh.z, with_sum, o2, ep.sum_scale, relu, ep.lo, ep.hi);
  float f3 = requant(acc.w, sc.w, sh.w, with_sum, o3, ep.sum_scale, relu, ep.lo, ep.hi);
  unsigned q0, q1, q2, q3;
  if (ep.out_type == EHIP_U8) {
    // the reference narrows the rounded s32 with an UNSIGNED saturation: negatives become 255
    q0 = usat8((unsigned)cvt_s32_rne(f0)); q1 = usat8((unsigned)cvt_s32_rne(f1));
    q2 = usat8((unsigned)cvt_s32_rne(f2)); q3 = usat8((unsigned)cvt_s32_rne(f3));
  } else {
    q0 = (unsigned)ssat8(cvt_s32_rne(f0)) & 0xff; q1 = (unsigned)ssat8(cvt_s32_rne(f1)) & 0xff;
    q2 = (unsigned)ssat8(cvt_s32_rne(f2)) & 0xff; q3 = (unsigned)ssat8(cvt_s32_rne(f3)) & 0xff;
  }
  *dst = q0 | (q1 << 8) | (q2 << 16) | (q3 << 24);
}

}  // namespace ehip
#endif
