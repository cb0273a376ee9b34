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
inline unsigned div_magic(int d) { return d <= 1 ? 0u : (unsigned)((1ull << 32) / (unsigned)d + 1); }

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
  unsigned ohw_magic, ow_magic;  // floor(2^32 / d) + 1: n / d == umulhi(n, magic) while n * d < 2^32
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
  long long *trace;     // development aid, normally null (see EHIP_TRACE)
  int dbg;              // development aid: bit 0 = skip LDS operand reads, bit 1 = skip weight reloads
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
int gemm_num_variants();
const char *gemm_variant_name(int variant);

hipError_t launch_conv3x3(const Conv3x3Args &a, int n, int variant, size_t lds_bytes, hipStream_t s);
int conv3x3_pick_variant(int oh, int ow, int oc2);
int conv3x3_variant_pixels(int variant);
int conv3x3_variant_slots(int variant);   // 16-byte cells of one LDS buffer
int conv3x3_num_variants();
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
// n / d for n * d < 2^32 with magic = div_magic(d) (d == 1 has no 32-bit magic)
__device__ __forceinline__ int fastdiv(int n, int d, unsigned magic)
{
  return d == 1 ? n : (int)__umulhi((unsigned)n, magic);
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

// ---- fused requantization epilogue of the MFMA kernels -----------------------------------------
// A lane holds, for each of its NP pixels and MO 16-channel blocks, 4 consecutive output
// channels (one dword of u8/s8, one float4 of f32/s32).  The per-channel scale/shift are loaded
// once per kernel (hoisted by the caller), the sum operands are all requested before the first
// one is used, and the output type is a template parameter, so the epilogue is straight-line code
// whose memory latencies overlap instead of queueing behind each other.
__device__ __forceinline__ float requant1(int acc, float scale, float shift, bool relu, float lo, float hi)
{
  float f = __builtin_fmaf((float)acc, scale, shift);
  if (relu) {
    // max(f, lo) / min(f, hi) with the operand order of the reference (a NaN f yields lo)
    f = __builtin_fmaxf(f, lo);
    f = __builtin_fminf(f, hi);
  }
  return f;
}

template <int OUT>
__device__ __forceinline__ unsigned quant1(float f)
{
  // round-to-nearest-even, then the reference's narrowing: u8 saturates the s32 as UNSIGNED
  // (negatives become 255), s8 saturates signed.  v_cvt_i32_f32 already saturates out-of-range
  // values to INT_MAX/INT_MIN, both of which narrow like the x86 "integer indefinite"; only NaN
  // (which converts to 0 here, to 0x80000000 there) needs a fix-up.
  const float r = __builtin_rintf(f);
  int i = (int)r;
  i = (f != f) ? (int)0x80000000 : i;
  if (OUT == EHIP_U8) return usat8((unsigned)i);
  return (unsigned)ssat8(i) & 0xffu;
}

template <int MO, int NP, int OUT, bool SUM>
__device__ __forceinline__ void epilogue_tile(const Epilogue &ep, const v4i (&acc)[MO][NP], const float4 (&sc)[MO],
                                              const float4 (&sh)[MO], const size_t (&pix)[NP],
                                              const bool (&pvalid)[NP], const int (&oc_of)[MO], int oc_real,
                                              size_t oc2_stride, void *out)
{
  // oc_of[mo]: the lane's first channel (a multiple of 4) of its quad in block mo
  const bool relu = ep.with_relu != 0;
  unsigned old[MO][NP];
  if (SUM) {
#pragma unroll
    for (int mo = 0; mo < MO; ++mo)
#pragma unroll
      for (int np = 0; np < NP; ++np) {
        const int oc = oc_of[mo];
        const bool ok = pvalid[np] && oc < oc_real;
        const size_t e = ok ? pix[np] + (size_t)(oc >> 4) * oc2_stride + (oc & 15) : 0;
        old[mo][np] = *reinterpret_cast<const unsigned *>(static_cast<const uint8_t *>(out) + e);
      }
  }
#pragma unroll
  for (int mo = 0; mo < MO; ++mo) {
    const int oc = oc_of[mo];
    if (oc >= oc_real) continue;
#pragma unroll
    for (int np = 0; np < NP; ++np) {
      if (!pvalid[np]) continue;
      const size_t e = pix[np] + (size_t)(oc >> 4) * oc2_stride + (oc & 15);
      const v4i a4 = acc[mo][np];
      if (OUT == EHIP_S32) {
        *reinterpret_cast<v4i *>(static_cast<int *>(out) + e) = a4;
      } else if (OUT == EHIP_F32) {
        float4 r;
        r.x = requant1(a4.x, sc[mo].x, sh[mo].x, relu, ep.lo, ep.hi);
        r.y = requant1(a4.y, sc[mo].y, sh[mo].y, relu, ep.lo, ep.hi);
        r.z = requant1(a4.z, sc[mo].z, sh[mo].z, relu, ep.lo, ep.hi);
        r.w = requant1(a4.w, sc[mo].w, sh[mo].w, relu, ep.lo, ep.hi);
        *reinterpret_cast<float4 *>(static_cast<float *>(out) + e) = r;
      } else {
        float f0 = __builtin_fmaf((float)a4.x, sc[mo].x, sh[mo].x);
        float f1 = __builtin_fmaf((float)a4.y, sc[mo].y, sh[mo].y);
        float f2 = __builtin_fmaf((float)a4.z, sc[mo].z, sh[mo].z);
        float f3 = __builtin_fmaf((float)a4.w, sc[mo].w, sh[mo].w);
        if (SUM) {
          const unsigned o = old[mo][np];
          int o0, o1, o2, o3;
          if (OUT == EHIP_U8) {
            o0 = o & 0xff; o1 = (o >> 8) & 0xff; o2 = (o >> 16) & 0xff; o3 = o >> 24;
          } else {
            o0 = (int)(signed char)(o & 0xff); o1 = (int)(signed char)((o >> 8) & 0xff);
            o2 = (int)(signed char)((o >> 16) & 0xff); o3 = (int)(signed char)(o >> 24);
          }
          f0 = __builtin_fmaf((float)o0, ep.sum_scale, f0);
          f1 = __builtin_fmaf((float)o1, ep.sum_scale, f1);
          f2 = __builtin_fmaf((float)o2, ep.sum_scale, f2);
          f3 = __builtin_fmaf((float)o3, ep.sum_scale, f3);
        }
        if (relu) {
          f0 = __builtin_fminf(__builtin_fmaxf(f0, ep.lo), ep.hi);
          f1 = __builtin_fminf(__builtin_fmaxf(f1, ep.lo), ep.hi);
          f2 = __builtin_fminf(__builtin_fmaxf(f2, ep.lo), ep.hi);
          f3 = __builtin_fminf(__builtin_fmaxf(f3, ep.lo), ep.hi);
        }
        const unsigned q = quant1<OUT>(f0) | (quant1<OUT>(f1) << 8) | (quant1<OUT>(f2) << 16) | (quant1<OUT>(f3) << 24);
        *reinterpret_cast<unsigned *>(static_cast<uint8_t *>(out) + e) = q;
      }
    }
  }
}

// one uniform switch on the output type around the whole tile epilogue
template <int MO, int NP>
__device__ __forceinline__ void epilogue_dispatch(const Epilogue &ep, const v4i (&acc)[MO][NP], const float4 (&sc)[MO],
                                                  const float4 (&sh)[MO], const size_t (&pix)[NP],
                                                  const bool (&pvalid)[NP], const int (&oc_of)[MO], int oc_real,
                                                  size_t oc2_stride, void *out)
{
  switch (ep.out_type) {
  case EHIP_U8:
    if (ep.with_sum) epilogue_tile<MO, NP, EHIP_U8, true>(ep, acc, sc, sh, pix, pvalid, oc_of, oc_real, oc2_stride, out);
    else epilogue_tile<MO, NP, EHIP_U8, false>(ep, acc, sc, sh, pix, pvalid, oc_of, oc_real, oc2_stride, out);
    break;
  case EHIP_S8:
    if (ep.with_sum) epilogue_tile<MO, NP, EHIP_S8, true>(ep, acc, sc, sh, pix, pvalid, oc_of, oc_real, oc2_stride, out);
    else epilogue_tile<MO, NP, EHIP_S8, false>(ep, acc, sc, sh, pix, pvalid, oc_of, oc_real, oc2_stride, out);
    break;
  case EHIP_F32:
    epilogue_tile<MO, NP, EHIP_F32, false>(ep, acc, sc, sh, pix, pvalid, oc_of, oc_real, oc2_stride, out);
    break;
  default:
    epilogue_tile<MO, NP, EHIP_S32, false>(ep, acc, sc, sh, pix, pvalid, oc_of, oc_real, oc2_stride, out);
    break;
  }
}

}  // namespace ehip
#endif
