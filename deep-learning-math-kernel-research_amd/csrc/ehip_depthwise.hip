// Depthwise 3x3 stride-1 u8 x s8 convolution with fused requantization: a bandwidth kernel.
//
// Replaces elx_int8_conv_direct_depthwise_t::__execute_c160 + conv_c160
// (src/elx_int8_conv_direct_depthwise_xopt.hpp:19-66, src/elx_int8_conv_direct_depthwise.cpp:294-319)
// and the depthwise micro-kernel (src/kernel/elk_u8s8_depthwise_conv.hxx:219-474).
//
// There is no contraction over channels, so the matrix cores have nothing to do: every lane owns
// one output column of one 16-channel block and walks RB output rows down it, so that each input
// cell (16 bytes = the 16 channels of a pixel) is loaded once per three columns instead of nine
// times; neighbouring lanes read neighbouring cells (coalesced 16-byte accesses) and the overlap
// between columns is served by the vector L1.  Out-of-image taps are skipped exactly as the
// reference skips them.
//
// The u8 store reproduces the reference's width-block rule: inside every block of T output columns
// (Tr for the last block) the columns before 4*floor(Tz/4) are rounded toward -infinity and
// byte-merged without saturation, the remaining ones are rounded to nearest even and saturated.
#include "ehip_internal.hpp"

namespace ehip {

template <int RB>
__global__ __launch_bounds__(kBlock) void k_depthwise3x3_u8s8(DepthwiseArgs a)
{
  const int ohb = (a.oh + RB - 1) / RB;
  const long long total = (long long)a.n * a.g2 * ohb * a.ow;
  const long long idx = (long long)blockIdx.x * kBlock + threadIdx.x;
  if (idx >= total) return;
  const int ow = (int)(idx % a.ow);
  long long rest = idx / a.ow;
  const int hb = (int)(rest % ohb);
  const long long ng = rest / ohb;  // n * g2 + g2 index
  const int g2 = (int)(ng % a.g2);
  const int oh0 = hb * RB;

  // weights of this 16-channel block: [9][16] s8
  uint4 wv[9];
  const uint4 *wp = reinterpret_cast<const uint4 *>(a.w) + (size_t)g2 * 9;
#pragma unroll
  for (int k = 0; k < 9; ++k) wv[k] = wp[k];

  int acc[RB][16];
#pragma unroll
  for (int r = 0; r < RB; ++r)
#pragma unroll
    for (int c = 0; c < 16; ++c) acc[r][c] = 0;

  const uint4 *plane = reinterpret_cast<const uint4 *>(a.in) + (size_t)ng * a.ih * a.iw;
#pragma unroll
  for (int hr = 0; hr < RB + 2; ++hr) {
    const int ih = oh0 - a.pad_t + hr;
    if (ih < 0 || ih >= a.ih) continue;
    uint4 x[3];
#pragma unroll
    for (int kw = 0; kw < 3; ++kw) {
      const int iw = ow - a.pad_l + kw;
      x[kw] = (iw >= 0 && iw < a.iw) ? plane[(size_t)ih * a.iw + iw] : make_uint4(0u, 0u, 0u, 0u);
    }
#pragma unroll
    for (int r = 0; r < RB; ++r) {
      const int kh = hr - r;  // input row ih feeds output row oh0 + r through tap row kh
      if (kh < 0 || kh > 2) continue;
#pragma unroll
      for (int kw = 0; kw < 3; ++kw) {
        const unsigned xd[4] = {x[kw].x, x[kw].y, x[kw].z, x[kw].w};
        const uint4 w4 = wv[kh * 3 + kw];
        const unsigned wd[4] = {w4.x, w4.y, w4.z, w4.w};
#pragma unroll
        for (int d = 0; d < 4; ++d)
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            const int xb = (int)((xd[d] >> (8 * k)) & 0xffu);
            const int wb = (int)(signed char)((wd[d] >> (8 * k)) & 0xffu);
            acc[r][4 * d + k] += xb * wb;
          }
      }
    }
  }

  // width-block rule for this column
  const int blk = ow / a.T;
  const int tpos = ow - blk * a.T;
  const int Tz = blk == a.wt - 1 ? a.Tr : a.T;
  const bool floor_col = a.out_type == EHIP_U8 && tpos < 4 * (Tz / 4);
  const bool relu = a.with_relu != 0;

  float sc[16], sh[16];
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    const float4 s4 = reinterpret_cast<const float4 *>(a.scale)[g2 * 4 + d];
    const float4 z4 = reinterpret_cast<const float4 *>(a.shift)[g2 * 4 + d];
    sc[4 * d] = s4.x; sc[4 * d + 1] = s4.y; sc[4 * d + 2] = s4.z; sc[4 * d + 3] = s4.w;
    sh[4 * d] = z4.x; sh[4 * d + 1] = z4.y; sh[4 * d + 2] = z4.z; sh[4 * d + 3] = z4.w;
  }

#pragma unroll
  for (int r = 0; r < RB; ++r) {
    const int oh = oh0 + r;
    if (oh >= a.oh) break;
    unsigned o[4] = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int c = 0; c < 16; ++c) {
      const float f = requant(acc[r][c], sc[c], sh[c], false, 0, 0.f, relu, a.lo, a.hi);
      unsigned q;
      if (a.out_type == EHIP_S32) {
        q = 0;
      } else if (floor_col) {
        const int fl = (!(f >= -2147483648.0f && f < 2147483648.0f)) ? (int)0x80000000 : (int)__builtin_floorf(f);
        q = (unsigned)fl & 0xffu;
      } else if (a.out_type == EHIP_U8) {
        q = usat8((unsigned)cvt_s32_rne(f));
      } else {
        q = (unsigned)ssat8(cvt_s32_rne(f)) & 0xffu;
      }
      o[c >> 2] |= q << (8 * (c & 3));
    }
    const size_t cell = ((size_t)ng * a.oh + oh) * a.ow + ow;
    if (a.out_type == EHIP_S32) {
      v4i *dst = reinterpret_cast<v4i *>(a.out) + cell * 4;
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        v4i v = {acc[r][4 * d], acc[r][4 * d + 1], acc[r][4 * d + 2], acc[r][4 * d + 3]};
        dst[d] = v;
      }
    } else {
      reinterpret_cast<uint4 *>(a.out)[cell] = make_uint4(o[0], o[1], o[2], o[3]);
    }
  }
}

hipError_t launch_depthwise(const DepthwiseArgs &a, hipStream_t s)
{
  // four rows per lane on tall planes, fewer where that would leave lanes idle
  const int rb = a.oh >= 16 ? 4 : (a.oh >= 7 ? 2 : 1);
  const int ohb = (a.oh + rb - 1) / rb;
  const long long total = (long long)a.n * a.g2 * ohb * a.ow;
  dim3 grid((unsigned)((total + kBlock - 1) / kBlock));
  if (rb == 4) hipLaunchKernelGGL(k_depthwise3x3_u8s8<4>, grid, dim3(kBlock), 0, s, a);
  else if (rb == 2) hipLaunchKernelGGL(k_depthwise3x3_u8s8<2>, grid, dim3(kBlock), 0, s, a);
  else hipLaunchKernelGGL(k_depthwise3x3_u8s8<1>, grid, dim3(kBlock), 0, s, a);
  return hipGetLastError();
}

}  // namespace ehip
