// The calibration side of the reference's test harness (tests/elt_conv_utils.cpp:290-352), on the device:
//
//   ehip_ref_conv_f32_range    the harness's fp32 reference convolution (ref_convolution2d,
//                              tests/elt_conv_utils.cpp:666-750) with the minimum and maximum of its result --
//                              what output_quant and sum_quant are calibrated from;
//   ehip_calibrate_output_quant  the harness's rule that turns those ranges into output_quant / sum_quant
//                              (tests/elt_conv_utils.cpp:313-346).
//
// ref_convolution2d starts every output from the bias (plus the old output with with_ip_sum), adds the
// products in the order (ic, kh, kw) skipping padded taps, and clamps negatives to zero with with_relu.
// The kernel below keeps that order, one thread per output value, with each `out += x * w` as one fmaf.
// It is a calibration tool, not a hot path: ~10 TFLOP/s is plenty for a once-per-layer call.
#include "ehip_internal.hpp"

namespace ehip {

// block = 16 output channels (one unit) x 16 consecutive output pixels of one image
__global__ __launch_bounds__(256) void k_ref_conv_f32(RefConvArgs a)
{
  const int ov = threadIdx.x & 15, pl = threadIdx.x >> 4;
  const int npix = a.oh * a.ow;
  const int pblocks = (npix + 15) / 16;
  const int pb = blockIdx.x % pblocks, o2 = blockIdx.x / pblocks % a.oc2, n = blockIdx.x / pblocks / a.oc2;
  const int pix = pb * 16 + pl, oc = o2 * 16 + ov;
  const bool live = pix < npix && oc < a.oc;
  float lo = INFINITY, hi = -INFINITY;
  if (live) {
    const int oh = pix / a.ow, ow = pix % a.ow;
    const size_t oidx = a.out_nhwc ? ((size_t)n * npix + pix) * a.oc + oc
                                   : (((size_t)n * a.oc2 + o2) * npix + pix) * 16 + ov;
    float acc = a.with_bias ? a.bias[oc] : 0.0f;
    if (a.with_sum) acc = a.out[oidx] + acc;
    const int icg = a.ic / a.g, ocg = a.oc / a.g;
    const int grp = oc / ocg;
    for (int i = 0; i < icg; ++i) {
      const int ic = grp * icg + i;
      for (int kh = 0; kh < a.kh; ++kh) {
        const int ih = oh * a.sh - a.pad_t + kh;
        if (ih < 0 || ih >= a.ih) continue;
        for (int kw = 0; kw < a.kw; ++kw) {
          const int iw = ow * a.sw - a.pad_l + kw;
          if (iw < 0 || iw >= a.iw) continue;
          const size_t xi = a.in_nhwc ? (((size_t)n * a.ih + ih) * a.iw + iw) * a.ic + ic
                                      : ((((size_t)n * a.ic2 + ic / 16) * a.ih + ih) * a.iw + iw) * 16 + ic % 16;
          const size_t wi = a.w_goihw ? (((size_t)oc * icg + i) * a.kh + kh) * a.kw + kw
                                      : (((((size_t)o2 * a.ic2 + ic / 16) * a.kh + kh) * a.kw + kw) * 16 + ic % 16) * 16 + ov;
          acc = fmaf(a.in[xi], a.w[wi], acc);
        }
      }
    }
    if (a.with_relu && acc < 0.0f) acc = 0.0f;
    if (a.out) a.out[oidx] = acc;
    lo = hi = acc;
  }
  // block range: wave shuffles, then the four waves through LDS
  for (int off = 32; off > 0; off >>= 1) {
    lo = fminf(lo, __shfl_xor(lo, off, 64));
    hi = fmaxf(hi, __shfl_xor(hi, off, 64));
  }
  __shared__ float red[8];
  if ((threadIdx.x & 63) == 0) {
    red[(threadIdx.x >> 6) * 2] = lo;
    red[(threadIdx.x >> 6) * 2 + 1] = hi;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    a.partials[2 * (size_t)blockIdx.x] = fminf(fminf(red[0], red[2]), fminf(red[4], red[6]));
    a.partials[2 * (size_t)blockIdx.x + 1] = fmaxf(fmaxf(red[1], red[3]), fmaxf(red[5], red[7]));
  }
}

hipError_t launch_ref_conv_f32(const RefConvArgs &a, unsigned blocks)
{
  hipLaunchKernelGGL(k_ref_conv_f32, dim3(blocks), dim3(256), 0, nullptr, a);
  return hipGetLastError();
}

}  // namespace ehip
