// TEST INFRASTRUCTURE ONLY.
//
// Entry points into the reference's own test harness, compiled from where it lies
// (/root/reference/tests/elt_conv_utils.cpp together with src/elx_reorder.cpp; see oracle/Makefile):
//
//   ref_harness_conv2d    test::ref_convolution2d<float, float, float, float>
//                         (tests/elt_conv_utils.cpp:666-750) on plain nchw / (g)oihw tensors;
//   ref_harness_prepare   test::prepare_conv_data (tests/elt_conv_utils.cpp:87-463) for the int8 data-type
//                         configurations of a direct layer: it draws the fp32 tensors, calibrates
//                         input_quant / output_quant / sum_quant from the fp32 reference convolution
//                         (:264-346) and quantizes the input and the sum operand (:354-401, :444-462).
//
// The descriptors are raw zeroed storage with the fields these two functions read filled in: the
// descriptor's constructor and setup() live in the executor library, which is not built here.
// Used by tests/golden/cases.py to write the harness fixtures and by the tests that pin the oracle's
// restatement of the harness (orc_ref_conv_f32, orc_calibrate_output_quant, orc_quantize_input_u8).
#include <cstdlib>
#include <cstring>

#include "euler.hpp"
#include "elt_conv_utils.hpp"

using namespace euler;

namespace {
struct raw_desc {
  alignas(64) char buf[sizeof(eld_conv_t)];
  eld_conv_t &fill(int n, int g, int ic, int oc, int ih, int iw, int oh, int ow, int kh, int kw, int pt, int pl, int sh,
                   int sw, int with_bias, int with_relu, int with_sum)
  {
    memset(buf, 0, sizeof(buf));
    eld_conv_t &d = *reinterpret_cast<eld_conv_t *>(buf);
    d.dims = {n, g, ic, oc, ih, iw, oh, ow, kh, kw};
    d.pads = {pl, 0, pt, 0};
    d.strides = {sh, sw};
    d.dilations = {1, 1};
    d.formats = {nchw, g > 1 ? goihw : oihw, nchw};
    d.algorithm = CONV_DIRECT;
    d.with_bias = with_bias != 0;
    d.with_relu = with_relu != 0;
    d.with_ip_sum = with_sum != 0;
    d.sizes = {(size_t)n * ic * ih * iw, (size_t)oc * (ic / g) * kh * kw, (size_t)n * oc * oh * ow, (size_t)oc};
    d.byte_sizes = {d.sizes.input * 4, d.sizes.weights * 4, d.sizes.output * 4, d.sizes.bias * 4};
    return d;
  }
};
}  // namespace

extern "C" int ref_harness_conv2d(int n, int g, int ic, int oc, int ih, int iw, int oh, int ow, int kh, int kw, int pt,
                                  int pl, int sh, int sw, int with_bias, int with_relu, int with_sum, float *output,
                                  float *input, float *weights, float *bias)
{
  raw_desc r;
  eld_conv_t &d = r.fill(n, g, ic, oc, ih, iw, oh, ow, kh, kw, pt, pl, sh, sw, with_bias, with_relu, with_sum);
  return test::ref_convolution2d<float, float, float, float>(d, output, input, weights, bias);
}

// out_s8: 0 = the U8F32U8F32 configuration, 1 = U8F32S8F32; zero_point: the "...z" variants (input z = 128).
// The four *_ref arrays are filled by the harness; input_q / sum_q (one byte per element) receive what it
// quantized; quant = {input scale, input z, output scale, output z, sum scale}.
extern "C" int ref_harness_prepare(int out_s8, int zero_point, int n, int g, int ic, int oc, int ih, int iw, int oh,
                                   int ow, int kh, int kw, int pt, int pl, int sh, int sw, int with_relu, int with_sum,
                                   float *input_ref, float *weights_ref, float *output_ref, float *bias_ref,
                                   uint8_t *input_q, uint8_t *sum_q, float *quant)
{
  raw_desc r0, r1;
  eld_conv_t &ref = r0.fill(n, g, ic, oc, ih, iw, oh, ow, kh, kw, pt, pl, sh, sw, 1, with_relu, with_sum);
  eld_conv_t &d = r1.fill(n, g, ic, oc, ih, iw, oh, ow, kh, kw, pt, pl, sh, sw, 1, with_relu, with_sum);
  uint8_t *in = nullptr;
  float *w = nullptr, *b = nullptr;
  void *out = nullptr;
  if (out_s8) {
    int8_t *o = nullptr;
    test::prepare_conv_data<uint8_t, float, int8_t, float>(
        ref, d, input_ref, weights_ref, output_ref, bias_ref, &in, &w, &o, &b, nullptr, nullptr, nullptr, nchw, oihw, false,
        zero_point ? test::U8F32S8F32z : test::U8F32S8F32, false, true);
    out = o;
  } else {
    uint8_t *o = nullptr;
    test::prepare_conv_data<uint8_t, float, uint8_t, float>(
        ref, d, input_ref, weights_ref, output_ref, bias_ref, &in, &w, &o, &b, nullptr, nullptr, nullptr, nchw, oihw, false,
        zero_point ? test::U8F32U8F32z : test::U8F32U8F32, false, true);
    out = o;
  }
  memcpy(input_q, in, ref.sizes.input);
  if (with_sum) memcpy(sum_q, out, ref.sizes.output);
  quant[0] = d.input_quant.scale;
  quant[1] = d.input_quant.z;
  quant[2] = d.output_quant.scale;
  quant[3] = d.output_quant.z;
  quant[4] = d.sum_quant.scale;
  free(in);
  free(w);
  free(b);
  free(out);
  return 0;
}
