// Drives the C++ API the way a program written against the reference does (tests/elt_conv.cpp:
// fill eld_conv_t, setup(), elx_conv() on HOST buffers in the blocked formats made with reorder<>),
// so that the pytest side can compare the result with the CPU oracle.
//
//   euler_api_check <in.bin> <out.bin> n ic oc hw k pad stride out_type algorithm with_sum T out_scale sum_scale g nhwc
//                   [in_type tile_size execution_mode tinput_scale tinput_z]
//
// in.bin : input nchw (u8, or f32 when in_type says so) | f32 weights oihw (goihw for g > 1) | f32 bias[oc] |
//          [old output nchw, output type]
// out.bin: output nchw in the output type
// The five optional arguments describe a Winograd layer the way the reference's benchmark does
// (tests/elt_conv.cpp: --alg=wino --tile-size --execution-mode, wino_tinput_quant from calibration).
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include <hip/hip_runtime_api.h>

#include "euler.hpp"
#include "euler_reorder.hpp"

using namespace euler;

static size_t up16(size_t x) { return (x + 15) / 16 * 16; }

int main(int argc, char **argv)
{
  if (argc != 18 && argc != 23) {
    fprintf(stderr, "usage: see source\n");
    return 2;
  }
  const char *in_path = argv[1], *out_path = argv[2];
  const int n = atoi(argv[3]), ic = atoi(argv[4]), oc = atoi(argv[5]), hw = atoi(argv[6]), k = atoi(argv[7]);
  const int pad = atoi(argv[8]), stride = atoi(argv[9]), out_type = atoi(argv[10]), algorithm = atoi(argv[11]);
  const int with_sum = atoi(argv[12]), T = atoi(argv[13]);
  const float out_scale = (float)atof(argv[14]), sum_scale = (float)atof(argv[15]);
  const int g = atoi(argv[16]);
  const bool use_nhwc = atoi(argv[17]) != 0;   // activations [n][h][w][c] on both sides
  const bool wino = argc == 23;
  const int in_type = wino ? atoi(argv[18]) : (int)u8;
  const int tile_size = wino ? atoi(argv[19]) : 0;
  const unsigned execution_mode = wino ? (unsigned)strtoul(argv[20], nullptr, 0) : 0;
  const float tinput_scale = wino ? (float)atof(argv[21]) : 0.0f, tinput_z = wino ? (float)atof(argv[22]) : 0.0f;
  const size_t isz = in_type == f32 ? 4 : 1;
  const int oh = (hw + 2 * pad - k) / stride + 1;
  const size_t osz = out_type == f32 ? 4 : 1;

  FILE *f = fopen(in_path, "rb");
  if (!f) return 3;
  std::vector<uint8_t> x((size_t)n * ic * hw * hw * isz);
  std::vector<float> w((size_t)oc * (ic / g) * k * k), bias(up16(oc), 0.0f);
  std::vector<uint8_t> old((size_t)n * oc * oh * oh * osz);
  if (fread(x.data(), 1, x.size(), f) != x.size()) return 3;
  if (fread(w.data(), 4, w.size(), f) != w.size()) return 3;
  if (fread(bias.data(), 4, oc, f) != (size_t)oc) return 3;
  if (with_sum && fread(old.data(), 1, old.size(), f) != old.size()) return 3;
  fclose(f);

  eld_conv_t desc;
  desc.dims = {n, g, ic, oc, hw, hw, oh, oh, k, k};
  desc.pads = {pad, pad, pad, pad};
  desc.strides = {stride, stride};
  desc.dilations = {1, 1};
  desc.data_type.input = (uint8_t)in_type; desc.data_type.weights = f32; desc.data_type.output = (uint8_t)out_type; desc.data_type.bias = f32;
  desc.formats = {use_nhwc ? nhwc : nChw16c, g > 1 ? goihw : OIhw16i16o, use_nhwc ? nhwc : nChw16c};
  desc.algorithm = algorithm;
  desc.with_relu = true; desc.with_bias = true; desc.with_ip_sum = with_sum != 0;
  desc.relu_bound.lower = 0.0f;
  desc.relu_bound.upper = out_type == s8 ? 127.0f : (g > 1 ? 255.0f : FLT_MAX);
  desc.flatting = {0, T};
  desc.input_quant = {in_type == f32 ? 1.0f : 1.0f / 255.0f, 0.0f};
  if (wino) {
    desc.tile_size = tile_size;
    desc.execution_mode = execution_mode;
    desc.wino_tinput_quant = {tinput_scale, tinput_z};
  }
  desc.output_quant = {out_scale, 0.0f};
  desc.sum_quant = {sum_scale, 0.0f};
  desc.sampling_kind = CALIBRATED;
  const int rc = desc.setup();
  if (rc != ELD_OK) {
    fprintf(stderr, "setup failed: %d\n", rc);
    return 4;
  }

  std::vector<uint8_t> xb(desc.byte_sizes.input), ob(desc.byte_sizes.output, 0x5a);
  std::vector<float> wb(desc.sizes.weights, 0.0f);
  if (use_nhwc && isz == 1) reorder<uint8_t, nhwc, nchw>(xb.data(), x.data(), n, ic, hw, hw);
  else if (use_nhwc) reorder<float, nhwc, nchw>((float *)xb.data(), (float *)x.data(), n, ic, hw, hw);
  else if (isz == 1) reorder<uint8_t, nChw16c, nchw>(xb.data(), x.data(), n, ic, hw, hw);
  else reorder<float, nChw16c, nchw>((float *)xb.data(), (float *)x.data(), n, ic, hw, hw);
  if (g > 1) memcpy(wb.data(), w.data(), w.size() * 4);   // depthwise weights stay goihw
  else reorder<float, OIhw16i16o, oihw>(wb.data(), w.data(), oc, ic, k, k);
  if (with_sum) {
    if (use_nhwc && osz == 1) reorder<uint8_t, nhwc, nchw>(ob.data(), old.data(), n, oc, oh, oh);
    else if (use_nhwc) reorder<float, nhwc, nchw>((float *)ob.data(), (float *)old.data(), n, oc, oh, oh);
    else if (osz == 1) reorder<uint8_t, nChw16c, nchw>(ob.data(), old.data(), n, oc, oh, oh);
    else reorder<float, nChw16c, nchw>((float *)ob.data(), (float *)old.data(), n, oc, oh, oh);
  }
  // first call prepares the weights; the second is the steady state (the sum operand is re-staged)
  std::vector<uint8_t> ob0 = ob;
  if (elx_conv(desc, ob.data(), xb.data(), wb.data(), bias.data()) != ELX_OK) return 5;
  ob = ob0;
  if (elx_conv(desc, ob.data(), xb.data(), wb.data(), bias.data()) != ELX_OK) return 5;
  if (getenv("EULER_CHECK_MANAGED_OUTPUT")) {
    // Eager mode (the descriptor's default) with the output in managed memory: the result must be complete when
    // elx_conv returns, as the reference's eager mode is (src/elx_conv.cpp:226-230).  The host reads it straight
    // after the call, with no synchronisation of its own, and that is what gets compared.
    uint8_t *ym = nullptr;
    if (hipMallocManaged(reinterpret_cast<void **>(&ym), ob.size()) != hipSuccess) return 8;
    memcpy(ym, ob0.data(), ob.size());
    if (elx_conv(desc, ym, xb.data(), wb.data(), bias.data()) != ELX_OK) return 5;
    memcpy(ob.data(), ym, ob.size());
    (void)hipFree(ym);
  }

  std::vector<uint8_t> out((size_t)n * oc * oh * oh * osz);
  if (use_nhwc && osz == 1) reorder<uint8_t, nchw, nhwc>(out.data(), ob.data(), n, oc, oh, oh);
  else if (use_nhwc) reorder<float, nchw, nhwc>((float *)out.data(), (float *)ob.data(), n, oc, oh, oh);
  else if (osz == 1) reorder<uint8_t, nchw, nChw16c>(out.data(), ob.data(), n, oc, oh, oh);
  else reorder<float, nchw, nChw16c>((float *)out.data(), (float *)ob.data(), n, oc, oh, oh);
  f = fopen(out_path, "wb");
  if (!f || fwrite(out.data(), 1, out.size(), f) != out.size()) return 6;
  fclose(f);
  // error path of the entry point: null pointers are refused with the reference's code
  if (elx_conv(desc, nullptr, xb.data(), wb.data(), bias.data()) != ELX_GENERAL_ERROR) return 7;
  printf("ok %zu bytes\n", out.size());
  return 0;
}
