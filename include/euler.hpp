// Public C++ surface of the MI355X build: the same names, enum values, descriptor fields (in
// the same order) and call sequence as Euler's include/euler.hpp, so that code written against
// the reference compiles and runs unchanged:
//
//     euler::eld_conv_t desc;  ...fill...  desc.setup();
//     euler::elx_conv(desc, output, input, weights, bias);
//
// Only the quantized (u8 x s8 -> s32) executors exist behind it: direct 1x1, direct 3x3,
// depthwise 3x3 and Winograd F(4x4,3x3) with the int8 GEMM.  Everything else makes setup()
// return ELD_UNIMPLEMENTED.  Pointers handed to elx_conv() may be host pointers (staged through
// device buffers owned by the descriptor, as a drop-in needs) or device pointers (used in place).
#ifndef EULER_MI355X_EULER_HPP
#define EULER_MI355X_EULER_HPP

#include <cfloat>
#include <cstddef>
#include <cstdint>
#include <string>
#include <tuple>

#define EULER_API __attribute__((visibility("default")))

namespace euler {

using float16 = short;
using bfloat16 = unsigned short;

// <input, weights, output, bias> element types of the user tensors
template <typename... Types> struct ConvTypes {
  static_assert(sizeof...(Types) == 4, "four types: input, weights, output, bias");
  using InputType = typename std::tuple_element<0, std::tuple<Types...>>::type;
  using WeightsType = typename std::tuple_element<1, std::tuple<Types...>>::type;
  using OutputType = typename std::tuple_element<2, std::tuple<Types...>>::type;
  using BiasType = typename std::tuple_element<3, std::tuple<Types...>>::type;
};

namespace conv {
using FP32 = ConvTypes<float, float, float, float>;
using FP16 = ConvTypes<float16, float16, float16, float16>;
using FP16O = ConvTypes<float, float, float16, float>;
using U8S8F32F32 = ConvTypes<uint8_t, int8_t, float, float>;
using U8F32F32F32 = ConvTypes<uint8_t, float, float, float>;
using U8F32U8F32 = ConvTypes<uint8_t, float, uint8_t, float>;
using U8F32S8F32 = ConvTypes<uint8_t, float, int8_t, float>;
}  // namespace conv

// algorithm
enum { CONV_AUTO = 0, CONV_DIRECT_1X1 = 1, CONV_DIRECT = 2, CONV_DIRECT_VMG = 3, CONV_WINOGRAD = 4, DECONV_DIRECT = 5 };
// eld_conv_t::setup() result
enum { ELD_OK = 0, ELD_UNIMPLEMENTED = 1, ELD_GENERAL_ERROR = 2 };
// elx_conv() result
enum { ELX_OK = 0, ELX_UNIMPLEMENTED = 1, ELX_GENERAL_ERROR = 2 };
// streaming hint (accepted, ignored on the GPU)
enum { STORE_DEFAULT = 0, STORE_NORMAL = 1, STORE_STREAMING = 2 };
// element types
enum : uint8_t { data_type_undef = 0, f32 = 1, f16 = 2, u8 = 3, s8 = 4, s32 = 5 };
// tensor formats
enum {
  format_undef = 0, nchw = 1, nhwc = 2, nChw16c = 3, nChw8c = 4, oihw = 5, hwio = 6, OIhw16i16o = 7,
  OIhw8i8o = 8, goihw = 9, ghwio = 10, gOIhw16i16o = 11, gOIhw8i8o = 12
};
enum prop_kinds { forward_training = 0, forward_inference = 1, backward_data = 2, backward_weights = 3 };
typedef enum { FINE = 0, COARSE = 1, CALIBRATED = 2 } sampling_kind_t;

#define EL_NO_CALI (FLT_MAX)

struct elx_conv_t;  // the executor behind a descriptor (opaque)

struct EULER_API eld_conv_t {
  struct { int n, g, ic, oc, ih, iw, oh, ow, kh, kw; } dims;
  struct { int l, r, t, b; } pads;
  struct { int h, w; } strides;
  struct { int h, w; } dilations;

  struct {
    union {
      struct { uint8_t input, weights, output, bias; };
      uint32_t flat;
    };
  } data_type;

  // blocked: nChw16c / OIhw16i16o / nChw16c (depthwise weights: goihw)
  struct { int input, weights, output; } formats;

  int prop_kind;
  int algorithm;
  int tile_size;  // Winograd only: 4 = F(2x2,3x3), 5 = F(3x3,3x3), 6 = F(4x4,3x3); 0 = chosen by setup()

  bool with_relu;
  bool with_bias;
  bool with_ip_sum;
  bool with_op_sum;
  bool with_argmax;
  bool f16c_opt;
  bool is_inference;
  bool use_scratch_pad;
  bool disable_autoparam;
  bool eager_mode;
  bool stream_sync;
  struct { float lower = 0, upper = FLT_MAX; } relu_bound;

  int nthreads;
  int execution_mode;
  struct { int o, t; } flatting;
  struct { int i, o; } blocking;
  struct { int i, o, g; } partition;
  struct { int input, output; } streaming_hint;
  struct { bool input, weights, output; } format_as_blocked;

  // A_fp32 = scale * (A_quant - z)
  struct { float scale, z; } input_quant, wino_tinput_quant, output_quant, sum_quant;
  sampling_kind_t sampling_kind;

  void *scratch_pad;
  std::string name;

  eld_conv_t();
  ~eld_conv_t();
  eld_conv_t(const eld_conv_t &) = delete;
  eld_conv_t &operator=(const eld_conv_t &) = delete;
  int setup(bool fully_setup = true);

  // filled by setup()
  struct { size_t input, weights, output, bias; } byte_sizes;
  struct { size_t input, weights, output, bias; } sizes;

  elx_conv_t *xc;
};

int EULER_API elx_conv(eld_conv_t &desc, void *output, void *input, void *weights, void *bias);

}  // namespace euler

#endif
