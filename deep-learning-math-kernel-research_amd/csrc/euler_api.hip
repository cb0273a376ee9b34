// The C++ `euler::` API (include/euler.hpp, include/euler_reorder.hpp) on top of the C-ABI.
//
//   eld_conv_t::eld_conv_t / setup  <- src/eld_conv.cpp:21-316 (defaults, sizes, dispatch)
//   elx_conv                        <- src/elx_conv.cpp:213-240 (argument check, eager execute)
//   reorder<T,dst,src>              <- src/elx_reorder.cpp:11-232 (host-side index maps)
//
// Errors: where the reference prints and abort()s, setup() returns ELD_UNIMPLEMENTED /
// ELD_GENERAL_ERROR with the same code values; the message is available from ehip_last_error().
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <thread>
#include <vector>

#include "euler.hpp"
#include "euler_reorder.hpp"
#include "euler_hip.h"

namespace euler {

// what a descriptor owns: the C-ABI handle plus device staging buffers for host-pointer callers
struct elx_conv_t {
  ehip_conv_t *handle = nullptr;
  void *d_input = nullptr, *d_weights = nullptr, *d_output = nullptr, *d_bias = nullptr;
  const void *weights_seen = nullptr;
  ~elx_conv_t()
  {
    if (handle) ehip_conv_destroy(handle);
    void *p[] = {d_input, d_weights, d_output, d_bias};
    for (void *q : p)
      if (q) (void)hipFree(q);
  }
};

namespace {

inline size_t alignup16(size_t x) { return (x + 15) / 16 * 16; }

bool is_device_pointer(const void *p)
{
  hipPointerAttribute_t attr;
  hipError_t e = hipPointerGetAttributes(&attr, p);
  if (e != hipSuccess) {
    (void)hipGetLastError();  // plain host memory: clear the sticky error
    return false;
  }
  return attr.type == hipMemoryTypeDevice || attr.type == hipMemoryTypeManaged;
}

size_t elem_size(uint8_t dt)
{
  switch (dt) {
  case f32: return 4;
  case f16: return 2;
  case u8:
  case s8: return 1;
  case s32: return 4;
  default: return 0;
  }
}

// stage a host buffer into a lazily allocated device buffer; device pointers pass through
bool stage_in(const void *user, void **dev_buf, size_t bytes, const void **out)
{
  if (is_device_pointer(user)) {
    *out = user;
    return true;
  }
  if (!*dev_buf && hipMalloc(dev_buf, bytes) != hipSuccess) return false;
  if (hipMemcpy(*dev_buf, user, bytes, hipMemcpyHostToDevice) != hipSuccess) return false;
  *out = *dev_buf;
  return true;
}

}  // namespace

eld_conv_t::eld_conv_t()
{
  // the reference leaves several fields unset (src/eld_conv.cpp:21-50); they are given inert
  // values here so that a descriptor filled the reference's way behaves the same
  memset(&dims, 0, sizeof(dims));
  dims.g = 1;
  pads = {1, 1, 1, 1};
  strides = {1, 1};
  dilations = {1, 1};
  data_type.flat = 0;
  formats = {format_undef, format_undef, format_undef};
  prop_kind = forward_inference;
  algorithm = CONV_DIRECT;
  tile_size = 0;
  with_relu = with_bias = with_ip_sum = with_op_sum = with_argmax = false;
  f16c_opt = false;
  is_inference = true;
  use_scratch_pad = false;
  disable_autoparam = false;
  eager_mode = true;
  stream_sync = false;
  nthreads = 0;
  execution_mode = 0;
  flatting = {0, 0};
  blocking = {0, 0};
  partition = {1, 1, 1};
  streaming_hint = {0, 0};
  format_as_blocked = {false, false, false};
  input_quant = {EL_NO_CALI, EL_NO_CALI};
  wino_tinput_quant = {EL_NO_CALI, EL_NO_CALI};
  output_quant = {EL_NO_CALI, EL_NO_CALI};
  sum_quant = {0.0f, 0.0f};
  sampling_kind = FINE;
  scratch_pad = nullptr;
  name = "ioi";
  sizes = {0, 0, 0, 0};
  byte_sizes = {0, 0, 0, 0};
  xc = nullptr;
}

eld_conv_t::~eld_conv_t()
{
  delete xc;
  xc = nullptr;
}

int eld_conv_t::setup(bool fully_setup)
{
  const int V = 16;
  const int g = dims.g;
  if (g <= 0 || dims.ic % g != 0 || dims.oc % g != 0) return ELD_GENERAL_ERROR;
  const int icg = dims.ic / g, ocg = dims.oc / g;

  if (formats.input == format_undef) formats.input = (g == 1 && icg < V) ? nchw : nChw16c;
  if (formats.weights == format_undef) formats.weights = g == 1 ? hwio : ghwio;
  if (formats.output == format_undef) formats.output = nChw16c;

  const bool in_blocked = formats.input == nChw16c, out_blocked = formats.output == nChw16c;
  const bool w_blocked = formats.weights == OIhw16i16o || formats.weights == gOIhw16i16o;
  sizes.input = (size_t)dims.n * dims.ih * dims.iw * (in_blocked ? alignup16(dims.ic) : (size_t)dims.ic);
  // "+ 4 * V": the reference over-allocates the weights for its software pipeline (src/eld_conv.cpp:102-105)
  sizes.weights = (size_t)dims.g * dims.kh * dims.kw *
      (w_blocked ? alignup16(icg) * alignup16(ocg) : (size_t)ocg * icg) + 4 * V;
  sizes.output = (size_t)dims.n * dims.oh * dims.ow * (out_blocked ? alignup16(dims.oc) : (size_t)dims.oc);
  sizes.bias = out_blocked ? alignup16(dims.oc) : (size_t)dims.oc;
  byte_sizes.input = elem_size(data_type.input) * sizes.input;
  byte_sizes.weights = elem_size(data_type.weights) * sizes.weights;
  byte_sizes.output = elem_size(data_type.output) * sizes.output;
  byte_sizes.bias = elem_size(data_type.bias) * sizes.bias;

  const int oh = (dims.ih + pads.t + pads.b - dims.kh) / strides.h + 1;
  const int ow = (dims.iw + pads.l + pads.r - dims.kw) / strides.w + 1;
  if (oh != dims.oh || ow != dims.ow)
    fprintf(stderr, "euler: Padding parameter error. pads.r/pads.b will be auto adjusted\n");

  delete xc;
  xc = nullptr;
  if (prop_kind != forward_inference) return ELD_GENERAL_ERROR;

  if (algorithm == CONV_AUTO) {
    if (dims.kh == 1 && dims.kw == 1) algorithm = CONV_DIRECT_1X1;
    else if (icg >= V && dims.kh == 3 && dims.kw == 3 && dilations.h == 1 && dilations.w == 1 && strides.h == 1 &&
             strides.w == 1 && pads.l == 1 && pads.r == 1 && pads.t == 1 && pads.b == 1)
      algorithm = CONV_WINOGRAD;
    else algorithm = CONV_DIRECT;
  }
  if (!fully_setup) return ELD_OK;

  ehip_conv_desc_t d;
  memset(&d, 0, sizeof(d));
  d.n = dims.n; d.g = dims.g; d.ic = dims.ic; d.oc = dims.oc; d.ih = dims.ih; d.iw = dims.iw;
  d.oh = dims.oh; d.ow = dims.ow; d.kh = dims.kh; d.kw = dims.kw;
  d.pad_l = pads.l; d.pad_r = pads.r; d.pad_t = pads.t; d.pad_b = pads.b;
  d.stride_h = strides.h; d.stride_w = strides.w; d.dilation_h = dilations.h; d.dilation_w = dilations.w;
  d.input_type = data_type.input; d.weights_type = data_type.weights;
  d.output_type = data_type.output; d.bias_type = data_type.bias;
  d.input_fmt = formats.input; d.weights_fmt = formats.weights; d.output_fmt = formats.output;
  d.algorithm = algorithm; d.tile_size = tile_size; d.execution_mode = execution_mode;
  d.with_relu = with_relu; d.with_bias = with_bias; d.with_ip_sum = with_ip_sum;
  d.flatting_o = flatting.o; d.flatting_t = flatting.t;
  d.sampling_kind = sampling_kind;
  d.input_scale = input_quant.scale; d.input_z = input_quant.z;
  d.tinput_scale = wino_tinput_quant.scale; d.tinput_z = wino_tinput_quant.z;
  d.output_scale = output_quant.scale; d.output_z = output_quant.z;
  d.sum_scale = sum_quant.scale; d.sum_z = sum_quant.z;
  d.relu_lower = relu_bound.lower; d.relu_upper = relu_bound.upper;
  if (with_op_sum || with_argmax) return ELD_UNIMPLEMENTED;
  if (algorithm == CONV_WINOGRAD && tile_size == 0) {
    // the reference's choice between F(4x4,3x3) and F(2x2,3x3), written back like there (src/eld_conv.cpp:231-236)
    const int t = dims.n * ((dims.oh + 3) / 4) * ((dims.ow + 3) / 4);
    const int ocp = (dims.oc + 15) / 16 * 16;
    const float mac_per_read = (float)((double)t * ocp) / (float)(t + ocp);
    d.tile_size = tile_size = mac_per_read > 25.0f ? 6 : 4;
  }

  ehip_conv_t *h = nullptr;
  const int rc = ehip_conv_create(&d, &h);
  if (rc != EHIP_OK) {
    fprintf(stderr, "euler: setup: %s\n", ehip_last_error());
    return rc == EHIP_UNIMPLEMENTED ? ELD_UNIMPLEMENTED : ELD_GENERAL_ERROR;
  }
  xc = new elx_conv_t();
  xc->handle = h;
  return ELD_OK;
}

int elx_conv(eld_conv_t &desc, void *output, void *input, void *weights, void *bias)
{
  elx_conv_t *xc = desc.xc;
  if (input == nullptr || weights == nullptr || output == nullptr || (desc.with_bias && bias == nullptr) ||
      xc == nullptr || xc->handle == nullptr) {
    fprintf(stderr, "euler: Parameter error. Invalid input data!\n");
    return ELX_GENERAL_ERROR;
  }
  const void *din = nullptr, *dw = nullptr, *db = nullptr;
  if (!stage_in(input, &xc->d_input, desc.byte_sizes.input, &din)) return ELX_GENERAL_ERROR;
  // weights and bias are consumed once (first run), like the reference's is_first_run_
  if (xc->weights_seen != weights) {
    if (!stage_in(weights, &xc->d_weights, desc.byte_sizes.weights, &dw)) return ELX_GENERAL_ERROR;
    if (bias && !stage_in(bias, &xc->d_bias, desc.byte_sizes.bias, &db)) return ELX_GENERAL_ERROR;
    if (xc->weights_seen == nullptr) {
      if (ehip_conv_prepare(xc->handle, dw, db, nullptr) != EHIP_OK) return ELX_GENERAL_ERROR;
    }
    xc->weights_seen = weights;
  } else {
    db = xc->d_bias ? xc->d_bias : bias;
  }
  void *dout = output;
  const bool out_on_device = is_device_pointer(output);
  if (!out_on_device) {
    if (!xc->d_output && hipMalloc(&xc->d_output, desc.byte_sizes.output) != hipSuccess) return ELX_GENERAL_ERROR;
    dout = xc->d_output;
    if (desc.with_ip_sum &&
        hipMemcpy(dout, output, desc.byte_sizes.output, hipMemcpyHostToDevice) != hipSuccess)
      return ELX_GENERAL_ERROR;
  }
  const int rc = ehip_conv_execute(xc->handle, dout, din, nullptr, db, nullptr);
  if (rc != EHIP_OK) {
    fprintf(stderr, "euler: execute: %s\n", ehip_last_error());
    return rc == EHIP_UNIMPLEMENTED ? ELX_UNIMPLEMENTED : ELX_GENERAL_ERROR;
  }
  if (!out_on_device) {
    if (hipMemcpy(output, dout, desc.byte_sizes.output, hipMemcpyDeviceToHost) != hipSuccess) return ELX_GENERAL_ERROR;
  } else if (desc.eager_mode || desc.stream_sync) {
    // Device or managed tensors.  Eager mode (the descriptor's default) returns with the result complete, as the
    // reference's does (src/elx_conv.cpp:226-230): a host that reads a managed output, or a consumer on a
    // non-blocking stream, may use it straight away.  A caller that chains layers on the device asks for the
    // reference's stream mode instead (eager_mode = false): the layer is then only ordered on the NULL stream,
    // like every later kernel or copy that touches its tensors, and stream_sync adds the wait
    // (src/elx_conv.cpp:231-236).
    if (hipStreamSynchronize(nullptr) != hipSuccess) return ELX_GENERAL_ERROR;
  }
  return ELX_OK;
}

// ---- reorders (host memory) --------------------------------------------------------------------
// The reference spreads every reorder over its thread pool (src/elx_reorder.cpp:35-93, estl::parallel_for
// over the outer dimensions).  Here the outermost loop of each reorder is cut into contiguous ranges, one
// per host thread; OMP_NUM_THREADS caps the thread count as it does the reference's, and a tensor of a few
// thousand elements stays on the calling thread.
namespace {
int reorder_threads(size_t rows, size_t elements)
{
  size_t t = std::thread::hardware_concurrency();
  if (const char *e = getenv("OMP_NUM_THREADS")) {
    const long v = strtol(e, nullptr, 10);
    if (v > 0) t = (size_t)v;
  }
  t = std::min(t, rows);
  t = std::min(t, elements / 32768 + 1);
  return (int)std::max<size_t>(t, 1);
}

// fn(first_row, last_row) over [0, rows), ranges of nearly equal length on separate threads
template <typename F> void parallel_rows(size_t rows, size_t elements, F fn)
{
  const int nt = reorder_threads(rows, elements);
  if (nt <= 1) {
    fn((size_t)0, rows);
    return;
  }
  std::vector<std::thread> pool;
  pool.reserve(nt - 1);
  for (int t = 1; t < nt; ++t) pool.emplace_back(fn, rows * t / nt, rows * (t + 1) / nt);
  fn((size_t)0, rows / nt);
  for (auto &th : pool) th.join();
}
}  // namespace

template <typename Type> reorder<Type, nchw, nhwc>::reorder(Type *dst, Type *src, int n, int c, int h, int w)
{
  const size_t hw = (size_t)h * w;
  parallel_rows((size_t)n * c, (size_t)n * c * hw, [=](size_t r0, size_t r1) {
    for (size_t r = r0; r < r1; ++r) {
      const size_t _n = r / c, _c = r % c;
      Type *d = dst + r * hw;
      const Type *s = src + _n * hw * c + _c;
      for (size_t p = 0; p < hw; ++p) d[p] = s[p * c];
    }
  });
}

template <typename Type> reorder<Type, nhwc, nchw>::reorder(Type *dst, Type *src, int n, int c, int h, int w)
{
  const size_t hw = (size_t)h * w;
  parallel_rows((size_t)n * h, (size_t)n * c * hw, [=](size_t r0, size_t r1) {
    for (size_t r = r0; r < r1; ++r) {
      const size_t _n = r / h, _h = r % h;
      for (int _w = 0; _w < w; ++_w) {
        Type *d = dst + (r * w + _w) * c;
        const Type *s = src + _n * c * hw + _h * w + _w;
        for (int _c = 0; _c < c; ++_c) d[_c] = s[_c * hw];
      }
    }
  });
}

template <typename Type> reorder<Type, nchw, nChw16c>::reorder(Type *dst, Type *src, int n, int c, int h, int w)
{
  const size_t hw = (size_t)h * w, C2 = ((size_t)c + 15) / 16;
  parallel_rows((size_t)n * c, (size_t)n * c * hw, [=](size_t r0, size_t r1) {
    for (size_t r = r0; r < r1; ++r) {
      const size_t _n = r / c, ch = r % c;
      Type *d = dst + r * hw;
      const Type *s = src + (_n * C2 + ch / 16) * hw * 16 + ch % 16;
      for (size_t p = 0; p < hw; ++p) d[p] = s[p * 16];
    }
  });
}

template <typename Type> reorder<Type, nChw16c, nchw>::reorder(Type *dst, Type *src, int n, int c, int h, int w)
{
  const size_t hw = (size_t)h * w, C2 = ((size_t)c + 15) / 16;
  parallel_rows((size_t)n * C2, (size_t)n * C2 * 16 * hw, [=](size_t r0, size_t r1) {
    for (size_t r = r0; r < r1; ++r) {
      const size_t _n = r / C2, c2 = r % C2;
      const int real = (int)std::min<size_t>(16, c - c2 * 16);   // the last unit's tail is zero-filled
      Type *d = dst + r * hw * 16;
      const Type *s = src + (_n * c + c2 * 16) * hw;
      for (size_t p = 0; p < hw; ++p)
        for (int v = 0; v < 16; ++v) d[p * 16 + v] = v < real ? s[v * hw + p] : (Type)0;
    }
  });
}

namespace {
template <typename Type> void plain_to_blocked_weights(Type *dst, Type *src, int g, int o, int i, int h, int w)
{
  const size_t O2 = ((size_t)o + 15) / 16, I2 = ((size_t)i + 15) / 16, hw = (size_t)h * w;
  parallel_rows((size_t)g * O2 * I2, (size_t)g * O2 * I2 * hw * 256, [=](size_t r0, size_t r1) {
    for (size_t r = r0; r < r1; ++r) {
      const size_t _g = r / (O2 * I2), o2 = r / I2 % O2, i2 = r % I2;
      for (size_t p = 0; p < hw; ++p)
        for (int iv = 0; iv < 16; ++iv)
          for (int ov = 0; ov < 16; ++ov) {
            const size_t oc = o2 * 16 + ov, ic = i2 * 16 + iv;
            dst[((r * hw + p) * 16 + iv) * 16 + ov] =
                (oc < (size_t)o && ic < (size_t)i) ? src[((_g * o + oc) * i + ic) * hw + p] : (Type)0;
          }
    }
  });
}
template <typename Type> void blocked_to_plain_weights(Type *dst, Type *src, int g, int o, int i, int h, int w)
{
  const size_t O2 = ((size_t)o + 15) / 16, I2 = ((size_t)i + 15) / 16, hw = (size_t)h * w;
  parallel_rows((size_t)g * o, (size_t)g * o * i * hw, [=](size_t r0, size_t r1) {
    for (size_t r = r0; r < r1; ++r) {
      const size_t _g = r / o, oc = r % o;
      for (size_t ic = 0; ic < (size_t)i; ++ic)
        for (size_t p = 0; p < hw; ++p)
          dst[(r * i + ic) * hw + p] =
              src[((((_g * O2 + oc / 16) * I2 + ic / 16) * hw + p) * 16 + ic % 16) * 16 + oc % 16];
    }
  });
}
template <typename Type> void hwio_to_oihw(Type *dst, Type *src, int g, int o, int i, int h, int w)
{
  const size_t hw = (size_t)h * w;
  parallel_rows((size_t)g * o, (size_t)g * o * i * hw, [=](size_t r0, size_t r1) {
    for (size_t r = r0; r < r1; ++r) {
      const size_t _g = r / o, oc = r % o;
      for (size_t ic = 0; ic < (size_t)i; ++ic)
        for (size_t p = 0; p < hw; ++p) dst[(r * i + ic) * hw + p] = src[((_g * hw + p) * i + ic) * o + oc];
    }
  });
}
template <typename Type> void oihw_to_hwio(Type *dst, Type *src, int g, int o, int i, int h, int w)
{
  const size_t hw = (size_t)h * w;
  parallel_rows((size_t)g * hw, (size_t)g * o * i * hw, [=](size_t r0, size_t r1) {
    for (size_t r = r0; r < r1; ++r) {
      const size_t _g = r / hw, p = r % hw;
      for (size_t ic = 0; ic < (size_t)i; ++ic)
        for (size_t oc = 0; oc < (size_t)o; ++oc) dst[(r * i + ic) * o + oc] = src[((_g * o + oc) * i + ic) * hw + p];
    }
  });
}
}  // namespace

template <typename Type> reorder<Type, OIhw16i16o, oihw>::reorder(Type *dst, Type *src, int o, int i, int h, int w)
{
  plain_to_blocked_weights(dst, src, 1, o, i, h, w);
}
template <typename Type> reorder<Type, oihw, OIhw16i16o>::reorder(Type *dst, Type *src, int o, int i, int h, int w)
{
  blocked_to_plain_weights(dst, src, 1, o, i, h, w);
}
template <typename Type>
reorder<Type, gOIhw16i16o, goihw>::reorder(Type *dst, Type *src, int g, int o, int i, int h, int w)
{
  plain_to_blocked_weights(dst, src, g, o, i, h, w);
}
template <typename Type>
reorder<Type, goihw, gOIhw16i16o>::reorder(Type *dst, Type *src, int g, int o, int i, int h, int w)
{
  blocked_to_plain_weights(dst, src, g, o, i, h, w);
}
template <typename Type> reorder<Type, oihw, hwio>::reorder(Type *dst, Type *src, int o, int i, int h, int w)
{
  hwio_to_oihw(dst, src, 1, o, i, h, w);
}
template <typename Type> reorder<Type, hwio, oihw>::reorder(Type *dst, Type *src, int o, int i, int h, int w)
{
  oihw_to_hwio(dst, src, 1, o, i, h, w);
}
template <typename Type> reorder<Type, goihw, ghwio>::reorder(Type *dst, Type *src, int g, int o, int i, int h, int w)
{
  hwio_to_oihw(dst, src, g, o, i, h, w);
}
template <typename Type> reorder<Type, ghwio, goihw>::reorder(Type *dst, Type *src, int g, int o, int i, int h, int w)
{
  oihw_to_hwio(dst, src, g, o, i, h, w);
}

#define INSTANTIATE(T)                                                                              \
  template struct reorder<T, nchw, nhwc>;                                                           \
  template struct reorder<T, nhwc, nchw>;                                                           \
  template struct reorder<T, nchw, nChw16c>;                                                        \
  template struct reorder<T, nChw16c, nchw>;                                                        \
  template struct reorder<T, OIhw16i16o, oihw>;                                                     \
  template struct reorder<T, oihw, OIhw16i16o>;                                                     \
  template struct reorder<T, gOIhw16i16o, goihw>;                                                   \
  template struct reorder<T, goihw, gOIhw16i16o>;                                                   \
  template struct reorder<T, oihw, hwio>;                                                           \
  template struct reorder<T, hwio, oihw>;                                                           \
  template struct reorder<T, goihw, ghwio>;                                                         \
  template struct reorder<T, ghwio, goihw>;
INSTANTIATE(float)
INSTANTIATE(uint8_t)
#undef INSTANTIATE

}  // namespace euler
