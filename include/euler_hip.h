/*
 * C-ABI of the MI355X (gfx950) implementation of Euler's int8 convolution path.
 *
 * This is the boundary a host-language binding (the C++ `euler::` API in euler.hpp, a ctypes /
 * cgo / JNI stub ...) talks to: plain pointers, sizes and PODs, no C++ or torch types.  Every
 * pointer named *_dev is a DEVICE pointer; the caller owns input/weights/bias/output, the
 * handle owns its workspace (packed s8 weights, per-channel scale/shift, Winograd
 * intermediates).  All functions return EHIP_OK (0) or an EHIP_* error code and never abort;
 * ehip_last_error() gives the text of the calling thread's last failure.
 *
 * Enum values are the reference's (include/euler.hpp:35-103) so that a descriptor can be
 * copied field by field.
 */
#ifndef EULER_HIP_H
#define EULER_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define EHIP_API __attribute__((visibility("default")))

/* status codes: 0/1/2 match ELD_OK / ELD_UNIMPLEMENTED / ELD_GENERAL_ERROR and the ELX_* trio
 * (include/euler.hpp:44-56) */
enum { EHIP_OK = 0, EHIP_UNIMPLEMENTED = 1, EHIP_GENERAL_ERROR = 2, EHIP_HIP_ERROR = 3 };

/* data types (include/euler.hpp:66-73) */
enum { EHIP_DT_UNDEF = 0, EHIP_F32 = 1, EHIP_F16 = 2, EHIP_U8 = 3, EHIP_S8 = 4, EHIP_S32 = 5 };

/* algorithms (include/euler.hpp:35-42) */
enum { EHIP_CONV_AUTO = 0, EHIP_CONV_DIRECT_1X1 = 1, EHIP_CONV_DIRECT = 2, EHIP_CONV_WINOGRAD = 4 };

/* formats (include/euler.hpp:75-89) */
enum {
  EHIP_FMT_UNDEF = 0, EHIP_NCHW = 1, EHIP_NHWC = 2, EHIP_NCHW16C = 3, EHIP_OIHW = 5,
  EHIP_OIHW16I16O = 7, EHIP_GOIHW = 9
};

/* The fields of eld_conv_t (include/euler.hpp:110-172) that the int8 path reads, as a POD.
 * output_type EHIP_S32 is an extension: the raw s32 accumulators are written instead of the
 * requantized result (used to check the contraction on its own). */
typedef struct ehip_conv_desc {
  int32_t n, g, ic, oc, ih, iw, oh, ow, kh, kw;      /* dims                     */
  int32_t pad_l, pad_r, pad_t, pad_b;                /* pads                     */
  int32_t stride_h, stride_w, dilation_h, dilation_w;
  int32_t input_type, weights_type, output_type, bias_type;
  int32_t input_fmt, weights_fmt, output_fmt;
  int32_t algorithm, tile_size, execution_mode;
  int32_t with_relu, with_bias, with_ip_sum;
  int32_t flatting_o, flatting_t;                    /* flatting.{o,t}: t is the width block T;
                                                        only the depthwise u8 store depends on it */
  int32_t sampling_kind;                             /* must be CALIBRATED (2)   */
  float input_scale, input_z;                        /* input_quant              */
  float tinput_scale, tinput_z;                      /* wino_tinput_quant        */
  float output_scale, output_z;                      /* output_quant             */
  float sum_scale, sum_z;                            /* sum_quant                */
  float relu_lower, relu_upper;                      /* relu_bound               */
} ehip_conv_desc_t;

typedef struct ehip_conv ehip_conv_t;

/* what ehip_conv_query copies out (host buffers, canonical plain layouts) */
enum {
  EHIP_Q_WEIGHTS_S8 = 1,   /* direct: [OCp][ICp][kh][kw]; depthwise: [G][3][3]; winograd: [36][OCp][ICp] */
  EHIP_Q_SCALE = 2,        /* f32 [OCp] (winograd [36][OCp])                                            */
  EHIP_Q_SHIFT = 3,        /* f32, same shape                                                           */
  EHIP_Q_WSUM = 4,         /* s32, same shape: sum of the quantized weights                              */
  EHIP_Q_TINPUT_U8 = 5,    /* winograd: transformed+quantized input of the last execute [36][ICp/16][t][16] */
  EHIP_Q_TOUTPUT_F32 = 6   /* winograd: GEMM result of the last execute [36][OCp/16][t][16]             */
};

/* Binds the calling thread to `device` and checks that it is a gfx950.  Optional: the other
 * entry points use the current device. */
EHIP_API int ehip_init(int device);
EHIP_API const char *ehip_last_error(void);

/* Replaces eld_conv_t::setup(): validates the descriptor, picks the executor
 * (src/eld_conv.cpp:166-313: direct 1x1 / direct KxK / depthwise / Winograd F(4,3) int8) and
 * allocates the device workspace.  Unsupported shapes return EHIP_UNIMPLEMENTED where the
 * reference calls el_error()/abort().  What is accepted:
 *  - CONV_DIRECT_1X1 (src/elx_int8_conv_direct_1x1.cpp): u8 input, u8/s8/s32 output, stride 1 or 2,
 *    no padding, sum fusion; activations nChw16c or nhwc on either side (nhwc: channels % 16 == 0);
 *  - CONV_DIRECT with a 1x1 kernel (a160, src/elx_int8_conv_direct.cpp:574-718): also f32 output;
 *  - CONV_DIRECT with a 3/5/7 kernel (c160, src/elx_int8_conv_direct.cpp:66-77): stride 1 or 2, every
 *    pad k/2 or k/2 - 1 (right/bottom pads follow from oh/ow), ow % flatting_t == 0; nChw16c or nhwc on
 *    either side (nhwc: channels % 16 == 0, except that a layer with at most 4 input channels -- a
 *    network's first layer -- takes nhwc input of ic bytes per pixel at a 4-byte aligned address);
 *  - depthwise 3x3 (g == ic == oc, src/elx_int8_conv_direct_depthwise.cpp): stride 1 or 2, pads 0/1,
 *    u8/s8 output, weights goihw;
 *  - CONV_WINOGRAD tile_size 4, 5 or 6 (0: the reference's automatic choice; src/elx_int8_conv_wino.cpp, src/eld_conv.cpp:231-270): f32 tensors with execution_mode 0xa1xx, or
 *    u8 input with f32/u8/s8 output (U8F32F32F32 / U8F32U8F32 / U8F32S8F32, src/eld_conv.cpp:275-281);
 *    wino_tinput_quant must be set (calibrated sampling); with_ip_sum adds the old output (f32, or the
 *    u8 / s8 code, unscaled) before the ReLU as the reference's output transform does; activations
 *    nChw16c or nhwc on either side (nhwc: channels % 16 == 0).
 * A non-zero input zero point with padding is accepted by the 3/5/7 direct kernels (the shift then
 * depends on the output pixel's set of valid taps, src/elx_int8_conv_direct.cpp:227-423).  The depthwise
 * executor follows the reference: one shift of z times all nine weights, padded taps adding nothing
 * (src/elx_int8_conv_direct_depthwise.cpp:247-289); the Winograd executor uses the input scale only
 * (src/elx_conv_wino_trans_input.cpp:367-368) and, like the reference's setup, refuses u8 input with a
 * non-zero zero point (src/eld_conv.cpp:223-228). */
EHIP_API int ehip_conv_create(const ehip_conv_desc_t *desc, ehip_conv_t **out);
EHIP_API int ehip_conv_destroy(ehip_conv_t *conv);

/* Replaces the first-run branch of every executor (`is_first_run_`,
 * e.g. src/elx_int8_conv_direct_1x1_xopt.hpp:27-35): per-channel abs-max quantization of the f32
 * weights to s8, packing for the MFMA kernels, and folding of the quantization scales, bias and
 * zero points into one scale/shift pair per output channel
 * (src/elx_int8_conv_direct_1x1.cpp:234-355, src/elx_int8_conv_direct.cpp:311-500,
 *  src/elx_int8_conv_direct_depthwise.cpp:200-292, src/elx_conv_wino_trans_weights.cpp:437-553).
 * weights_dev: f32 OIhw16i16o (depthwise: goihw); bias_dev: f32 [OCp] or NULL. */
EHIP_API int ehip_conv_prepare(ehip_conv_t *conv, const void *weights_dev, const void *bias_dev,
                               void *hip_stream);

/* Replaces elx_conv_t::execute() (src/elx_conv.hpp:125, src/elx_conv.cpp:213-240) for the
 * steady state.  Asynchronous on `hip_stream` (NULL = the default stream).  With with_ip_sum the
 * output buffer also holds the sum operand.  If the handle has not been prepared yet,
 * weights_dev/bias_dev are used to do so first (the reference's lazy first run); afterwards
 * they are ignored and may be NULL. */
EHIP_API int ehip_conv_execute(ehip_conv_t *conv, void *output_dev, const void *input_dev,
                               const void *weights_dev, const void *bias_dev, void *hip_stream);

/* Steady-state driver: enqueues `count` back-to-back executions of a prepared handle on
 * `hip_stream` without returning to the caller in between (what the reference's benchmark loop
 * around elx_conv() does, tests/elt_conv.cpp:445-448).  No counterpart inside the library. */
EHIP_API int ehip_conv_execute_repeat(ehip_conv_t *conv, void *output_dev, const void *input_dev,
                                      const void *bias_dev, int count, void *hip_stream);

/* The stages of a Winograd layer on their own, `count` times back to back: what the reference runs as three
 * objects of its own, elx_conv_wino_trans_input_t::execute (src/elx_conv_wino_trans_input.cpp:599-654),
 * elx_int8_conv_wino_gemm_t::execute (src/elx_int8_conv_wino_gemm.cpp:23-205) and
 * elx_conv_wino_trans_output_t::execute (src/elx_conv_wino_trans_output.cpp:212-423), called one after the other by
 * the executor (src/elx_int8_conv_wino_xopt.hpp:70-121).  `stages` is a mask: 1 = input transform into the
 * handle's transformed-input buffer, 2 = the A x A GEMMs (in the fused schedule together with the output
 * transform, into output_dev), 4 = the stand-alone output transform (three-kernel schedule only).  A stage reads
 * what an earlier call's stage left in the handle's buffers.  For stage-level measurements and tests. */
EHIP_API int ehip_conv_execute_stages(ehip_conv_t *conv, void *output_dev, const void *input_dev, const void *bias_dev,
                                      int stages, int count, void *hip_stream);

/* Copies workspace contents to a host buffer in a canonical layout (see EHIP_Q_*).  Synchronous.
 * Returns the number of bytes through *bytes when host_dst is NULL. */
EHIP_API int ehip_conv_query(ehip_conv_t *conv, int what, void *host_dst, size_t *bytes);

/* Name of the kernel variant execute() launches (for profiles), and its launch geometry.  Where the launcher chooses
 * between forms of a kernel (epilogue forms, the fused Winograd stage), the name is final after the first execute. */
EHIP_API const char *ehip_conv_kernel_name(ehip_conv_t *conv);

/* Replaces the harness-side fp32 -> u8 activation quantization
 * (tests/elt_conv_utils.cpp:354-401): dst = (uint8_t) round(src / scale + z) with that helper's
 * tie rule. */
EHIP_API int ehip_quantize_input_u8(void *dst_dev, const void *src_dev, size_t count, float scale,
                                    float z, void *hip_stream);

/* Replaces the harness-side calibration of wino_tinput_quant (tests/elt_conv_utils.cpp:222-262):
 * min and max over the fp32 Winograd-transformed input.  u8 input: over the transformed CODES
 * (multiply by the input scale for real units).  Synchronous. */
EHIP_API int ehip_wino_tinput_range(const ehip_conv_desc_t *desc, const void *input_dev,
                                    float *min_out, float *max_out);

/* Replaces the harness's fp32 reference convolution where it serves calibration (ref_convolution2d,
 * tests/elt_conv_utils.cpp:666-750, called from :300-304): every output starts from the bias (plus the old
 * output with with_ip_sum), takes the products in the order (ic, kh, kw) with padded taps skipped, one
 * fused multiply-add each, and is clamped at zero with with_relu.  All tensors fp32: input and output in
 * the descriptor's activation formats (nChw16c or nhwc), weights OIhw16i16o (g = 1), oihw or goihw.
 * output_f32_dev may be NULL when only the range is wanted (it must be given with with_ip_sum: it holds
 * the sum operand on entry).  *min_out / *max_out: range of the result, over real channels only.
 * Synchronous, allocates a temporary. */
EHIP_API int ehip_ref_conv_f32_range(const ehip_conv_desc_t *desc, void *output_f32_dev, const void *input_f32_dev,
                                     const void *weights_dev, const void *bias_dev, float *min_out, float *max_out);

/* Replaces the harness's rule for output_quant and sum_quant (tests/elt_conv_utils.cpp:306-346), host
 * arithmetic only.  out_min / out_max: range of the fp32 reference output; sum_absmax: largest magnitude
 * of the fp32 sum operand (read only with with_ip_sum).  With ReLU or an s8 output:
 * scale = max(|min|, |max|) / representation, z = 0; otherwise scale = (max - min + 1e-6) / representation,
 * z = -min * representation / (max - min + 1e-6).  sum_scale = (sum_absmax / representation) / scale.
 * `representation` is the code range the scales map onto: the harness uses 127 for every type
 * (PRECISION_REPRESENTATION_7B); 255 uses the whole range of a u8 tensor. */
EHIP_API int ehip_calibrate_output_quant(const ehip_conv_desc_t *desc, float out_min, float out_max, float sum_absmax,
                                         float representation, float *output_scale, float *output_z, float *sum_scale);

/* No counterpart in the reference.  ehip_wino_tinput_range for callers that cannot allocate device
 * memory (a stream under HIP graph capture, a serving loop or a harness that forbids hipMalloc): the
 * per-unit partial minima / maxima go to a static device array of the library (32 KB on every GPU the
 * library runs on, held until the process ends) instead of to memory from hipMalloc, the result goes to
 * minmax_out_dev[0] = min, [1] = max (two floats of DEVICE memory owned by the caller), and the three
 * kernels are enqueued on `hip_stream` without a synchronisation.  Calls no hipMalloc / hipFree.
 * Limit: at most 65536 input channels (4096 units of 16), else EHIP_UNIMPLEMENTED.  All calls on one
 * GPU share that GPU's array: calls that overlap in time on one GPU (two streams, two threads) race;
 * calls on one stream are safe, each one re-initialises what it uses.  ehip_init(device) resolves the
 * array's address for the device ahead of the first call (otherwise the first call does). */
EHIP_API int ehip_wino_tinput_range_noalloc(const ehip_conv_desc_t *desc, const void *input_dev,
                                            float *minmax_out_dev, void *hip_stream);

/* Device-side layout reorders with the index maps of src/elx_reorder.cpp:35-93
 * (elem_size 1 or 4).  nchw <-> nChw16c and oihw -> OIhw16i16o; channel tails are zero-filled. */
EHIP_API int ehip_reorder_nchw_to_blocked(void *dst_dev, const void *src_dev, int elem_size, int n,
                                          int c, int h, int w, void *hip_stream);
EHIP_API int ehip_reorder_blocked_to_nchw(void *dst_dev, const void *src_dev, int elem_size, int n,
                                          int c, int h, int w, void *hip_stream);
EHIP_API int ehip_reorder_oihw_to_blocked(void *dst_dev, const void *src_dev, int o, int i, int h,
                                          int w, void *hip_stream);

#ifdef __cplusplus
}
#endif
#endif /* EULER_HIP_H */
