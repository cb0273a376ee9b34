/*
 * TEST INFRASTRUCTURE ONLY.
 *
 * CPU restatement ("oracle") of the reference's quantized-convolution arithmetic.  Only the
 * tests, the smoke check and the benchmark's cpu_baseline leg may load it; the product
 * library never does.  Every function names the reference file:line it restates.
 *
 * Conventions
 *   - activations are nChw16c: [n][C/16][h][w][16]; user weights are OIhw16i16o f32:
 *     [OC/16][IC/16][kh][kw][16 ic][16 oc]; depthwise user weights are goihw f32 [g][kh][kw].
 *   - quantized weights leave the oracle in a plain order ([OCp][ICp][kh][kw] s8, OCp/ICp =
 *     channel counts rounded up to 16) so that they can be compared with any packed layout.
 *   - float glue is written with explicit fmaf() exactly where the reference's compiled code
 *     (g++ -O2, default -ffp-contract=fast) performs one fused rounding; this file is built
 *     with -ffp-contract=off so nothing else fuses.
 *
 * Pinning status (what checks each part; see tests/test_oracle_*.py, tests/test_golden.py):
 *   - fused-rounding pattern of the GEMM/conv/depthwise epilogues, depthwise floor/round split,
 *     unsigned saturation, Winograd tile transforms (tile sizes 4, 5, 6): pinned against the
 *     reference's own kernel templates compiled from /root/reference (oracle/ref_kernels.cpp).
 *   - Winograd glue -- tile gather and border handling, the quantization fma(V, in_S / tin_S, ceil(z)) ->
 *     unsigned conversion -> saturation, the calibration range, per-(position, oc) weight quantization,
 *     scale and shift: pinned against the reference's two transform translation units compiled from
 *     /root/reference (oracle/ref_wino_glue.cpp), including inputs searched so that a dropped fusion
 *     changes the code.
 *   - integer contractions: pinned by brute-force integer convolution in numpy.
 *   - direct / depthwise weight quantization (abs-max, (w*127)/absmax, round-half-even) and scale/shift
 *     folding with every zero point non-zero, and the per-pixel shift rows of a zero point with padding:
 *     the executors that hold these folds do not link without tables the reference's build generates, so
 *     they are pinned by an independent long-double evaluation of the contraction pattern their compiled
 *     objects hold (vfmadd bias*repS+z, vfnmadd of the zero-point term, unfused sum_z*sum_S), on data
 *     checked to tell that pattern from its neighbours.
 *   - reorders: closed-form index maps, pinned by numpy transposes.
 *   - harness (fp32 reference convolution, output / sum scale calibration, input quantization): pinned against
 *     the reference's own harness translation unit compiled from /root/reference (oracle/ref_harness.cpp).
 *   - not pinned by anything but the source: the ORDER of exact integer additions in the executors.
 */
#ifndef EULER_ORACLE_H
#define EULER_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* same numbering as the reference's data-type enum (include/euler.hpp:66-73) */
enum { ORC_F32 = 1, ORC_U8 = 3, ORC_S8 = 4, ORC_S32 = 5 };

typedef struct orc_conv_params {
  int32_t n, g, ic, oc, ih, iw, oh, ow, kh, kw;
  int32_t pad_t, pad_l, stride_h, stride_w;
  int32_t out_type;            /* ORC_F32 / ORC_U8 / ORC_S8 */
  int32_t with_bias, with_relu, with_sum;
  int32_t T;                   /* width-block size (flatting.t); only depthwise u8 output depends on it */
  float in_scale, in_z;        /* input_quant  */
  float out_scale, out_z;      /* output_quant */
  float sum_scale, sum_z;      /* sum_quant    */
  float tin_scale, tin_z;      /* wino_tinput_quant */
  float relu_lo, relu_hi;      /* relu_bound   */
  int32_t wino_tile;           /* Winograd tile size A: 0 or 6 = F(4x4,3x3), 4 = F(2x2,3x3), 5 = F(3x3,3x3) */
} orc_conv_params;

/* ---- layout reorders: src/elx_reorder.cpp:35-93 ---- */
void orc_reorder_nchw_to_blocked_f32(float *dst, const float *src, int n, int c, int h, int w);
void orc_reorder_nchw_to_blocked_u8(uint8_t *dst, const uint8_t *src, int n, int c, int h, int w);
void orc_reorder_blocked_to_nchw_f32(float *dst, const float *src, int n, int c, int h, int w);
void orc_reorder_blocked_to_nchw_u8(uint8_t *dst, const uint8_t *src, int n, int c, int h, int w);
void orc_reorder_oihw_to_blocked_f32(float *dst, const float *src, int o, int i, int h, int w);
void orc_reorder_blocked_to_oihw_f32(float *dst, const float *src, int o, int i, int h, int w);

/* ---- harness-side input quantization: tests/elt_conv_utils.cpp:354-401 ---- */
void orc_quantize_input_u8(uint8_t *dst, const float *src, size_t count, float scale, float z);

/* ---- harness: fp32 reference convolution and the calibration rule built on it ----
 * orc_ref_conv_f32: tests/elt_conv_utils.cpp:666-750 on plain tensors (input / output nchw, weights oihw, or
 * goihw [g][oc/g][ic/g][kh][kw] for g > 1): out = (old out +) bias, then += x * w over (ic, kh, kw) with
 * padded taps skipped, each step one fused multiply-add as the compiled harness has it, then ReLU.
 * `output` holds the sum operand on entry when p->with_sum.
 * orc_calibrate_output_quant: tests/elt_conv_utils.cpp:306-346 (see ehip_calibrate_output_quant). */
int orc_ref_conv_f32(const orc_conv_params *p, float *output, const float *input, const float *weights,
                     const float *bias);
void orc_calibrate_output_quant(int with_relu, int out_type, int with_sum, float out_min, float out_max,
                                float sum_absmax, float representation, float *output_scale, float *output_z,
                                float *sum_scale);

/* ---- direct 1x1 / KxK ----
 * weight quantization + scale/shift folding:
 *   src/elx_int8_conv_direct_1x1.cpp:234-355, src/elx_int8_conv_direct.cpp:311-500.
 * wq [OCp][ICp][kh][kw] s8, scale/shift [OCp] f32, wsum [OCp] s32. */
int orc_direct_prepare(const orc_conv_params *p, const float *w_blocked, const float *bias,
                       int8_t *wq, float *scale, float *shift, int32_t *wsum);
/* contraction + epilogue: src/kernel/elk_u8s8_gemm.hxx:168-266,269-406,
 * src/kernel/elk_u8s8_conv.hxx:190-252,679-901, src/elx_int8_conv_direct.cpp:574-718.
 * `output` is nChw16c of out_type and, with_sum, also holds the sum operand on entry.
 * `acc` (optional) receives the raw s32 accumulators, nChw16c. */
int orc_direct_execute(const orc_conv_params *p, const uint8_t *input, const int8_t *wq,
                       const float *scale, const float *shift, void *output, int32_t *acc);
/* input_z != 0 with padding (src/elx_int8_conv_direct.cpp:227-423): the shift of an output pixel
 * folds the weights of the taps that fall inside the image for that pixel.  shift_map [oh][ow][OCp]. */
int orc_direct_border_shifts(const orc_conv_params *p, const float *w_blocked, const float *bias,
                             float *shift_map);
int orc_direct_execute_border(const orc_conv_params *p, const uint8_t *input, const int8_t *wq,
                              const float *scale, const float *shift_map, void *output, int32_t *acc);

/* ---- depthwise 3x3 ----
 * src/elx_int8_conv_direct_depthwise.cpp:200-292; wq [G][3][3], scale/shift [G], G = g up to 16. */
int orc_depthwise_prepare(const orc_conv_params *p, const float *w_goihw, const float *bias,
                          int8_t *wq, float *scale, float *shift, int32_t *wsum);
/* src/kernel/elk_u8s8_depthwise_conv.hxx:219-286,288-474 */
int orc_depthwise_execute(const orc_conv_params *p, const uint8_t *input, const int8_t *wq,
                          const float *scale, const float *shift, void *output, int32_t *acc);

/* ---- Winograd F(4x4,3x3), int8 GEMM ----
 * User input fp32, or u8 codes handed over as floats (the reference converts the codes to float
 * and transforms them as they are, src/kernel/elk_conv_wino_4x4_3x3_input.hxx:40-47; the input scale
 * only enters the quantization factor in_S / tin_S).  User output fp32, u8 or s8 (p->out_type).
 * tiles: t = n*ht*wt + th*wt + tw (src/elx_conv_wino_trans_input.cpp:10-24).
 * twq [36][OCp][ICp] s8; tscale/tshift [36][OCp];
 * tinput [36][ICp/16][t][16] u8; toutput [36][OCp/16][t][16] f32. */
int orc_wino_tiles(const orc_conv_params *p);
/* fp32 transform only (what the reference harness dumps to calibrate wino_tinput_quant,
 * tests/elt_conv_utils.cpp:222-262): min/max over all transformed-input elements. */
int orc_wino_tinput_range(const orc_conv_params *p, const float *input, float *min_out, float *max_out);
/* src/kernel/elk_conv_wino_4x4_3x3_weights.hxx:18-72 + src/elx_conv_wino_trans_weights.cpp:437-535 */
int orc_wino_prepare(const orc_conv_params *p, const float *w_blocked, int8_t *twq,
                     float *tscale, float *tshift);
/* src/kernel/elk_conv_wino_4x4_3x3_input.hxx:13-352 + src/elx_conv_wino_trans_input.cpp:599-654 */
int orc_wino_trans_input(const orc_conv_params *p, const float *input, uint8_t *tinput);
/* src/elx_int8_conv_wino_gemm.cpp:23-76 + src/kernel/elk_u8s8_gemm.hxx:200-208 */
int orc_wino_gemm(const orc_conv_params *p, const uint8_t *tinput, const int8_t *twq,
                  const float *tscale, const float *tshift, float *toutput, int32_t *acc);
/* src/kernel/elk_conv_wino_4x4_3x3_output.hxx:19-201 + src/elx_conv_wino_trans_output.cpp:212-277 */
int orc_wino_trans_output(const orc_conv_params *p, const float *toutput, const float *bias,
                          void *output);
/* what the output transform does to one value after Y = At M A (bias, output quantization, ReLU,
 * rounding, saturation; src/kernel/elk_conv_wino_4x4_3x3_output.hxx:94-111,159-195) */
int orc_wino_output_value(float y, int with_bias, float bias, int out_type, float out_scale, float out_z,
                          int with_relu, float *f32_out);

/* single 6x6 / 3x3 / 4x4 tile transforms, exposed so they can be compared one-to-one with the
 * reference's compiled kernel templates */
void orc_wino_tile_input(const float d[36], float v[36]);         /* interior tiles */
void orc_wino_tile_input_border(const float d[36], float v[36]);  /* tiles that touch the zero border */
void orc_wino_tile_weights(const float g[9], float u[36]);
void orc_wino_tile_output(const float m[36], float y[16]);
/* any tile size A in {4, 5, 6}; arrays are [A][A] (output: [A-2][A-2]) row-major
 * (src/kernel/elk_conv_wino_2x2_3x3_*.hxx, src/kernel/elk_conv_wino_3x3_3x3_*.hxx) */
void orc_wino_tile_input_a(int A, int border, const float *d, float *v);
void orc_wino_tile_weights_a(int A, const float g[9], float *u);
void orc_wino_tile_output_a(int A, const float *m, float *y);
int orc_wino_output_value_a(int A, float y, int with_bias, float bias, int out_type, float out_scale, float out_z,
                            int with_relu, float *f32_out);
int orc_wino_output_value_sum(int A, float y, int with_bias, float bias, int out_type, float out_scale, float out_z,
                              int with_relu, int with_sum, float old, float *f32_out);

/* epilogue on one value, exposed for the same reason (out_kind ORC_*; returns the f32 result
 * for ORC_F32 through *fout, else the quantized byte through the return value) */
int orc_epilogue(int out_kind, int32_t acc, float scale, float shift, int with_sum, int old_q,
                 float sum_scale, int with_relu, float lo, float hi, float *fout);

int orc_num_threads(void);
int orc_has_vnni(void);

#ifdef __cplusplus
}
#endif
#endif
