// Internal declarations shared by the gfx950 kernels and the C-ABI layer.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>
#include <string>

#include "euler_hip.h"

namespace ehip {

typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int kWave = 64;
constexpr int kBlock = 256;      // 4 waves per workgroup everywhere
constexpr int kOcTile = 256;     // packed weights are zero-padded to a multiple of this many rows

inline int up(int x, int m) { return (x + m - 1) / m * m; }
inline unsigned div_magic(int d) { return d <= 1 ? 0u : (unsigned)((1ull << 32) / (unsigned)d + 1); }

enum Family { FAM_GEMM_1X1 = 1, FAM_CONV_3X3 = 2, FAM_DEPTHWISE = 3, FAM_WINOGRAD = 4, FAM_CONV_FEWCH = 5 };

// requantization epilogue parameters, by value in kernel arguments
struct Epilogue {
  const float *scale;   // [batch][OCpp]
  const float *shift;   // [batch][OCpp]
  const int *comp;      // [batch][OCpp]  128 * sum of the packed weights (u8 -> s8 remap)
  float sum_scale, lo, hi;
  int out_type;         // EHIP_F32 / U8 / S8 / S32
  int with_sum, with_relu;
  // Non-zero input zero point with padding: the shift depends on which taps fall inside the image
  // for the output pixel.  shift_tab holds one shift row per class of pixels ([class][tab_stride]);
  // null = the shift depends on the channel only.
  const float *shift_tab;
  int tab_stride;
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
  int in_nhwc, out_nhwc;       // activations as [n][h][w][c] instead of [n][c/16][h][w][16] (c % 16 == 0)
  int kh, kw, pad_t, pad_l, ih;   // kh * kw > 1: direct convolution as a GEMM over [tap][unit] (blocked input)
  const int *cls_h, *cls_w;       // with ep.shift_tab: class of an output row / column; class = cls_h * ncls_w + cls_w
  int ncls_w;
  int sk_wo;                      // set by the small-K launcher: waves of a workgroup along the channels (1, 2, 4)
  int k_units, k_real;            // set by the launcher: units the K loop walks (a multiple of KC), real ones
  unsigned ic2_magic, kw_magic;
  int nx, ny;                  // set by the launcher: pixel blocks, channel blocks
  long long *trace;            // development aid, normally null (see EHIP_TRACE)
  int lean;                    // set by the launcher: lean_mode() of the epilogue (0 = general epilogue)
  unsigned u1_magic;           // set by the resident-tile launcher: div_magic(units_pad + 1)
  int wr_region, wr_stage, wr_nbuf;   // set by the weights-resident launcher: pixels per region, bytes per LDS stage, stages
};

struct Conv3x3Args {
  const uint8_t *in;    // [n][ic2][ih][iw][16]
  const int8_t *w;      // [9][units_pad][OCpp][16]
  void *out;            // [n][oc2][oh][ow][16]
  Epilogue ep;
  int ih, iw, oh, ow;
  int pad_t, pad_l;
  int ic2, units_pad, oc2, ocpp;
  int chunk_units;      // ic2 units staged per LDS fill (even)
  int vw;               // virtual row width: ow + 2 (stride 1), ow + 1 (stride 2)
  unsigned vw_magic;    // div_magic(vw)
  long long *trace;     // development aid, normally null (see EHIP_TRACE)
  int gx, gy, tiles, tiles_per_xcd;   // set by the launcher: pixel tiles per image, channel tiles, all tiles, ceil(tiles / 8)
  int lean;             // set by the launcher: lean_mode() of the epilogue (0 = general epilogue)
};

struct DepthwiseArgs {
  const uint8_t *in;    // [n][g2][ih][iw][16]
  const int8_t *w;      // [g2][kh = 3][16 channels][kw0 kw1 kw2 0]
  void *out;            // [n][g2][oh][ow][16]
  const float *scale, *shift;  // [G]
  const int *wsum;      // [G] sum of the packed weights per channel
  const uint4 *wdiag;   // [g2][6][64] A operands of the matrix-core kernel (launch_depthwise_diag)
  int n, g2, ih, iw, oh, ow, pad_t, pad_l;
  int stride;           // 1 or 2, both directions
  int T, Tr, wt;        // width blocking of the reference kernel (decides floor vs round per column)
  int lanes_per_plane;  // set by the launcher: row blocks x column pairs x 4
  int strips_per_wg;    // set by the launcher (matrix-core kernel): consecutive strips a workgroup walks
  int planes_per_block, lanes_padded;   // set by the launcher (dot4 kernel): small planes sharing a workgroup, lanes per plane rounded up to waves
  int blocks_per_plane; // set by the launcher: workgroups per plane
  unsigned wp_magic, T_magic;  // div_magic of the column pairs per row and of T
  int out_type, with_relu;
  float lo, hi;
};

struct WinoArgs {
  const void *in;       // [n][ic2][ih][iw][16] f32, or u8 codes (in_u8)
  uint8_t *tin;         // [36][ic2][t][16], or (tin_blocked) [t / 32][36][ic2][32][16]
  int tin_blocked;      // the fused schedule's layout: everything a block of 32 tiles needs is one contiguous run
  const float *tout;    // [36][oc2][t][16]
  void *out;            // [n][oc2][oh][ow][16] f32 / u8 / s8 (out_type)
  const float *bias;
  int in_u8, out_type;
  float out_repS, out_z;   // u8 / s8 output: 1 / output_S, ceil(output_z)
  int n, ic2, oc2, ih, iw, oh, ow, ht, wt, nt, t, pad_t, pad_l;
  int tile;             // tile size A: 6 (or 0) = F(4x4,3x3), 4 = F(2x2,3x3), 5 = F(3x3,3x3); 36 below reads A * A
  int nblocks, items_per_xcd;   // set by the input-transform launcher: blocks of 64 tiles; ceil(blocks x units / 8)
  int buf_gather;       // set by the input-transform launcher: the input is below 4 GB, gather with buffer loads (2: u8 input by whole cells)
  float mrepS, mz;      // input_S / tinput_S, ceil(tinput_z)
  int with_bias, with_relu;
  int with_sum;         // in-place sum: the old output is added before the ReLU (stand-alone output transform only)
  int in_nhwc, out_nhwc;   // activations as [n][h][w][c] (c % 16 == 0) instead of nChw16c
};

struct WinoFusedArgs {
  const uint8_t *tin;   // [36][ic2][t][16] u8, or (tin_blocked) [t / 32][36][ic2][32][16]
  int tin_blocked;
  const int8_t *w;      // [36][units_pad][OCpp][16] s8
  void *out;            // [n][oc2][oh][ow][16] f32 / u8 / s8 (out_type)
  const float *bias;
  const float *scale, *shift;  // [36][OCpp]
  const int *comp;
  int out_type;
  float out_repS, out_z;   // u8 / s8 output: 1 / output_S, ceil(output_z)
  int n, ic2, units_pad, oc2, ocpp, oh, ow, ht, wt, nt, t;
  int with_bias, with_relu;
  int with_sum;         // in-place sum: the old output is added before the ReLU
  int tile;             // tile size A: 6 (or 0), 5, 4
  int out_nhwc;         // output as [n][h][w][c] (c % 16 == 0)
  int nx, ny;           // set by the launcher: blocks of 32 tiles, of 64 channels
  float4 *tpart;        // first-stage results parked between the two passes of the 512-channel lanes kernel (wino_lanes_tpart_bytes)
  long long *trace;     // development aid, normally null (see EHIP_TRACE)
};

// ---- launch plans -------------------------------------------------------------------------------
// What a launcher works out from the layer -- kernel, grid, LDS size, derived arguments, the EHIP_* knobs
// read from the environment, the one-off hipFuncSetAttribute -- is kept in the handle after the first
// launch: later executes of the handle patch the tensor pointers into the kept argument block and launch.
template <typename Args>
struct LaunchPlan {
  bool valid = false;
  void (*kernel)(Args) = nullptr;
  dim3 grid, block;
  unsigned lds = 0;
  Args args;
  const char *name = nullptr;   // set by a launcher whose choice of kernel the handle cannot know beforehand
  // set by a launcher whose kernel takes leading scalar arguments besides the block (`kernel` is then that
  // kernel's pointer under the one-argument type): how to launch the plan
  hipError_t (*enqueue)(const LaunchPlan &, hipStream_t) = nullptr;
};
template <typename Args>
inline hipError_t plan_launch(LaunchPlan<Args> *plan, void (*kernel)(Args), dim3 grid, dim3 block, size_t lds, const Args &a,
                              hipStream_t s)
{
  hipLaunchKernelGGL(kernel, grid, block, lds, s, a);
  const hipError_t e = hipGetLastError();
  if (plan && e == hipSuccess) {   // kept only once the first launch has gone out
    plan->kernel = kernel;
    plan->grid = grid;
    plan->block = block;
    plan->lds = (unsigned)lds;
    plan->args = a;
    plan->valid = true;
  }
  return e;
}
// A launcher that fills a plan by hand launches through this: the plan becomes valid when the launch has gone out.
template <typename Args>
inline hipError_t plan_first_launch(LaunchPlan<Args> *p, hipStream_t s)
{
  hipError_t e;
  if (p->enqueue) {
    e = p->enqueue(*p, s);
  } else {
    hipLaunchKernelGGL(p->kernel, p->grid, p->block, p->lds, s, p->args);
    e = hipGetLastError();
  }
  p->valid = e == hipSuccess;
  return e;
}
// Later launches of a valid plan: the kept plan is only read.  The tensors of this call are patched into a COPY of
// the argument block, so executes of one handle from several threads or streams never see each other's pointers.
template <typename Args, typename Patch>
inline hipError_t plan_relaunch(const LaunchPlan<Args> &plan, Patch patch, hipStream_t s)
{
  LaunchPlan<Args> local = plan;
  patch(local.args);
  if (local.enqueue) return local.enqueue(local, s);
  hipLaunchKernelGGL(local.kernel, local.grid, local.block, local.lds, s, local.args);
  return hipGetLastError();
}

// ---- launchers (implemented next to their kernels) ------------------------------------------
hipError_t launch_gemm(const GemmArgs &a, int nbatch, int variant, hipStream_t s, LaunchPlan<GemmArgs> *plan = nullptr);
bool gemm_smallk_applies(int ic2, int taps, int nbatch);
int gemm_pick_variant(int p_total, int oc2, int ic2, int nbatch, int stride);
int gemm_variant_chunk(int variant);
int gemm_num_variants();
const char *gemm_variant_name(int variant);

// 1x1 layers with many input channels, blocked activations: pixel tile resident in LDS, weights streamed
int gemm1x1_res_pick(const GemmArgs &a, int nbatch);   // variant, or -1 when the layer is not one for it
const char *gemm1x1_res_name(int variant);
hipError_t launch_gemm1x1_res(const GemmArgs &a, int variant, hipStream_t s, LaunchPlan<GemmArgs> *plan = nullptr);
// 1x1 layers of 256 / 512 / 1024 input channels with the lean epilogue: weights resident in registers, pixels streamed
bool gemm1x1_wres_applies(const GemmArgs &a, int nbatch);
hipError_t launch_gemm1x1_wres(const GemmArgs &a, hipStream_t s, LaunchPlan<GemmArgs> *plan = nullptr);

hipError_t launch_conv3x3v(const Conv3x3Args &a, int n, int variant, hipStream_t s, LaunchPlan<Conv3x3Args> *plan = nullptr);
int conv3x3v_pick_variant(int n, int oh, int ow, int oc2, int stride);   // stride 1 or 2 (both directions); -1: rows too wide for every variant
int conv3x3v_chunk_units(int variant, int ic2);
int conv3x3v_num_variants();
const char *conv3x3v_variant_name(int variant);

hipError_t launch_depthwise(const DepthwiseArgs &a, hipStream_t s, LaunchPlan<DepthwiseArgs> *plan = nullptr);
hipError_t launch_depthwise_diag(const int8_t *wpacked, int g2n, void *diag, hipStream_t s);
bool depthwise_mfma_applies(int stride, int oh, int ow, int pad_t, int pad_l, int out_type, int with_relu, float lo, float hi,
                            long long planes, int ih, int iw);
hipError_t launch_wino_trans_input(const WinoArgs &a, hipStream_t s, LaunchPlan<WinoArgs> *plan = nullptr);
hipError_t launch_wino_trans_output(const WinoArgs &a, hipStream_t s, LaunchPlan<WinoArgs> *plan = nullptr);
hipError_t launch_wino_gemm_output(const WinoFusedArgs &a, hipStream_t s, LaunchPlan<WinoFusedArgs> *plan = nullptr);
// at most 256 input channels, u8 / s8 output: the form without an exchange between GEMMs and transform (ehip_wino_lanes.hip)
bool wino_lanes_applies(const WinoFusedArgs &a);
// device memory the lanes kernel needs besides the tensors (0 for most layers): a.tpart
size_t wino_lanes_tpart_bytes(int tile, int ic2, int oc2, int t);
hipError_t launch_wino_gemm_output_lanes(const WinoFusedArgs &a, hipStream_t s, LaunchPlan<WinoFusedArgs> *plan = nullptr);
// min / max of the transformed input: partials = 2 * a.ic2 dwords of device scratch, result = two floats
// of device memory (min, max); three launches on `s`, nothing else
hipError_t launch_wino_range(const WinoArgs &a, int ic_real, unsigned *partials, float *minmax_out_dev, hipStream_t s);
// the current device's copy of the library's static range scratch (2 * kRangeScratchUnits dwords);
// resolved once per device, no allocation
constexpr int kRangeScratchUnits = 4096;   // 16-channel units: up to 65536 input channels, 32 KB
hipError_t wino_range_scratch(unsigned **ptr);

// weight preparation
hipError_t launch_prepare_direct(const float *w_blocked, const float *bias, int oc, int ic, int kh, int kw,
                                 int units_pad, int ocpp, const ehip_conv_desc_t &d, float *absmax_scratch,
                                 int8_t *wpacked, float *scale, float *shift, int *wsum, int *comp, hipStream_t s);
// k x k direct convolution of an input with at most four channels (first layers): ppc = 16 / ic
// pixels per 16-byte operand cell, nu = ceil(kw / ppc) cells per kernel row
struct FewChArgs {
  const uint8_t *in;    // nhwc: [n][ih][iw][ic] (compact); blocked: [n][1][ih][iw][16]
  const int8_t *w;      // [kh * nu cells][OCpp rows][16] s8
  void *out;            // [n][oc2][oh*ow][16] or nhwc
  Epilogue ep;
  int n, ih, iw, oh, ow, ic, kh, kw;
  int stride_h, stride_w, pad_t, pad_l;
  int oc2, ocpp;
  int in_nhwc, out_nhwc;
  const int *cls_h, *cls_w;   // with ep.shift_tab: class of an output row / column; class = cls_h * ncls_w + cls_w
  int ncls_w, nclass;
  // set by the launcher
  int tab_lds;          // != 0: dword offset in LDS of on-chip copies of the class tables and shift rows
  int ppc, nu, cells;   // cells = kh * nu
  int rows, strips;     // output rows per workgroup, workgroups per image
  int nrows_in, lrow;   // staged input rows and their pitch in bytes (a multiple of 4)
  int wo;               // waves of a workgroup along the channels (1, 2, 4)
  int icl;              // bytes per pixel in a staged row and in an operand cell (conv_fewch_icl); set by the caller
  int lean;             // lean_mode() of the epilogue, per-pixel shift rows allowed (0 = general epilogue)
  unsigned ow_magic, iw_magic, lrow4_magic, lrow16_magic;
};
// Bytes a pixel takes in the staged rows and operand cells of the few-channel kernel: its ic channels, except
// that three channels are padded to four (the fourth multiplies a zero weight) where that costs no extra cell
// per kernel row (3x3 and 7x7 kernels: ceil(kw / 4) == ceil(kw / 5)) -- every cell then starts on a dword.
// EHIP_FEWCH_PAD_PIXEL=0 keeps three bytes.  A handle asks once and keeps the answer.
int conv_fewch_icl(int ic, int kw);
bool conv_fewch_applies(int ic, int kh, int kw);
int conv_fewch_row_pitch(int icl, int kw, int iw, int ow, int stride_w, int pad_l);   // icl: conv_fewch_icl()
hipError_t launch_conv_fewch(FewChArgs &a, hipStream_t s, LaunchPlan<FewChArgs> *plan = nullptr);
hipError_t launch_prepare_direct_px(const float *w, const float *bias, int oc, int ic, int icl, int kh, int kw, int ppc, int nu,
                                    int ocpp, const ehip_conv_desc_t &d, float *absmax, int8_t *wpacked, float *scale,
                                    float *shift, int *wsum, int *comp, hipStream_t s);
hipError_t launch_fold_direct_border_px(const int8_t *wpacked, const float *absmax, const float *bias, int oc, int ic,
                                        int ppc, int nu, int ocpp, const ehip_conv_desc_t &d, const int *rects,
                                        int nclass, float *shift_tab, hipStream_t s);
hipError_t launch_fold_direct_border(const int8_t *wpacked, const float *absmax, const float *bias, int oc, int kw,
                                     int units_pad, int ocpp, const ehip_conv_desc_t &d, const int *rects, int nclass,
                                     float *shift_tab, hipStream_t s);
hipError_t launch_prepare_depthwise(const float *w_goihw, const float *bias, int g, const ehip_conv_desc_t &d,
                                    int8_t *wpacked, float *scale, float *shift, int *wsum, hipStream_t s);
hipError_t launch_prepare_wino(const float *w_blocked, int oc, int ic, int tile, int units_pad, int ocpp,
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
// n / d for any 0 <= n < 2^31: the estimate above is never too small and at most one too large
__device__ __forceinline__ int fastdiv_any(int n, int d, unsigned magic)
{
  if (d == 1) return n;
  unsigned q = __umulhi((unsigned)n, magic);
  if (q * (unsigned)d > (unsigned)n) --q;
  return (int)q;
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

// ---- weight row order ---------------------------------------------------------------------------
// Inside every group of 32 rows the packed weights are stored in the order in which the 32x32 MFMA
// hands rows to lanes: packed row 8g + 4h + j holds output channel 16h + 4g + j (g = 0..3, h = 0..1,
// j = 0..3).  A lane of the result (which owns rows 8g + 4h + j for its own h and all g, j) then
// holds 16 CONSECUTIVE output channels, i.e. exactly one 16-channel cell of the blocked output.
__host__ __device__ __forceinline__ int packed_row_of_oc(int oc)
{
  const int o = oc & 31;
  return (oc & ~31) + 8 * ((o >> 2) & 3) + 4 * (o >> 4) + (o & 3);
}
__host__ __device__ __forceinline__ int oc_of_packed_row(int r)
{
  const int i = r & 31;
  return (r & ~31) + 16 * ((i >> 2) & 1) + 4 * (i >> 3) + (i & 3);
}

// ---- fused requantization epilogue of the MFMA kernels -----------------------------------------
// A lane holds, for each of its TN pixels and TM 32-row tiles, 16 consecutive output channels: one
// 16-byte cell of u8/s8 output, four float4 of f32/s32 output.  The per-channel constants of the
// first tile are requested while the last k-steps run, the sum operands of a tile are all
// requested before the first is used, and the output type is a template parameter, so the
// epilogue is straight-line code whose memory latencies overlap.
typedef int v16i __attribute__((ext_vector_type(16)));

struct OcConsts {      // of 16 consecutive output channels
  float4 sc[4], sh[4];
  v4i comp[4];
};
__device__ __forceinline__ void load_consts(OcConsts &k, const Epilogue &ep, long long idx)
{
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    k.sc[q] = *reinterpret_cast<const float4 *>(ep.scale + idx + 4 * q);
    k.sh[q] = *reinterpret_cast<const float4 *>(ep.shift + idx + 4 * q);
    k.comp[q] = *reinterpret_cast<const v4i *>(ep.comp + idx + 4 * q);
  }
}

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

// four channels -> one dword of u8/s8 codes
template <int OUT, bool SUM, bool FAST>
__device__ __forceinline__ unsigned quant4(const Epilogue &ep, int a0, int a1, int a2, int a3, const float4 &sc,
                                           const float4 &sh, unsigned old)
{
  float f0 = __builtin_fmaf((float)a0, sc.x, sh.x);
  float f1 = __builtin_fmaf((float)a1, sc.y, sh.y);
  float f2 = __builtin_fmaf((float)a2, sc.z, sh.z);
  float f3 = __builtin_fmaf((float)a3, sc.w, sh.w);
  if (SUM) {
    int o0, o1, o2, o3;
    if (OUT == EHIP_U8) {
      o0 = old & 0xff; o1 = (old >> 8) & 0xff; o2 = (old >> 16) & 0xff; o3 = old >> 24;
    } else {
      o0 = (int)(signed char)(old & 0xff); o1 = (int)(signed char)((old >> 8) & 0xff);
      o2 = (int)(signed char)((old >> 16) & 0xff); o3 = (int)(signed char)(old >> 24);
    }
    f0 = __builtin_fmaf((float)o0, ep.sum_scale, f0);
    f1 = __builtin_fmaf((float)o1, ep.sum_scale, f1);
    f2 = __builtin_fmaf((float)o2, ep.sum_scale, f2);
    f3 = __builtin_fmaf((float)o3, ep.sum_scale, f3);
  }
  if (FAST) {
    // ReLU with a lower bound >= 0: every value is in [0, hi], so "round to nearest even, then
    // saturate" is a clamp to the code range and one v_cvt_pk_u8_f32 per byte, which rounds to
    // nearest even (the wave's float mode, never changed here) and saturates to 0..255 itself
    const float hi = OUT == EHIP_S8 ? __builtin_fminf(ep.hi, 127.0f) : ep.hi;
    // lo <= hi here, so min(max(f, lo), hi) is the median of the three -- also for a NaN f, where
    // v_med3_f32 falls back to min3 = lo, which is what max(NaN, lo) = lo gives the reference
    f0 = __builtin_amdgcn_fmed3f(f0, ep.lo, hi);
    f1 = __builtin_amdgcn_fmed3f(f1, ep.lo, hi);
    f2 = __builtin_amdgcn_fmed3f(f2, ep.lo, hi);
    f3 = __builtin_amdgcn_fmed3f(f3, ep.lo, hi);
    unsigned q = __builtin_amdgcn_cvt_pk_u8_f32(f0, 0, 0);
    q = __builtin_amdgcn_cvt_pk_u8_f32(f1, 1, q);
    q = __builtin_amdgcn_cvt_pk_u8_f32(f2, 2, q);
    return __builtin_amdgcn_cvt_pk_u8_f32(f3, 3, q);
  }
  if (ep.with_relu) {
    f0 = __builtin_fminf(__builtin_fmaxf(f0, ep.lo), ep.hi);
    f1 = __builtin_fminf(__builtin_fmaxf(f1, ep.lo), ep.hi);
    f2 = __builtin_fminf(__builtin_fmaxf(f2, ep.lo), ep.hi);
    f3 = __builtin_fminf(__builtin_fmaxf(f3, ep.lo), ep.hi);
  }
  return quant1<OUT>(f0) | (quant1<OUT>(f1) << 8) | (quant1<OUT>(f2) << 16) | (quant1<OUT>(f3) << 24);
}

// acc[mt][nt]: s32 sums WITHOUT the u8->s8 compensation (it is added here).  k0 = constants of the
// lane's channels in tile 0, cidx = their index in the per-channel arrays (tile mt: + 32 * mt),
// oc_first = the lane's first channel in tile 0 (a multiple of 16), pix[nt] = element offset of
// the pixel's cell in 16-channel block 0, block_stride = elements between 16-channel blocks.
//
// 4-byte outputs (f32, s32) can go through a wave-private 4 KB LDS patch `xlds` (XPOSE): a lane's
// 16 results are 64 bytes of ONE pixel, so a direct store instruction would scatter 64 pieces of
// 16 bytes; after the exchange four neighbouring lanes hold the four quarters of one pixel and an
// instruction writes 1 KB of consecutive memory.  pixT/validT[nt][k] describe pixel
// (lane / 4) + 16 * k of pixel tile nt, which is the pixel the lane stores after the exchange.
// The patch is laid out [16-channel block][pixel][quarter ^ ((pixel / 4) & 3)] in 16-byte cells,
// which keeps both the writes (fixed quarter, 16 pixels) and the reads (4 pixels x 4 quarters)
// spread over all banks.
// NOCOMP: the accumulators already hold the compensation (they started from it instead of zero).
template <int TM, int TN, int OUT, bool SUM, bool FAST, bool XPOSE, bool TAB, bool NOCOMP>
__device__ __forceinline__ void epilogue_wave_typed(const Epilogue &ep, const v16i (&acc)[TM][TN], const OcConsts &k0,
                                                    long long cidx, int oc_first, const size_t (&pix)[TN],
                                                    const bool (&pvalid)[TN], int oc_real, size_t block_stride,
                                                    void *out, v4i *xlds, const size_t (&pixT)[TN][2],
                                                    const bool (&validT)[TN][2], const int *cls)
{
  const bool relu = ep.with_relu != 0;
  const int lane = threadIdx.x & 63;
  OcConsts k = k0;
#pragma unroll
  for (int mt = 0; mt < TM; ++mt) {
    if (mt > 0) load_consts(k, ep, cidx + 32 * mt);   // tile 0's came with the last k-steps
    const int oc = oc_first + 32 * mt;
    const bool oc_ok = oc < oc_real;
    size_t e[TN];
    bool ok[TN];
    v4i old[TN];
#pragma unroll
    for (int nt = 0; nt < TN; ++nt) {
      ok[nt] = oc_ok && pvalid[nt];
      e[nt] = ok[nt] ? pix[nt] + (size_t)(oc >> 4) * block_stride : 0;
      if (SUM) old[nt] = *reinterpret_cast<const v4i *>(static_cast<const uint8_t *>(out) + e[nt]);
    }
#pragma unroll
    for (int nt = 0; nt < TN; ++nt) {
      const v16i &a = acc[mt][nt];
      float4 shq[4] = {k.sh[0], k.sh[1], k.sh[2], k.sh[3]};
      if (TAB) {   // the shift row of the pixel's border class
#pragma unroll
        for (int q = 0; q < 4; ++q)
          shq[q] = *reinterpret_cast<const float4 *>(ep.shift_tab + (size_t)cls[nt] * ep.tab_stride + cidx + 32 * mt + 4 * q);
      }
      v4i s[4];
#pragma unroll
      for (int q = 0; q < 4; ++q)
        s[q] = NOCOMP ? v4i{a[4 * q], a[4 * q + 1], a[4 * q + 2], a[4 * q + 3]}
                      : v4i{a[4 * q] + k.comp[q].x, a[4 * q + 1] + k.comp[q].y, a[4 * q + 2] + k.comp[q].z,
                            a[4 * q + 3] + k.comp[q].w};
      if (OUT == EHIP_S32 || OUT == EHIP_F32) {
        if (OUT == EHIP_F32) {
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            float4 r;
            r.x = requant1(s[q].x, k.sc[q].x, shq[q].x, relu, ep.lo, ep.hi);
            r.y = requant1(s[q].y, k.sc[q].y, shq[q].y, relu, ep.lo, ep.hi);
            r.z = requant1(s[q].z, k.sc[q].z, shq[q].z, relu, ep.lo, ep.hi);
            r.w = requant1(s[q].w, k.sc[q].w, shq[q].w, relu, ep.lo, ep.hi);
            s[q] = v4i{__float_as_int(r.x), __float_as_int(r.y), __float_as_int(r.z), __float_as_int(r.w)};
          }
        }
        if (XPOSE) {
          const int l32 = lane & 31, lh = lane >> 5;
#pragma unroll
          for (int q = 0; q < 4; ++q) xlds[lh * 128 + l32 * 4 + (q ^ ((l32 >> 2) & 3))] = s[q];
          __builtin_amdgcn_wave_barrier();
          // the wave's two 16-channel blocks: oc_first - 16 * lh + 32 * mt + 16 * h
          const int ocw = oc - 16 * lh;
#pragma unroll
          for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int kk = 0; kk < 2; ++kk) {
              const int P = (lane >> 2) + 16 * kk, bq = lane & 3;
              const v4i v = xlds[h * 128 + P * 4 + (bq ^ ((P >> 2) & 3))];
              if (validT[nt][kk] && ocw + 16 * h < oc_real)
                *reinterpret_cast<v4i *>(static_cast<int *>(out) + pixT[nt][kk] +
                                         (size_t)((ocw + 16 * h) >> 4) * block_stride + 4 * bq) = v;
            }
          __builtin_amdgcn_wave_barrier();
        } else if (ok[nt]) {
#pragma unroll
          for (int q = 0; q < 4; ++q) *reinterpret_cast<v4i *>(static_cast<int *>(out) + e[nt] + 4 * q) = s[q];
        }
      } else {
        v4i cell;
#pragma unroll
        for (int q = 0; q < 4; ++q)
          cell[q] = (int)quant4<OUT, SUM, FAST>(ep, s[q].x, s[q].y, s[q].z, s[q].w, k.sc[q], shq[q],
                                               SUM ? (unsigned)old[nt][q] : 0u);
        if (ok[nt]) *reinterpret_cast<v4i *>(static_cast<uint8_t *>(out) + e[nt]) = cell;
      }
    }
  }
}

// one uniform switch on the output type (and on the cheap ReLU form) around the whole epilogue;
// xlds == nullptr: 4-byte outputs are stored directly.  TAB: per-pixel shift rows (ep.shift_tab, cls).
template <int TM, int TN, bool TAB, bool NOCOMP = false>
__device__ __forceinline__ void epilogue_wave_tab(const Epilogue &ep, const v16i (&acc)[TM][TN], const OcConsts &k0,
                                                  long long cidx, int oc_first, const size_t (&pix)[TN],
                                                  const bool (&pvalid)[TN], int oc_real, size_t block_stride, void *out,
                                                  v4i *xlds, const size_t (&pixT)[TN][2], const bool (&validT)[TN][2],
                                                  const int *cls)
{
#define EHIP_EPI(OUT, SUM, FAST, XP)                                                                                   \
  epilogue_wave_typed<TM, TN, OUT, SUM, FAST, XP, TAB, NOCOMP>(ep, acc, k0, cidx, oc_first, pix, pvalid, oc_real, block_stride, \
                                                       out, xlds, pixT, validT, cls)
  // cheap narrowing: ReLU bounds 0 <= lo <= hi (and lo inside the s8 code range for s8 output)
  const bool fast = ep.with_relu && ep.lo >= 0.0f && ep.hi >= ep.lo && (ep.out_type != EHIP_S8 || ep.lo <= 127.0f);
  switch (ep.out_type) {
  case EHIP_U8:
    if (ep.with_sum) { if (fast) EHIP_EPI(EHIP_U8, true, true, false); else EHIP_EPI(EHIP_U8, true, false, false); }
    else { if (fast) EHIP_EPI(EHIP_U8, false, true, false); else EHIP_EPI(EHIP_U8, false, false, false); }
    break;
  case EHIP_S8:
    if (ep.with_sum) { if (fast) EHIP_EPI(EHIP_S8, true, true, false); else EHIP_EPI(EHIP_S8, true, false, false); }
    else { if (fast) EHIP_EPI(EHIP_S8, false, true, false); else EHIP_EPI(EHIP_S8, false, false, false); }
    break;
  case EHIP_F32:
    if (xlds) EHIP_EPI(EHIP_F32, false, false, true); else EHIP_EPI(EHIP_F32, false, false, false);
    break;
  default:
    if (xlds) EHIP_EPI(EHIP_S32, false, false, true); else EHIP_EPI(EHIP_S32, false, false, false);
    break;
  }
#undef EHIP_EPI
}

// BORDER: the kernel can be asked for per-pixel shift rows (the k x k GEMM form); other kernels do
// not carry that code at all
template <int TM, int TN, bool BORDER = false, bool NOCOMP = false>
__device__ __forceinline__ void epilogue_wave(const Epilogue &ep, const v16i (&acc)[TM][TN], const OcConsts &k0,
                                              long long cidx, int oc_first, const size_t (&pix)[TN],
                                              const bool (&pvalid)[TN], int oc_real, size_t block_stride, void *out,
                                              v4i *xlds, const size_t (&pixT)[TN][2], const bool (&validT)[TN][2],
                                              const int *cls = nullptr)
{
  if (BORDER && ep.shift_tab)
    epilogue_wave_tab<TM, TN, true, NOCOMP>(ep, acc, k0, cidx, oc_first, pix, pvalid, oc_real, block_stride, out, xlds, pixT, validT, cls);
  else
    epilogue_wave_tab<TM, TN, false, NOCOMP>(ep, acc, k0, cidx, oc_first, pix, pvalid, oc_real, block_stride, out, xlds, pixT, validT, cls);
}


// ---- lean epilogue -------------------------------------------------------------------------------
// u8 / s8 output, ReLU with bounds 0 <= lo <= hi (lo <= 127 for s8), with or without the in-place sum,
// per-channel shift only: the case of nearly every layer of the tuned networks.  The launcher decides
// (lean_mode) so that the kernel carries no output-type switch on this path; the accumulators already hold
// the u8 -> s8 compensation.  A value costs a convert, a multiply-add, (a second one for the sum,) a
// clamp -- none when the bounds are exactly the u8 code range, which v_cvt_pk_u8_f32 saturates to by
// itself -- and a byte pack.  Arithmetic and rounding are those of quant4<.., FAST = true>.
// A lane's 16 output bytes.  NT: a non-temporal store -- the line is not kept in L2.  Measured: kernels that
// write several times what they read (1x1 layers with few input channels: 8-10 % faster, the strided 3x3
// GEMM 4 %) gain, the 3x3 and the resident-tile 1x1 kernel do not (0 to -1 %), so the caller chooses.
template <bool NT>
__device__ __forceinline__ void store_out16(uint8_t *p, const v4i &v)
{
  if (NT) __builtin_nontemporal_store(v, reinterpret_cast<v4i *>(p));
  else *reinterpret_cast<v4i *>(p) = v;
}
struct LeanConsts {   // scale and shift of the lane's 16 channels of each 32-channel tile
  float4 sc[4], sh[4];
};
__device__ __forceinline__ void load_lean_consts(LeanConsts &k, const Epilogue &ep, long long idx)
{
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    k.sc[q] = *reinterpret_cast<const float4 *>(ep.scale + idx + 4 * q);
    k.sh[q] = *reinterpret_cast<const float4 *>(ep.shift + idx + 4 * q);
  }
}
// 0 = general epilogue; else bit 0 set, bit 1 = no clamp needed, bit 2 = with sum.  EHIP_LEAN_EPILOGUE=0 switches
// it off here, in the one place every launcher and every choice of kernel that depends on it asks.
inline int lean_mode(const Epilogue &e, bool out_nhwc)
{
  if (const char *env = getenv("EHIP_LEAN_EPILOGUE")) if (env[0] == '0') return 0;
  const bool q = e.out_type == EHIP_U8 || e.out_type == EHIP_S8;
  const bool fast = q && e.with_relu && !e.shift_tab && !out_nhwc && e.lo >= 0.0f && e.hi >= e.lo &&
      (e.out_type != EHIP_S8 || e.lo <= 127.0f);
  if (!fast) return 0;
  return 1 | ((e.out_type == EHIP_U8 && e.lo == 0.0f && e.hi >= 255.0f) ? 2 : 0) | (e.with_sum ? 4 : 0);
}
// cell[nt]: byte address of the lane's 16-byte cell of pixel tile nt in the wave's FIRST 16-channel block pair
// member (block lh of tile 0); tile_stride: bytes between the cells of consecutive 32-channel tiles.
// old_in: the sum operands if the caller has fetched them already (else null: they are read here).
template <int TM, int TN, bool SUM, bool CLAMP, bool NT>
__device__ __forceinline__ void lean_store_typed(const Epilogue &ep, const v16i (&acc)[TM][TN], const LeanConsts (&k)[TM],
                                                 uint8_t *const (&cell)[TN], const bool (&pvalid)[TN], int oc_first,
                                                 int oc_real, size_t tile_stride, const v4i (*old_in)[TN])
{
  const bool s8 = ep.out_type == EHIP_S8;
  const float hi = s8 ? __builtin_fminf(ep.hi, 127.0f) : ep.hi;
#pragma unroll
  for (int nt = 0; nt < TN; ++nt) {
    v4i old[TM];
    if (SUM) {
#pragma unroll
      for (int mt = 0; mt < TM; ++mt) {
        if (old_in) {
          old[mt] = old_in[mt][nt];
        } else {
          const bool ok = pvalid[nt] && oc_first + 32 * mt < oc_real;
          old[mt] = *reinterpret_cast<const v4i *>(ok ? cell[nt] + mt * tile_stride : cell[nt]);
        }
      }
    }
#pragma unroll
    for (int mt = 0; mt < TM; ++mt) {
      v4i out;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const float sc[4] = {k[mt].sc[q].x, k[mt].sc[q].y, k[mt].sc[q].z, k[mt].sc[q].w};
        const float sh[4] = {k[mt].sh[q].x, k[mt].sh[q].y, k[mt].sh[q].z, k[mt].sh[q].w};
        unsigned pk = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          float f = __builtin_fmaf((float)acc[mt][nt][4 * q + j], sc[j], sh[j]);
          if (SUM) {
            const unsigned b = ((unsigned)old[mt][q] >> (8 * j)) & 0xffu;
            const int o = s8 ? (int)(signed char)b : (int)b;
            f = __builtin_fmaf((float)o, ep.sum_scale, f);
          }
          if (CLAMP) f = __builtin_amdgcn_fmed3f(f, ep.lo, hi);
          pk = __builtin_amdgcn_cvt_pk_u8_f32(f, j, pk);
        }
        out[q] = (int)pk;
      }
      if (pvalid[nt] && oc_first + 32 * mt < oc_real) store_out16<NT>(cell[nt] + mt * tile_stride, out);
    }
  }
}
template <int TM, int TN, bool NT = false>
__device__ __forceinline__ void lean_store(int mode, const Epilogue &ep, const v16i (&acc)[TM][TN], const LeanConsts (&k)[TM],
                                           uint8_t *const (&cell)[TN], const bool (&pvalid)[TN], int oc_first, int oc_real,
                                           size_t tile_stride, const v4i (*old_in)[TN] = nullptr)
{
  // one uniform branch, four straight copies
  if (mode & 4) {
    if (mode & 2) lean_store_typed<TM, TN, true, false, NT>(ep, acc, k, cell, pvalid, oc_first, oc_real, tile_stride, old_in);
    else lean_store_typed<TM, TN, true, true, NT>(ep, acc, k, cell, pvalid, oc_first, oc_real, tile_stride, old_in);
  } else {
    if (mode & 2) lean_store_typed<TM, TN, false, false, NT>(ep, acc, k, cell, pvalid, oc_first, oc_real, tile_stride, old_in);
    else lean_store_typed<TM, TN, false, true, NT>(ep, acc, k, cell, pvalid, oc_first, oc_real, tile_stride, old_in);
  }
}

// the harness's fp32 reference convolution (calibration), ehip_harness.hip
struct RefConvArgs {
  const float *in, *w, *bias;
  float *out;        // nullable unless with_sum
  float *partials;   // [blocks][2]
  int n, g, ic, oc, ih, iw, oh, ow, kh, kw, pad_t, pad_l, sh, sw;
  int in_nhwc, out_nhwc, w_goihw, with_relu, with_sum, with_bias;
  int ic2, oc2;
};

hipError_t launch_ref_conv_f32(const RefConvArgs &a, unsigned blocks);

}  // namespace ehip
#endif
