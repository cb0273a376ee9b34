// C-ABI layer (include/euler_hip.h): descriptor validation and executor choice, device
// workspace, weight preparation, launches.  No kernels here.
#include <cfloat>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <utility>
#include <vector>

#include "ehip_internal.hpp"

using namespace ehip;

namespace {
thread_local std::string g_last_error;
}

namespace ehip {
void set_error(const std::string &msg) { g_last_error = msg; }
}  // namespace ehip

#define HIP_TRY(expr)                                                                              \
  do {                                                                                             \
    hipError_t _e = (expr);                                                                        \
    if (_e != hipSuccess) {                                                                        \
      set_error(std::string(#expr) + ": " + hipGetErrorString(_e));                                \
      return EHIP_HIP_ERROR;                                                                       \
    }                                                                                              \
  } while (0)

struct ehip_conv {
  ehip_conv_desc_t d;
  int family = 0;
  int variant = 0;
  bool prepared = false;
  std::string kernel_name;

  int ic2 = 0, oc2 = 0, ocpp = 0, units_pad = 0, taps = 1, nbatch = 1;
  int8_t *wpacked = nullptr;
  size_t wpacked_bytes = 0;
  float *scale = nullptr, *shift = nullptr, *absmax = nullptr;
  int *wsum = nullptr, *comp = nullptr;
  size_t per_oc = 0;  // elements in scale/shift/wsum/comp

  // k x k direct with a non-zero input zero point and padding: classes of output pixels by their
  // set of valid taps (a rectangle of kernel rows x columns) and one shift row per class
  int nclass = 0, ncls_w = 0;
  int *cls_h = nullptr, *cls_w = nullptr, *rects = nullptr;
  float *shift_tab = nullptr;
  // k x k direct with at most four input channels: ppc = 16 / ic pixels per 16-byte cell, nu cells per
  // kernel row; gtaps = taps of the K axis of the packed weights (kh * nu there, kh * kw otherwise)
  int ppc = 0, nu = 0, gtaps = 1, icl = 0;   // icl: bytes per pixel in a cell (conv_fewch_icl)
  // 3x3
  int chunk_units = 2;
  // depthwise
  int T = 1, Tr = 1, wtb = 1;
  // Winograd
  int ht = 0, wt = 0, nt = 0, t = 0, wino_tile = 6;
  int chunk_n = 0;   // images per pass of the three-stage pipeline (intermediates sized for it)
  bool fused = true; // GEMM and output transform in one kernel (no f32 GEMM result in memory)
  uint8_t *tin = nullptr;
  bool tin_blocked = false;   // Winograd, fused schedule: tin as [t / 32][36][ic2][32][16]
  float *tout = nullptr;
  size_t tin_bytes = 0, tout_bytes = 0;

  // launch plans of the steady state (filled by the first execute, see LaunchPlan); the Winograd ones are
  // used only when the layer runs in one pass (no chunking)
  int stage_mask = 7;   // Winograd: which stages execute() launches (ehip_conv_execute_stages)
  LaunchPlan<GemmArgs> plan_gemm;
  LaunchPlan<Conv3x3Args> plan_3x3;
  LaunchPlan<FewChArgs> plan_fewch;
  LaunchPlan<DepthwiseArgs> plan_dw;
  LaunchPlan<WinoArgs> plan_wino_in, plan_wino_out;
  LaunchPlan<WinoFusedArgs> plan_wino_fused;
};

namespace {

const float kNoCali = FLT_MAX;  // EL_NO_CALI

int fail(int code, const std::string &msg)
{
  set_error(msg);
  return code;
}

void free_all(ehip_conv *c)
{
  // (scale, shift and comp are one allocation: see setup_workspace)
  void *ptrs[] = {c->wpacked, c->scale, c->absmax, c->wsum, c->tin, c->tout,
                  c->cls_h, c->cls_w, c->rects, c->shift_tab};
  for (void *p : ptrs)
    if (p) (void)hipFree(p);
}

template <typename T>
int dev_alloc(T **p, size_t count, bool zero)
{
  HIP_TRY(hipMalloc(reinterpret_cast<void **>(p), count * sizeof(T)));
  if (zero) HIP_TRY(hipMemset(*p, 0, count * sizeof(T)));
  return EHIP_OK;
}

// tile_size 0: the reference's choice between 6 and 4 (src/eld_conv.cpp:231-236)
int wino_auto_tile(const ehip_conv_desc_t &d)
{
  const int t = d.n * ((d.oh + 3) / 4) * ((d.ow + 3) / 4);
  const int ocp = up(d.oc, 16);
  const float mac_per_read = (float)((double)t * ocp) / (float)(t + ocp);
  return mac_per_read > 25.0f ? 6 : 4;
}

// mirrors the dispatch of eld_conv_t::setup (src/eld_conv.cpp:148-313) for the int8 executors
int classify(ehip_conv *c)
{
  ehip_conv_desc_t &d = c->d;
  if (d.g <= 0 || d.ic % d.g || d.oc % d.g) return fail(EHIP_GENERAL_ERROR, "dims: groups: ic|oc != g * x");
  const bool depthwise = d.g == d.ic && d.g == d.oc && d.g > 1;
  const int icg = d.ic / d.g;
  if (d.dilation_h != 1 || d.dilation_w != 1) return fail(EHIP_UNIMPLEMENTED, "dilation is not supported by the int8 path");

  if (d.algorithm == EHIP_CONV_AUTO) {
    if (d.kh == 1 && d.kw == 1) d.algorithm = EHIP_CONV_DIRECT_1X1;
    else if (icg >= 16 && d.kh == 3 && d.kw == 3 && d.stride_h == 1 && d.stride_w == 1 && d.pad_l == 1 &&
             d.pad_r == 1 && d.pad_t == 1 && d.pad_b == 1)
      d.algorithm = EHIP_CONV_WINOGRAD;
    else d.algorithm = EHIP_CONV_DIRECT;
  }

  const bool in_u8 = d.input_type == EHIP_U8 && d.weights_type == EHIP_F32 && d.bias_type == EHIP_F32;
  const bool out_q = d.output_type == EHIP_U8 || d.output_type == EHIP_S8;
  const bool all_f32 = d.input_type == EHIP_F32 && d.weights_type == EHIP_F32 && d.output_type == EHIP_F32 &&
      d.bias_type == EHIP_F32;

  if (d.algorithm != EHIP_CONV_WINOGRAD) {
    if (!in_u8) return fail(EHIP_UNIMPLEMENTED, "only the u8-input int8 executors are built (fp32 paths are out of scope)");
    if (d.sampling_kind != 2) return fail(EHIP_UNIMPLEMENTED, "int8 direct: non-calibrated sampling_kind not supported");
    if (d.input_scale == kNoCali || d.input_z == kNoCali) return fail(EHIP_GENERAL_ERROR, "input_quant is not set");
    if (out_q && (d.output_scale == kNoCali || d.output_z == kNoCali || d.output_scale == 0.0f))
      return fail(EHIP_GENERAL_ERROR, "output_quant is not set");
    // nhwc activations (src/elx_int8_conv_direct_1x1.cpp:374-396,417-468, src/elx_int8_conv_direct.cpp:596-668)
    // are built for the 1x1 GEMM family; the reference refuses channel tails there as well
    // ("Or not support", src/elx_int8_conv_direct_1x1.cpp:88-91)
    const bool in_ok = d.input_fmt == EHIP_NCHW16C || d.input_fmt == EHIP_NHWC;
    const bool out_ok = d.output_fmt == EHIP_NCHW16C || d.output_fmt == EHIP_NHWC;
    if (!in_ok || !out_ok) return fail(EHIP_UNIMPLEMENTED, "activation formats: nChw16c or nhwc");
    // nhwc on either side of the 1x1 and kh x kw direct executors; with at most four channels (the
    // first layer of an image network) the nhwc input is compact: ic bytes per pixel
    const bool fewch = d.algorithm == EHIP_CONV_DIRECT && !depthwise && conv_fewch_applies(d.ic, d.kh, d.kw);
    if (d.input_fmt == EHIP_NHWC && depthwise)
      return fail(EHIP_UNIMPLEMENTED, "nhwc input is not built for depthwise convolutions");
    if (d.output_fmt == EHIP_NHWC && depthwise)
      return fail(EHIP_UNIMPLEMENTED, "nhwc output is not built for depthwise convolutions");
    if ((d.input_fmt == EHIP_NHWC && d.ic % 16 && !fewch) || (d.output_fmt == EHIP_NHWC && d.oc % 16))
      return fail(EHIP_UNIMPLEMENTED, "nhwc: channel counts must be multiples of 16");
  }

  if (d.algorithm == EHIP_CONV_DIRECT_1X1) {
    if (d.kh != 1 || d.kw != 1) return fail(EHIP_GENERAL_ERROR, "Algorithm CONV_DIRECT_1X1 not supported for this shape.");
    if (!(out_q || d.output_type == EHIP_S32)) return fail(EHIP_UNIMPLEMENTED, "direct_1x1: int8: only u8/s8 output");
    if (d.g != 1) return fail(EHIP_UNIMPLEMENTED, "direct_1x1: groups are not supported");
    if (d.pad_l || d.pad_t || d.stride_h * (d.oh - 1) + 1 > d.ih || d.stride_w * (d.ow - 1) + 1 > d.iw)
      return fail(EHIP_UNIMPLEMENTED, "no support for padding in 1x1 u8s8 conv");
    if (d.stride_h > 2 || d.stride_w > 2 || d.stride_h != d.stride_w)
      return fail(EHIP_UNIMPLEMENTED, "direct_1x1: int8: Shape not supported");
    if (d.stride_w == 2 && d.flatting_t > 0 && d.ow % d.flatting_t)
      return fail(EHIP_UNIMPLEMENTED, "direct_1x1: int8: No Tr support for ws == 2");
    if (d.weights_fmt != EHIP_OIHW16I16O) return fail(EHIP_UNIMPLEMENTED, "weights must be OIhw16i16o");
    if (d.with_ip_sum && d.output_type == EHIP_S32) return fail(EHIP_UNIMPLEMENTED, "s32 output has no sum fusion");
    c->family = FAM_GEMM_1X1;
    return EHIP_OK;
  }

  if (d.algorithm == EHIP_CONV_DIRECT) {
    if (depthwise) {
      if (!(out_q || d.output_type == EHIP_S32)) return fail(EHIP_UNIMPLEMENTED, "depthwise: only u8/s8 output");
      if (d.kh != 3 || d.kw != 3 || d.pad_l > 1 || d.pad_t > 1)
        return fail(EHIP_UNIMPLEMENTED, "direct_depthwise: int8: shape not supported");
      if (d.stride_h != d.stride_w || d.stride_h < 1 || d.stride_h > 2)
        return fail(EHIP_UNIMPLEMENTED, "direct_depthwise: stride must be 1 or 2");
      if (d.g % 16) return fail(EHIP_UNIMPLEMENTED, "conv: g blocking error for depthwise conv");
      if (d.weights_fmt != EHIP_GOIHW) return fail(EHIP_UNIMPLEMENTED, "direct_depthwise: format not supported");
      if (d.with_ip_sum) return fail(EHIP_UNIMPLEMENTED, "direct_depthwise: no sum fusion");
      // a non-zero input zero point: as in the reference, a padded tap adds nothing to the sum while the
      // shift takes z times all nine weights (src/elx_int8_conv_direct_depthwise.cpp:247-289,
      // src/kernel/elk_u8s8_depthwise_conv.hxx:316-413) -- no border correction
      c->family = FAM_DEPTHWISE;
      return EHIP_OK;
    }
    if (d.g != 1) return fail(EHIP_UNIMPLEMENTED, "direct: groups are not supported");
    if (!(out_q || d.output_type == EHIP_F32 || d.output_type == EHIP_S32))
      return fail(EHIP_UNIMPLEMENTED, "direct: output type not supported");
    if (d.weights_fmt != EHIP_OIHW16I16O) return fail(EHIP_UNIMPLEMENTED, "direct: format not supported");
    // the reference's direct executor silently drops with_ip_sum (src/elx_int8_conv_direct.cpp:121);
    // refuse instead of computing something else than asked
    if (d.with_ip_sum) return fail(EHIP_UNIMPLEMENTED, "direct: sum fusion is only available in CONV_DIRECT_1X1");
    if (d.kh == 1 && d.kw == 1) {
      if (d.pad_l || d.pad_t || d.stride_h * (d.oh - 1) + 1 > d.ih || d.stride_w * (d.ow - 1) + 1 > d.iw)
        return fail(EHIP_UNIMPLEMENTED, "direct: a160: padding is not built");
      if (d.stride_h > 2 || d.stride_w > 2) return fail(EHIP_UNIMPLEMENTED, "direct: a160: stride not supported");
      c->family = FAM_GEMM_1X1;
      return EHIP_OK;
    }
    // c160 shapes (src/elx_int8_conv_direct.cpp:66-77): 3/5/7 kernels, stride 1 or 2, every pad
    // k/2 - 1 or k/2.  Right and bottom pads follow from the output size, as the reference
    // recomputes them (src/elx_conv.cpp:36-37).
    const bool k_ok = (d.kh == 3 || d.kh == 5 || d.kh == 7) && (d.kw == 3 || d.kw == 5 || d.kw == 7);
    const bool s_ok = (d.stride_w == 1 || d.stride_w == 2) && (d.stride_h == 1 || d.stride_h == 2);
    const int rp = (d.ow - 1) * d.stride_w + d.kw - d.iw - d.pad_l, bp = (d.oh - 1) * d.stride_h + d.kh - d.ih - d.pad_t;
    auto pad_ok = [](int p, int k) { return p == k / 2 - 1 || p == k / 2; };
    if (k_ok && s_ok && pad_ok(d.pad_l, d.kw) && pad_ok(d.pad_t, d.kh) && pad_ok(rp < 0 ? d.kw / 2 - 1 : rp, d.kw) &&
        pad_ok(bp < 0 ? d.kh / 2 - 1 : bp, d.kh)) {
      const bool padded = d.pad_l || d.pad_t || rp > 0 || bp > 0;
      // zero point with padding (src/elx_int8_conv_direct.cpp:247-255): every pad must be coverable
      if (d.input_z != 0.0f && padded &&
          (d.pad_l + d.ow < d.kw || (rp > 0 ? rp : 0) + d.ow < d.kw || d.pad_t + d.oh < d.kh || (bp > 0 ? bp : 0) + d.oh < d.kh))
        return fail(EHIP_UNIMPLEMENTED, "Shape not support for U8 input with zero-point");
      const int T = d.flatting_t > d.ow ? d.ow : d.flatting_t;
      if (T > 0 && d.ow % T)
        return fail(EHIP_UNIMPLEMENTED, "direct: c160: ow must be a multiple of T (the reference mis-indexes shift for Tr != T)");
      const bool s1_3x3 = d.kh == 3 && d.kw == 3 && d.stride_h == 1 && d.stride_w == 1 &&
          d.ow == d.iw + d.pad_l + d.pad_r - 2 && d.oh == d.ih + d.pad_t + d.pad_b - 2;
      // the GEMM family walks [tap][unit] for kh x kw; it also owns the per-pixel shift that a zero
      // point with padding needs
      // 3x3 stride 2 runs the same kernel over four phase planes of the input (EHIP_CONV3X3V_S2=0: the GEMM form)
      const char *s2env = getenv("EHIP_CONV3X3V_S2");
      // (its staging plan holds a cell's byte offset inside one image plane in 31 bits)
      const bool s2_3x3 = d.kh == 3 && d.kw == 3 && d.stride_h == 2 && d.stride_w == 2 && !(s2env && s2env[0] == '0') &&
          (long long)d.ih * d.iw * 16 < (1ll << 31);
      c->family = ((s1_3x3 || s2_3x3) && !(d.input_z != 0.0f && padded) && d.output_fmt != EHIP_NHWC && d.input_fmt != EHIP_NHWC)
          ? FAM_CONV_3X3 : FAM_GEMM_1X1;
      {
        // at most four input channels: several pixels per operand cell, weights in registers
        const char *env = getenv("EHIP_FEWCH");
        if (conv_fewch_applies(d.ic, d.kh, d.kw) && (d.input_fmt == EHIP_NHWC || !(env && env[0] == '0')))
          c->family = FAM_CONV_FEWCH;
      }
      return EHIP_OK;
    }
    return fail(EHIP_UNIMPLEMENTED, "direct: c160: shape not supported");
  }

  if (d.algorithm == EHIP_CONV_WINOGRAD) {
    if (d.stride_h != 1 || d.stride_w != 1 || d.kh != 3 || d.kw != 3)
      return fail(EHIP_UNIMPLEMENTED, "Algorithm CONV_WINOGRAD: data shape not supported");
    if (d.g != 1) return fail(EHIP_UNIMPLEMENTED, "winograd: groups are not supported");
    // user types (src/eld_conv.cpp:275-305): u8 input with f32 / u8 / s8 output always takes the int8
    // implementation; all-f32 tensors take it when execution_mode says so
    const bool u8_user = in_u8 && (out_q || d.output_type == EHIP_F32);
    if (!all_f32 && !u8_user) return fail(EHIP_UNIMPLEMENTED, "winograd: user types must be f32 or u8 input with f32/u8/s8 output");
    if (all_f32 && (d.execution_mode & 0xF00) != 0x100)
      return fail(EHIP_UNIMPLEMENTED, "winograd: only the int8 implementation (execution_mode 0xa1xx) is built");
    if (out_q && (d.output_scale == kNoCali || d.output_z == kNoCali || d.output_scale == 0.0f))
      return fail(EHIP_GENERAL_ERROR, "output_quant is not set");
    // the reference stops here (el_error, src/eld_conv.cpp:223-228): its transform never reads the zero point
    if (u8_user && d.input_z != 0.0f)
      return fail(EHIP_UNIMPLEMENTED, "Support abs-max scaling for input only in Conv Winograd ...");
    if (d.tile_size == 0) d.tile_size = wino_auto_tile(d);
    // src/eld_conv.cpp:257-270: the int8 executor exists for tile sizes 4, 5 and 6
    if (d.tile_size < 4 || d.tile_size > 6) return fail(EHIP_UNIMPLEMENTED, "Unimplemented tile size");
    if (d.sampling_kind != 2) return fail(EHIP_UNIMPLEMENTED, "Winograd: to enable sampling from elk_u8s8_gemm");
    if (d.input_scale == kNoCali || d.input_z == kNoCali)
      return fail(EHIP_UNIMPLEMENTED, "winograd: input_quant must be set (FINE sampling is not built)");
    if (d.tinput_scale == kNoCali || d.tinput_scale == 0.0f) return fail(EHIP_GENERAL_ERROR, "wino_tinput_quant is not set");
    // activations nChw16c or nhwc (the reference has no channel tails with nhwc, src/elx_int8_conv_wino.cpp:120-125)
    if ((d.input_fmt != EHIP_NCHW16C && d.input_fmt != EHIP_NHWC) || (d.output_fmt != EHIP_NCHW16C && d.output_fmt != EHIP_NHWC) ||
        d.weights_fmt != EHIP_OIHW16I16O)
      return fail(EHIP_UNIMPLEMENTED, "winograd: activations nChw16c or nhwc, weights OIhw16i16o");
    if ((d.input_fmt == EHIP_NHWC && d.ic % 16) || (d.output_fmt == EHIP_NHWC && d.oc % 16))
      return fail(EHIP_UNIMPLEMENTED, "Unimplemented: nhwc with a channel tail");
    if (d.pad_t > 1 || d.pad_l > 1) return fail(EHIP_UNIMPLEMENTED, "winograd: pads > 1");
    c->family = FAM_WINOGRAD;
    return EHIP_OK;
  }
  return fail(EHIP_UNIMPLEMENTED, "algorithm not supported");
}

int setup_workspace(ehip_conv *c)
{
  const ehip_conv_desc_t &d = c->d;
  c->ic2 = up(d.ic, 16) / 16;
  c->oc2 = up(d.oc, 16) / 16;
  int rc;
  switch (c->family) {
  case FAM_CONV_3X3: {
    c->taps = c->gtaps = 9;
    c->nbatch = 1;
    if ((long long)(d.oh + 2) * (d.ow + 2) * (d.ow + 2) >= (1ll << 31))
      return fail(EHIP_UNIMPLEMENTED, "direct 3x3: image too large");
    c->variant = conv3x3v_pick_variant(d.n, d.oh, d.ow, c->oc2, d.stride_h);
    if (c->variant >= 0) {
      c->chunk_units = conv3x3v_chunk_units(c->variant, c->ic2);
      c->units_pad = up(c->ic2, c->chunk_units);
      c->kernel_name = conv3x3v_variant_name(c->variant);
      break;
    }
    c->family = FAM_GEMM_1X1;   // rows too wide for the staged tile: the GEMM form has no such limit
  }
  // fall through
  case FAM_CONV_FEWCH:
  case FAM_GEMM_1X1: {
    if ((long long)d.n * d.oh * d.ow >= (1ll << 30) || (long long)d.oh * d.ow * d.ow >= (1ll << 32))
      return fail(EHIP_UNIMPLEMENTED, "direct: more than 2^30 output pixels");
    c->taps = d.kh * d.kw;
    c->nbatch = 1;
    if (c->taps > 1 && (long long)d.n * c->ic2 * d.ih * d.iw * 16 >= (1ll << 40))
      return fail(EHIP_UNIMPLEMENTED, "direct: input too large");
    c->gtaps = c->taps;
    c->icl = conv_fewch_icl(d.ic, d.kw);
    if (c->family == FAM_CONV_FEWCH &&
        (size_t)d.kh * conv_fewch_row_pitch(c->icl, d.kw, d.iw, d.ow, d.stride_w, d.pad_l) > 48 * 1024) {
      // one strip's input rows do not fit in LDS
      if (d.input_fmt == EHIP_NHWC) return fail(EHIP_UNIMPLEMENTED, "direct: few-channel nhwc input: rows too wide");
      c->family = FAM_GEMM_1X1;
    }
    if (c->family == FAM_CONV_FEWCH) {
      c->ppc = 16 / c->icl;
      c->nu = (d.kw + c->ppc - 1) / c->ppc;
      c->gtaps = d.kh * c->nu;
    }
    c->variant = gemm_pick_variant(d.n * d.oh * d.ow, c->oc2, c->ic2 * c->gtaps, 1, c->taps > 1 ? 1 : d.stride_w);
    // kh x kw: the K axis is [tap][ic2 real units]; only its end is padded to the kernel's chunk
    c->units_pad = c->taps > 1 ? c->ic2 : up(c->ic2, gemm_variant_chunk(c->variant));
    c->kernel_name = gemm_smallk_applies(c->ic2, c->taps, 1) ? "k_gemm_smallk_u8s8" : gemm_variant_name(c->variant);
    if (c->family == FAM_CONV_FEWCH) c->kernel_name = "k_conv_fewch_u8s8";
    if (c->family == FAM_GEMM_1X1 && c->taps == 1 && !gemm_smallk_applies(c->ic2, c->taps, 1)) {
      // many input channels, blocked activations: the kernel that keeps its pixel tile resident
      GemmArgs g;
      memset(&g, 0, sizeof(g));
      g.kh = g.kw = 1;
      g.in_nhwc = d.input_fmt == EHIP_NHWC; g.out_nhwc = d.output_fmt == EHIP_NHWC;
      g.ic2 = c->ic2; g.units_pad = c->units_pad; g.oc2 = c->oc2; g.p_total = d.n * d.oh * d.ow;
      const int rv = gemm1x1_res_pick(g, 1);
      if (rv >= 0) c->kernel_name = gemm1x1_res_name(rv);
    }
    if (c->taps > 1 && d.input_z != 0.0f) {
      // classes of output rows / columns by their range of valid kernel rows / columns
      auto classes = [](int on, int in, int k, int stride, int pad, std::vector<int> &cls, std::vector<std::pair<int, int>> &rng) {
        cls.resize(on);
        for (int o = 0; o < on; ++o) {
          int lo = pad - o * stride; lo = lo < 0 ? 0 : lo;
          int hi = in - 1 + pad - o * stride; hi = hi > k - 1 ? k - 1 : hi;
          const std::pair<int, int> r(lo, hi);
          size_t i = 0;
          while (i < rng.size() && rng[i] != r) ++i;
          if (i == rng.size()) rng.push_back(r);
          cls[o] = (int)i;
        }
      };
      std::vector<int> ch, cw;
      std::vector<std::pair<int, int>> rh, rw;
      classes(d.oh, d.ih, d.kh, d.stride_h, d.pad_t, ch, rh);
      classes(d.ow, d.iw, d.kw, d.stride_w, d.pad_l, cw, rw);
      if (rh.size() * rw.size() > 1) {
        c->ncls_w = (int)rw.size();
        c->nclass = (int)(rh.size() * rw.size());
        std::vector<int> rects((size_t)c->nclass * 4);
        for (size_t i = 0; i < rh.size(); ++i)
          for (size_t j = 0; j < rw.size(); ++j) {
            int *r = &rects[(i * rw.size() + j) * 4];
            r[0] = rh[i].first; r[1] = rh[i].second; r[2] = rw[j].first; r[3] = rw[j].second;
          }
        if ((rc = dev_alloc(&c->cls_h, ch.size(), false)) != EHIP_OK) return rc;
        if ((rc = dev_alloc(&c->cls_w, cw.size(), false)) != EHIP_OK) return rc;
        if ((rc = dev_alloc(&c->rects, rects.size(), false)) != EHIP_OK) return rc;
        HIP_TRY(hipMemcpy(c->cls_h, ch.data(), ch.size() * sizeof(int), hipMemcpyHostToDevice));
        HIP_TRY(hipMemcpy(c->cls_w, cw.data(), cw.size() * sizeof(int), hipMemcpyHostToDevice));
        HIP_TRY(hipMemcpy(c->rects, rects.data(), rects.size() * sizeof(int), hipMemcpyHostToDevice));
      }
    }
    break;
  }
  case FAM_DEPTHWISE: {
    c->taps = 9;
    c->oc2 = c->ic2 = up(d.g, 16) / 16;
    c->T = d.flatting_t > 0 ? (d.flatting_t > d.ow ? d.ow : d.flatting_t) : 1;
    c->wtb = (d.ow + c->T - 1) / c->T;
    c->Tr = d.ow % c->T ? d.ow % c->T : c->T;
    // what the depthwise launchers pack into 16 or 8 bits and address with 32: refused here, at setup, so that a
    // handle that was created also executes
    if (d.ih >= 65536 || d.iw >= 65536 || d.oh >= 65536 || d.ow >= 65536 || d.pad_t > 255 || d.pad_l > 255 ||
        (long long)d.n * c->oc2 * d.oh * d.ow >= (1ll << 28) || (long long)d.n * c->oc2 * d.ih * d.iw >= (1ll << 28))
      return fail(EHIP_UNIMPLEMENTED, "direct_depthwise: tensor too large");
    c->kernel_name = depthwise_mfma_applies(d.stride_h, d.oh, d.ow, d.pad_t, d.pad_l, d.output_type, d.with_relu, d.relu_lower,
                                            d.relu_upper, (long long)d.n * c->oc2, d.ih, d.iw)
        ? "k_depthwise3x3_mfma" : "k_depthwise3x3_u8s8";
    break;
  }
  case FAM_WINOGRAD: {
    c->taps = 1;
    c->wino_tile = d.tile_size;
    c->nbatch = d.tile_size * d.tile_size;
    c->ht = (d.oh + d.tile_size - 3) / (d.tile_size - 2);
    c->wt = (d.ow + d.tile_size - 3) / (d.tile_size - 2);
    c->nt = c->ht * c->wt;
    // One pass over the whole batch.  (Running the stages over a few images at a time, with the intermediates
    // sized for one pass, was measured on MI355X and only costs: the 256 MB memory-side cache does not keep the
    // intermediates away from HBM.  The pass loop of execute stays: chunk_n images per pass.)
    c->chunk_n = d.n;
    c->t = c->nt * c->chunk_n;   // tiles per pass
    if ((long long)c->t >= (1ll << 31) / 64) return fail(EHIP_UNIMPLEMENTED, "winograd: too many tiles");
    c->variant = gemm_pick_variant(c->t, c->oc2, c->ic2, c->nbatch, 1);
    c->units_pad = up(c->ic2, gemm_variant_chunk(c->variant));
    {
      const char *env = getenv("EHIP_WINO_FUSED");
      // every tile size, with or without the in-place sum, runs the fused GEMM + output transform, as the
      // reference's a161 schedule does (src/eld_conv.cpp:255-281); EHIP_WINO_FUSED=0 keeps the three kernels
      c->fused = !(env && env[0] == '0');
    }
    c->kernel_name = c->fused ? std::string("k_wino_trans_input_u8 + k_wino_gemm_output")
                              : std::string("k_wino_trans_input_u8 + ") + gemm_variant_name(c->variant) + " + k_wino_trans_output";
    c->tin_blocked = c->fused;   // the fused schedule's layout: a workgroup's whole input is one contiguous run
    // (blocked: whole blocks of 32 tiles)  allocated with one pad unit behind it
    c->tin_bytes = (size_t)c->nbatch * c->ic2 * (c->tin_blocked ? up(c->t, 32) : c->t) * 16;
    c->tout_bytes = c->fused ? 16 : (size_t)c->nbatch * c->oc2 * c->t * 16 * sizeof(float);
    if (c->fused) {   // (the fused stage's own parking space, where its kernel asks for one)
      const size_t park = wino_lanes_tpart_bytes(d.tile_size, c->ic2, c->oc2, c->t);
      if (park > c->tout_bytes) c->tout_bytes = park;
    }
    // (the pad: an odd unit count makes the last k-step read one unit past its position -- in the blocked layout
    // 512 bytes past the last one, multiplied by zero weights)
    if ((rc = dev_alloc(&c->tin, c->tin_bytes + ((size_t)c->t * 16 > 1024 ? (size_t)c->t * 16 : 1024), true)) != EHIP_OK) return rc;
    if ((rc = dev_alloc(reinterpret_cast<uint8_t **>(&c->tout), c->tout_bytes, false)) != EHIP_OK) return rc;
    break;
  }
  default:
    return fail(EHIP_GENERAL_ERROR, "internal: no executor");
  }

  if (c->family == FAM_DEPTHWISE) {
    c->ocpp = c->oc2 * 16;
    // [g2][kh][16][4] s8, then the matrix-core kernel's diagonal A operands [g2][6][64][16 bytes]
    c->wpacked_bytes = (size_t)c->oc2 * 3 * 16 * 4 + (size_t)c->oc2 * 6 * 64 * 16;
  } else {
    c->ocpp = up(c->oc2 * 16, kOcTile);
    // (the K loop may run up to one chunk of 8 units past the last real one: zero rows)
    c->wpacked_bytes = (size_t)c->nbatch * up(c->gtaps * c->units_pad, 8) * c->ocpp * 16;
  }
  c->per_oc = (size_t)c->nbatch * c->ocpp;
  if ((rc = dev_alloc(&c->wpacked, c->wpacked_bytes, true)) != EHIP_OK) return rc;
  // scale, shift and compensation back to back, [3][per_oc]: a kernel can take them as one pointer among its
  // preloaded leading arguments and ask for all three before the rest of its argument block has arrived
  if ((rc = dev_alloc(&c->scale, 3 * c->per_oc, true)) != EHIP_OK) return rc;
  c->shift = c->scale + c->per_oc;
  c->comp = reinterpret_cast<int *>(c->scale + 2 * c->per_oc);
  if ((rc = dev_alloc(&c->absmax, c->per_oc, true)) != EHIP_OK) return rc;
  if ((rc = dev_alloc(&c->wsum, c->per_oc, true)) != EHIP_OK) return rc;
  if (c->nclass > 1 && (rc = dev_alloc(&c->shift_tab, (size_t)c->nclass * c->ocpp, true)) != EHIP_OK) return rc;
  return EHIP_OK;
}

Epilogue make_epilogue(const ehip_conv *c, int out_type, bool sum, bool relu)
{
  Epilogue e;
  e.scale = c->scale;
  e.shift = c->shift;
  e.comp = c->comp;
  e.sum_scale = c->d.sum_scale;
  e.lo = c->d.relu_lower;
  e.hi = c->d.relu_upper;
  e.out_type = out_type;
  e.with_sum = sum ? 1 : 0;
  e.with_relu = relu ? 1 : 0;
  e.shift_tab = nullptr;
  e.tab_stride = 0;
  return e;
}

WinoArgs make_wino_args(const ehip_conv_desc_t &d, int ic2, int oc2)
{
  WinoArgs w;
  memset(&w, 0, sizeof(w));
  w.n = d.n; w.ic2 = ic2; w.oc2 = oc2;
  w.ih = d.ih; w.iw = d.iw; w.oh = d.oh; w.ow = d.ow;
  w.tile = d.tile_size == 0 ? wino_auto_tile(d) : d.tile_size;
  w.ht = (d.oh + w.tile - 3) / (w.tile - 2); w.wt = (d.ow + w.tile - 3) / (w.tile - 2);
  w.nt = w.ht * w.wt; w.t = w.nt * d.n;
  w.pad_t = d.pad_t; w.pad_l = d.pad_l;
  w.with_bias = d.with_bias; w.with_relu = d.with_relu; w.with_sum = d.with_ip_sum;
  w.in_nhwc = d.input_fmt == EHIP_NHWC; w.out_nhwc = d.output_fmt == EHIP_NHWC;
  w.in_u8 = d.input_type == EHIP_U8;
  w.out_type = d.output_type;
  if (d.output_type == EHIP_U8 || d.output_type == EHIP_S8) {
    // src/elx_int8_conv_wino.cpp:272-276
    w.out_repS = 1.0f / d.output_scale;
    w.out_z = ceilf(d.output_z);
  }
  return w;
}

}  // namespace

extern "C" {

EHIP_API const char *ehip_last_error(void) { return g_last_error.c_str(); }

EHIP_API int ehip_init(int device)
{
  HIP_TRY(hipSetDevice(device));
  hipDeviceProp_t prop;
  HIP_TRY(hipGetDeviceProperties(&prop, device));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return fail(EHIP_GENERAL_ERROR, std::string("this library is built for gfx950 only, device is ") + prop.gcnArchName);
  // the device's address of the static range scratch, so that the first allocation-free call need not ask
  unsigned *scratch_dev = nullptr;
  HIP_TRY(wino_range_scratch(&scratch_dev));
  return EHIP_OK;
}

EHIP_API int ehip_conv_create(const ehip_conv_desc_t *desc, ehip_conv_t **out)
{
  if (!desc || !out) return fail(EHIP_GENERAL_ERROR, "null argument");
  *out = nullptr;
  ehip_conv *c = new ehip_conv();
  c->d = *desc;
  int rc = classify(c);
  if (rc == EHIP_OK) rc = setup_workspace(c);
  if (rc != EHIP_OK) {
    free_all(c);
    delete c;
    return rc;
  }
  *out = c;
  return EHIP_OK;
}

EHIP_API int ehip_conv_destroy(ehip_conv_t *c)
{
  if (!c) return EHIP_OK;
  free_all(c);
  delete c;
  return EHIP_OK;
}

EHIP_API const char *ehip_conv_kernel_name(ehip_conv_t *c) { return c ? c->kernel_name.c_str() : ""; }

EHIP_API int ehip_conv_prepare(ehip_conv_t *c, const void *weights_dev, const void *bias_dev, void *hip_stream)
{
  if (!c || !weights_dev) return fail(EHIP_GENERAL_ERROR, "Parameter error. Invalid input data!");
  if (c->d.with_bias && !bias_dev) return fail(EHIP_GENERAL_ERROR, "Parameter error. Invalid input data!");
  hipStream_t s = static_cast<hipStream_t>(hip_stream);
  const ehip_conv_desc_t &d = c->d;
  const float *w = static_cast<const float *>(weights_dev);
  const float *b = static_cast<const float *>(bias_dev);
  switch (c->family) {
  case FAM_CONV_FEWCH:
  case FAM_GEMM_1X1:
  case FAM_CONV_3X3:
    if (c->family == FAM_CONV_FEWCH) {
      HIP_TRY(launch_prepare_direct_px(w, b, d.oc, d.ic, c->icl, d.kh, d.kw, c->ppc, c->nu, c->ocpp, d, c->absmax, c->wpacked,
                                       c->scale, c->shift, c->wsum, c->comp, s));
      if (c->nclass > 1)
        HIP_TRY(launch_fold_direct_border_px(c->wpacked, c->absmax, b, d.oc, c->icl, c->ppc, c->nu, c->ocpp, d, c->rects,
                                             c->nclass, c->shift_tab, s));
      break;
    }
    HIP_TRY(launch_prepare_direct(w, b, d.oc, d.ic, d.kh, d.kw, c->units_pad, c->ocpp, d, c->absmax, c->wpacked,
                                  c->scale, c->shift, c->wsum, c->comp, s));
    if (c->nclass > 1)
      HIP_TRY(launch_fold_direct_border(c->wpacked, c->absmax, b, d.oc, d.kw, c->units_pad, c->ocpp, d, c->rects,
                                        c->nclass, c->shift_tab, s));
    break;
  case FAM_DEPTHWISE:
    HIP_TRY(launch_prepare_depthwise(w, b, d.g, d, c->wpacked, c->scale, c->shift, c->wsum, s));
    HIP_TRY(launch_depthwise_diag(c->wpacked, c->oc2, c->wpacked + (size_t)c->oc2 * 192, s));
    break;
  case FAM_WINOGRAD: {
    float *u_tmp = nullptr;
    const size_t n = (size_t)c->nbatch * up(d.oc, 16) * up(d.ic, 16);
    HIP_TRY(hipMalloc(reinterpret_cast<void **>(&u_tmp), n * sizeof(float)));
    hipError_t e = launch_prepare_wino(w, d.oc, d.ic, c->wino_tile, c->units_pad, c->ocpp, d, u_tmp, c->wpacked, c->scale,
                                       c->shift, c->wsum, c->comp, s);
    hipError_t e2 = hipStreamSynchronize(s);
    (void)hipFree(u_tmp);
    HIP_TRY(e);
    HIP_TRY(e2);
    break;
  }
  default:
    return fail(EHIP_GENERAL_ERROR, "internal: no executor");
  }
  c->prepared = true;
  return EHIP_OK;
}

// Development aid: a build with -DEHIP_TRACE takes the address of a device buffer for the kernels' clock
// stamps from the environment; the product build passes null and never looks.
static long long *trace_buffer()
{
#ifdef EHIP_TRACE
  const char *env = getenv("EHIP_TRACE_PTR");
  return reinterpret_cast<long long *>(env ? strtoull(env, nullptr, 0) : 0ull);
#else
  return nullptr;
#endif
}

EHIP_API int ehip_conv_execute(ehip_conv_t *c, void *output_dev, const void *input_dev, const void *weights_dev,
                               const void *bias_dev, void *hip_stream)
{
  if (!c || !output_dev || !input_dev) return fail(EHIP_GENERAL_ERROR, "Parameter error. Invalid input data!");
  if (!c->prepared) {
    int rc = ehip_conv_prepare(c, weights_dev, bias_dev, hip_stream);
    if (rc != EHIP_OK) return rc;
  }
  hipStream_t s = static_cast<hipStream_t>(hip_stream);
  const ehip_conv_desc_t &d = c->d;
  switch (c->family) {
  case FAM_GEMM_1X1: {
    GemmArgs a;
    memset(&a, 0, sizeof(a));
    a.in = static_cast<const uint8_t *>(input_dev);
    a.w = c->wpacked;
    a.out = output_dev;
    a.ep = make_epilogue(c, d.output_type, d.with_ip_sum && d.algorithm == EHIP_CONV_DIRECT_1X1, d.with_relu);
    a.p_total = d.n * d.oh * d.ow;
    a.ohw = d.oh * d.ow; a.ow = d.ow;
    a.ohw_magic = div_magic(a.ohw); a.ow_magic = div_magic(a.ow);
    a.ihw = d.ih * d.iw; a.iw = d.iw;
    a.stride_h = d.stride_h; a.stride_w = d.stride_w;
    a.ic2 = c->ic2; a.units_pad = c->units_pad; a.oc2 = c->oc2; a.ocpp = c->ocpp;
    a.in_nhwc = d.input_fmt == EHIP_NHWC; a.out_nhwc = d.output_fmt == EHIP_NHWC;
    a.kh = d.kh; a.kw = d.kw; a.pad_t = d.pad_t; a.pad_l = d.pad_l; a.ih = d.ih;
    if (c->nclass > 1) {
      a.ep.shift_tab = c->shift_tab; a.ep.tab_stride = c->ocpp;
      a.cls_h = c->cls_h; a.cls_w = c->cls_w; a.ncls_w = c->ncls_w;
    }
    a.trace = trace_buffer();
    HIP_TRY(launch_gemm(a, 1, c->variant, s, &c->plan_gemm));
    if (c->plan_gemm.name) c->kernel_name = c->plan_gemm.name;   // the launcher's choice depends on the epilogue
    break;
  }
  case FAM_CONV_FEWCH: {
    FewChArgs a;
    memset(&a, 0, sizeof(a));
    a.in = static_cast<const uint8_t *>(input_dev);
    a.w = c->wpacked;
    a.out = output_dev;
    a.ep = make_epilogue(c, d.output_type, false, d.with_relu);
    a.n = d.n; a.ih = d.ih; a.iw = d.iw; a.oh = d.oh; a.ow = d.ow; a.ic = d.ic; a.kh = d.kh; a.kw = d.kw;
    a.stride_h = d.stride_h; a.stride_w = d.stride_w; a.pad_t = d.pad_t; a.pad_l = d.pad_l;
    a.oc2 = c->oc2; a.ocpp = c->ocpp; a.icl = c->icl;
    a.in_nhwc = d.input_fmt == EHIP_NHWC; a.out_nhwc = d.output_fmt == EHIP_NHWC;
    if (c->nclass > 1) {
      a.ep.shift_tab = c->shift_tab; a.ep.tab_stride = c->ocpp;
      a.cls_h = c->cls_h; a.cls_w = c->cls_w; a.ncls_w = c->ncls_w; a.nclass = c->nclass;
    }
    if (a.in_nhwc && (reinterpret_cast<uintptr_t>(input_dev) & 3))
      return fail(EHIP_GENERAL_ERROR, "nhwc input of a few-channel layer must be 4-byte aligned");
    HIP_TRY(launch_conv_fewch(a, s, &c->plan_fewch));
    if (c->plan_fewch.name) c->kernel_name = c->plan_fewch.name;
    break;
  }
  case FAM_CONV_3X3: {
    Conv3x3Args a;
    memset(&a, 0, sizeof(a));
    a.in = static_cast<const uint8_t *>(input_dev);
    a.w = c->wpacked;
    a.out = output_dev;
    a.ep = make_epilogue(c, d.output_type, false, d.with_relu);
    a.ih = d.ih; a.iw = d.iw; a.oh = d.oh; a.ow = d.ow;
    a.pad_t = d.pad_t; a.pad_l = d.pad_l;
    a.ic2 = c->ic2; a.units_pad = c->units_pad; a.oc2 = c->oc2; a.ocpp = c->ocpp;
    a.chunk_units = c->chunk_units;
    a.vw = d.stride_h == 2 ? d.ow + 1 : d.ow + 2;
    a.vw_magic = div_magic(a.vw);
    a.trace = trace_buffer();
    HIP_TRY(launch_conv3x3v(a, d.n, c->variant, s, &c->plan_3x3));
    break;
  }
  case FAM_DEPTHWISE: {
    DepthwiseArgs a;
    memset(&a, 0, sizeof(a));
    a.in = static_cast<const uint8_t *>(input_dev);
    a.w = c->wpacked;
    a.out = output_dev;
    a.scale = c->scale; a.shift = c->shift; a.wsum = c->wsum;
    a.wdiag = reinterpret_cast<const uint4 *>(c->wpacked + (size_t)c->oc2 * 192);
    a.n = d.n; a.g2 = c->oc2; a.ih = d.ih; a.iw = d.iw; a.oh = d.oh; a.ow = d.ow;
    a.stride = d.stride_h;
    a.pad_t = d.pad_t; a.pad_l = d.pad_l;
    a.T = c->T; a.Tr = c->Tr; a.wt = c->wtb;
    a.out_type = d.output_type; a.with_relu = d.with_relu;
    a.lo = d.relu_lower; a.hi = d.relu_upper;
    HIP_TRY(launch_depthwise(a, s, &c->plan_dw));
    break;
  }
  case FAM_WINOGRAD: {
    if (d.with_bias && !bias_dev) return fail(EHIP_GENERAL_ERROR, "Parameter error. Invalid input data!");
    const bool one_pass = c->chunk_n >= d.n;   // the launch plans hold ONE pass's arguments
    for (int n0 = 0; n0 < d.n; n0 += c->chunk_n) {
      ehip_conv_desc_t dc = d;
      dc.n = d.n - n0 < c->chunk_n ? d.n - n0 : c->chunk_n;
      WinoArgs w = make_wino_args(dc, c->ic2, c->oc2);
      const size_t in_esz = d.input_type == EHIP_U8 ? 1 : 4, out_esz = d.output_type == EHIP_F32 ? 4 : 1;
      w.in = static_cast<const uint8_t *>(input_dev) + (size_t)n0 * c->ic2 * d.ih * d.iw * 16 * in_esz;
      w.tin = c->tin;
      w.tin_blocked = c->tin_blocked;
      w.tout = c->tout;
      w.out = static_cast<uint8_t *>(output_dev) + (size_t)n0 * c->oc2 * d.oh * d.ow * 16 * out_esz;
      w.bias = static_cast<const float *>(bias_dev);
      // mrepS = input_S * (1 / tinput_S), z = ceil(tinput_z)
      // (src/elx_conv_wino_trans_input.cpp:617-618, src/elx_int8_conv_wino.cpp:270-276)
      const float tin_repS = 1.0f / d.tinput_scale;
      w.mrepS = d.input_scale * tin_repS;
      w.mz = ceilf(d.tinput_z);
      if (c->stage_mask & 1) HIP_TRY(launch_wino_trans_input(w, s, one_pass ? &c->plan_wino_in : nullptr));
      if (c->fused) {
        if (!(c->stage_mask & 2)) continue;
        WinoFusedArgs f;
        memset(&f, 0, sizeof(f));
        f.tin = c->tin; f.tin_blocked = c->tin_blocked; f.w = c->wpacked; f.out = w.out; f.bias = w.bias;
        f.scale = c->scale; f.shift = c->shift; f.comp = c->comp;
        f.n = w.n; f.ic2 = c->ic2; f.units_pad = c->units_pad; f.oc2 = c->oc2; f.ocpp = c->ocpp;
        f.oh = d.oh; f.ow = d.ow; f.ht = w.ht; f.wt = w.wt; f.nt = w.nt; f.t = w.t;
        f.with_bias = d.with_bias; f.with_relu = d.with_relu; f.with_sum = d.with_ip_sum; f.tile = d.tile_size;
        f.out_type = w.out_type; f.out_repS = w.out_repS; f.out_z = w.out_z;
        f.out_nhwc = w.out_nhwc;
        f.tpart = c->tout_bytes > 16 ? reinterpret_cast<float4 *>(c->tout) : nullptr;
        f.trace = trace_buffer();
        HIP_TRY(launch_wino_gemm_output(f, s, one_pass ? &c->plan_wino_fused : nullptr));
        // (which form of the fused stage runs is the launcher's choice: known from the first execute on)
        if (c->plan_wino_fused.name && c->kernel_name.find(c->plan_wino_fused.name) == std::string::npos)
          c->kernel_name = std::string("k_wino_trans_input_u8 + ") + c->plan_wino_fused.name;
        continue;
      }
      GemmArgs a;
      memset(&a, 0, sizeof(a));
      a.in = c->tin;
      a.w = c->wpacked;
      a.out = c->tout;
      a.ep = make_epilogue(c, EHIP_F32, false, false);
      a.p_total = w.t;
      a.ohw = w.t; a.ow = w.t; a.ihw = w.t; a.iw = w.t;
      a.ohw_magic = div_magic(a.ohw); a.ow_magic = div_magic(a.ow);
      a.stride_h = 1; a.stride_w = 1;
      a.ic2 = c->ic2; a.units_pad = c->units_pad; a.oc2 = c->oc2; a.ocpp = c->ocpp;
      a.in_batch_stride = (long long)c->ic2 * w.t * 16;
      a.out_batch_stride = (long long)c->oc2 * w.t * 16;
      if (c->stage_mask & 2) HIP_TRY(launch_gemm(a, c->nbatch, c->variant, s, one_pass ? &c->plan_gemm : nullptr));
      if (c->stage_mask & 4) HIP_TRY(launch_wino_trans_output(w, s, one_pass ? &c->plan_wino_out : nullptr));
    }
    break;
  }
  default:
    return fail(EHIP_GENERAL_ERROR, "internal: no executor");
  }
  return EHIP_OK;
}

EHIP_API int ehip_conv_execute_stages(ehip_conv_t *c, void *output_dev, const void *input_dev, const void *bias_dev,
                                      int stages, int count, void *hip_stream)
{
  if (!c || !c->prepared) return fail(EHIP_GENERAL_ERROR, "execute_stages needs a prepared handle");
  if (c->family != FAM_WINOGRAD) return fail(EHIP_GENERAL_ERROR, "execute_stages: not a Winograd layer");
  if (stages < 1 || stages > 7) return fail(EHIP_GENERAL_ERROR, "execute_stages: stages is a mask of 1 | 2 | 4");
  c->stage_mask = stages;
  int rc = EHIP_OK;
  for (int i = 0; i < count && rc == EHIP_OK; ++i) rc = ehip_conv_execute(c, output_dev, input_dev, nullptr, bias_dev, hip_stream);
  c->stage_mask = 7;
  return rc;
}

EHIP_API int ehip_conv_execute_repeat(ehip_conv_t *c, void *output_dev, const void *input_dev,
                                      const void *bias_dev, int count, void *hip_stream)
{
  if (!c || !c->prepared) return fail(EHIP_GENERAL_ERROR, "execute_repeat needs a prepared handle");
  for (int i = 0; i < count; ++i) {
    const int rc = ehip_conv_execute(c, output_dev, input_dev, nullptr, bias_dev, hip_stream);
    if (rc != EHIP_OK) return rc;
  }
  return EHIP_OK;
}

EHIP_API int ehip_conv_query(ehip_conv_t *c, int what, void *host_dst, size_t *bytes)
{
  if (!c) return fail(EHIP_GENERAL_ERROR, "null handle");
  const ehip_conv_desc_t &d = c->d;
  const int ocp = c->oc2 * 16, icp = c->ic2 * 16;
  HIP_TRY(hipDeviceSynchronize());
  auto want = [&](size_t n) {
    if (bytes) *bytes = n;
    return host_dst != nullptr;
  };
  switch (what) {
  case EHIP_Q_WEIGHTS_S8: {
    if (!c->prepared) return fail(EHIP_GENERAL_ERROR, "not prepared");
    std::vector<int8_t> packed(c->wpacked_bytes);
    if (c->family == FAM_DEPTHWISE) {
      if (!want((size_t)ocp * 9)) return EHIP_OK;
      HIP_TRY(hipMemcpy(packed.data(), c->wpacked, c->wpacked_bytes, hipMemcpyDeviceToHost));
      int8_t *dst = static_cast<int8_t *>(host_dst);
      for (int g = 0; g < ocp; ++g)
        for (int k = 0; k < 9; ++k) dst[(size_t)g * 9 + k] = packed[(((size_t)(g >> 4) * 3 + k / 3) * 16 + (g & 15)) * 4 + k % 3];
      return EHIP_OK;
    }
    const int taps = c->taps;
    if (!want((size_t)c->nbatch * ocp * icp * taps)) return EHIP_OK;
    HIP_TRY(hipMemcpy(packed.data(), c->wpacked, c->wpacked_bytes, hipMemcpyDeviceToHost));
    int8_t *dst = static_cast<int8_t *>(host_dst);
    if (c->family == FAM_CONV_FEWCH) {
      for (int oc = 0; oc < ocp; ++oc)
        for (int ic = 0; ic < icp; ++ic)
          for (int tap = 0; tap < taps; ++tap) {
            const int kh = tap / d.kw, kw = tap % d.kw, j = kw / c->ppc, byte = (kw % c->ppc) * c->icl + ic;
            dst[((size_t)oc * icp + ic) * taps + tap] =
                ic < d.ic ? packed[((size_t)(kh * c->nu + j) * c->ocpp + packed_row_of_oc(oc)) * 16 + byte] : 0;
          }
      return EHIP_OK;
    }
    for (int b = 0; b < c->nbatch; ++b)
      for (int oc = 0; oc < ocp; ++oc)
        for (int ic = 0; ic < icp; ++ic)
          for (int tap = 0; tap < taps; ++tap)
            dst[(((size_t)b * ocp + oc) * icp + ic) * taps + tap] =
                packed[((((size_t)b * taps + tap) * c->units_pad + (ic >> 4)) * c->ocpp + packed_row_of_oc(oc)) * 16 + (ic & 15)];
    return EHIP_OK;
  }
  case EHIP_Q_SCALE:
  case EHIP_Q_SHIFT:
  case EHIP_Q_WSUM: {
    if (!c->prepared) return fail(EHIP_GENERAL_ERROR, "not prepared");
    if (!want((size_t)c->nbatch * ocp * 4)) return EHIP_OK;
    const void *src = what == EHIP_Q_SCALE ? (const void *)c->scale
        : what == EHIP_Q_SHIFT ? (const void *)c->shift : (const void *)c->wsum;
    std::vector<uint32_t> tmp(c->per_oc);
    HIP_TRY(hipMemcpy(tmp.data(), src, c->per_oc * 4, hipMemcpyDeviceToHost));
    uint32_t *dst = static_cast<uint32_t *>(host_dst);
    for (int b = 0; b < c->nbatch; ++b)
      for (int oc = 0; oc < ocp; ++oc) dst[(size_t)b * ocp + oc] = tmp[(size_t)b * c->ocpp + oc];
    return EHIP_OK;
  }
  case EHIP_Q_TINPUT_U8:
    if (c->family != FAM_WINOGRAD) return fail(EHIP_GENERAL_ERROR, "not a Winograd handle");
    if (c->chunk_n < d.n) return fail(EHIP_UNIMPLEMENTED, "the intermediates of a multi-pass layer hold its last pass only");
    if (c->tin_blocked) {   // back to the canonical [pos][ic2][t][16]
      const size_t canon = (size_t)c->nbatch * c->ic2 * c->t * 16;
      if (!want(canon)) return EHIP_OK;
      std::vector<uint8_t> raw(c->tin_bytes);
      HIP_TRY(hipMemcpy(raw.data(), c->tin, c->tin_bytes, hipMemcpyDeviceToHost));
      uint8_t *dst = static_cast<uint8_t *>(host_dst);
      for (int p = 0; p < c->nbatch; ++p)
        for (int u = 0; u < c->ic2; ++u)
          for (int t = 0; t < c->t; ++t)
            memcpy(dst + (((size_t)p * c->ic2 + u) * c->t + t) * 16,
                   raw.data() + ((((size_t)(t >> 5) * c->nbatch + p) * c->ic2 + u) * 32 + (t & 31)) * 16, 16);
      return EHIP_OK;
    }
    if (!want(c->tin_bytes)) return EHIP_OK;
    HIP_TRY(hipMemcpy(host_dst, c->tin, c->tin_bytes, hipMemcpyDeviceToHost));
    return EHIP_OK;
  case EHIP_Q_TOUTPUT_F32:
    if (c->family != FAM_WINOGRAD) return fail(EHIP_GENERAL_ERROR, "not a Winograd handle");
    if (c->chunk_n < d.n) return fail(EHIP_UNIMPLEMENTED, "the intermediates of a multi-pass layer hold its last pass only");
    if (c->fused) return fail(EHIP_UNIMPLEMENTED, "the fused schedule keeps the GEMM result on chip (set EHIP_WINO_FUSED=0)");
    if (!want(c->tout_bytes)) return EHIP_OK;
    HIP_TRY(hipMemcpy(host_dst, c->tout, c->tout_bytes, hipMemcpyDeviceToHost));
    return EHIP_OK;
  default:
    (void)d;
    return fail(EHIP_GENERAL_ERROR, "unknown query");
  }
}

EHIP_API int ehip_quantize_input_u8(void *dst_dev, const void *src_dev, size_t count, float scale, float z,
                                    void *hip_stream)
{
  if (!dst_dev || !src_dev) return fail(EHIP_GENERAL_ERROR, "null argument");
  if (scale == 0.0f) return fail(EHIP_GENERAL_ERROR, "scale is zero");
  HIP_TRY(launch_quantize_input(static_cast<uint8_t *>(dst_dev), static_cast<const float *>(src_dev), count, scale, z,
                                static_cast<hipStream_t>(hip_stream)));
  return EHIP_OK;
}

// shared by the two range entry points: descriptor checks and the kernel's arguments
static int range_args(const ehip_conv_desc_t *desc, const void *input_dev, WinoArgs *w)
{
  if (!desc || !input_dev) return fail(EHIP_GENERAL_ERROR, "null argument");
  const ehip_conv_desc_t &d = *desc;
  if (d.kh != 3 || d.kw != 3 || d.stride_h != 1 || d.stride_w != 1 ||
      (d.input_type != EHIP_F32 && d.input_type != EHIP_U8) ||
      (d.input_fmt != EHIP_NCHW16C && !(d.input_fmt == EHIP_NHWC && d.ic % 16 == 0)))
    return fail(EHIP_UNIMPLEMENTED, "tinput range: fp32 or u8 3x3 stride-1 layers, nChw16c or nhwc without a channel tail");
  if (d.tile_size != 0 && (d.tile_size < 4 || d.tile_size > 6)) return fail(EHIP_UNIMPLEMENTED, "Unimplemented tile size");
  if (d.n < 1 || d.ic < 1 || d.oh < 1 || d.ow < 1 || d.ih < 1 || d.iw < 1) return fail(EHIP_GENERAL_ERROR, "tinput range: empty tensor");
  *w = make_wino_args(d, up(d.ic, 16) / 16, up(d.oc, 16) / 16);
  if ((long long)w->nt * d.n >= (1ll << 31) / 64) return fail(EHIP_UNIMPLEMENTED, "tinput range: too many tiles");
  if (w->ic2 > 65535) return fail(EHIP_UNIMPLEMENTED, "tinput range: more than 65535 x 16 input channels");
  w->in = input_dev;
  return EHIP_OK;
}

EHIP_API int ehip_wino_tinput_range(const ehip_conv_desc_t *desc, const void *input_dev, float *min_out,
                                    float *max_out)
{
  if (!min_out || !max_out) return fail(EHIP_GENERAL_ERROR, "null argument");
  WinoArgs w;
  int rc = range_args(desc, input_dev, &w);
  if (rc != EHIP_OK) return rc;
  // per-unit partial results and, behind them, the two floats of the result
  unsigned *mm = nullptr;
  HIP_TRY(hipMalloc(reinterpret_cast<void **>(&mm), (2 * (size_t)w.ic2 + 2) * sizeof(unsigned)));
  hipError_t e = launch_wino_range(w, desc->ic, mm, reinterpret_cast<float *>(mm + 2 * (size_t)w.ic2), nullptr);
  float res[2] = {0.f, 0.f};
  if (e == hipSuccess) e = hipMemcpy(res, mm + 2 * (size_t)w.ic2, sizeof(res), hipMemcpyDeviceToHost);
  (void)hipFree(mm);
  HIP_TRY(e);
  *min_out = res[0];
  *max_out = res[1];
  return EHIP_OK;
}

EHIP_API int ehip_wino_tinput_range_noalloc(const ehip_conv_desc_t *desc, const void *input_dev, float *minmax_out_dev,
                                            void *hip_stream)
{
  if (!minmax_out_dev) return fail(EHIP_GENERAL_ERROR, "null argument");
  WinoArgs w;
  int rc = range_args(desc, input_dev, &w);
  if (rc != EHIP_OK) return rc;
  if (w.ic2 > kRangeScratchUnits)
    return fail(EHIP_UNIMPLEMENTED, "tinput range without allocation: at most " + std::to_string(kRangeScratchUnits * 16) +
                " input channels (the static scratch holds " + std::to_string(kRangeScratchUnits) + " units); got " +
                std::to_string(desc->ic));
  unsigned *partials = nullptr;
  HIP_TRY(wino_range_scratch(&partials));
  HIP_TRY(launch_wino_range(w, desc->ic, partials, minmax_out_dev, static_cast<hipStream_t>(hip_stream)));
  return EHIP_OK;
}

EHIP_API int ehip_reorder_nchw_to_blocked(void *dst_dev, const void *src_dev, int elem_size, int n, int c, int h,
                                          int w, void *hip_stream)
{
  if (!dst_dev || !src_dev || (elem_size != 1 && elem_size != 4)) return fail(EHIP_GENERAL_ERROR, "bad argument");
  HIP_TRY(launch_reorder_nchw_to_blocked(dst_dev, src_dev, elem_size, n, c, h, w, static_cast<hipStream_t>(hip_stream)));
  return EHIP_OK;
}

EHIP_API int ehip_reorder_blocked_to_nchw(void *dst_dev, const void *src_dev, int elem_size, int n, int c, int h,
                                          int w, void *hip_stream)
{
  if (!dst_dev || !src_dev || (elem_size != 1 && elem_size != 4)) return fail(EHIP_GENERAL_ERROR, "bad argument");
  HIP_TRY(launch_reorder_blocked_to_nchw(dst_dev, src_dev, elem_size, n, c, h, w, static_cast<hipStream_t>(hip_stream)));
  return EHIP_OK;
}

EHIP_API int ehip_reorder_oihw_to_blocked(void *dst_dev, const void *src_dev, int o, int i, int h, int w,
                                          void *hip_stream)
{
  if (!dst_dev || !src_dev) return fail(EHIP_GENERAL_ERROR, "bad argument");
  HIP_TRY(launch_reorder_oihw_to_blocked(static_cast<float *>(dst_dev), static_cast<const float *>(src_dev), o, i, h, w,
                                         static_cast<hipStream_t>(hip_stream)));
  return EHIP_OK;
}

}  // extern "C"

// ---- harness calibration (tests/elt_conv_utils.cpp:290-352) ------------------------------------
EHIP_API int ehip_ref_conv_f32_range(const ehip_conv_desc_t *desc, void *output_f32_dev, const void *input_f32_dev,
                                     const void *weights_dev, const void *bias_dev, float *min_out, float *max_out)
{
  if (!desc || !input_f32_dev || !weights_dev || !min_out || !max_out) return fail(EHIP_GENERAL_ERROR, "null argument");
  const ehip_conv_desc_t &d = *desc;
  if (d.with_bias && !bias_dev) return fail(EHIP_GENERAL_ERROR, "null argument");
  if (d.with_ip_sum && !output_f32_dev)
    return fail(EHIP_GENERAL_ERROR, "reference convolution: with_ip_sum needs the output buffer (it holds the sum operand)");
  if (d.n < 1 || d.g < 1 || d.ic < 1 || d.oc < 1 || d.ic % d.g || d.oc % d.g || d.oh < 1 || d.ow < 1 || d.kh < 1 || d.kw < 1)
    return fail(EHIP_GENERAL_ERROR, "reference convolution: bad dims");
  if (d.dilation_h != 1 || d.dilation_w != 1) return fail(EHIP_UNIMPLEMENTED, "reference convolution: dilation");
  const bool in_ok = d.input_fmt == EHIP_NCHW16C || d.input_fmt == EHIP_NHWC;
  const bool out_ok = d.output_fmt == EHIP_NCHW16C || d.output_fmt == EHIP_NHWC;
  const bool w_ok = (d.weights_fmt == EHIP_OIHW16I16O && d.g == 1) || d.weights_fmt == EHIP_GOIHW || d.weights_fmt == EHIP_OIHW;
  if (!in_ok || !out_ok || !w_ok)
    return fail(EHIP_UNIMPLEMENTED, "reference convolution: activations nChw16c or nhwc; weights OIhw16i16o (g = 1), oihw or goihw");
  RefConvArgs a = {};
  a.in = static_cast<const float *>(input_f32_dev);
  a.w = static_cast<const float *>(weights_dev);
  a.bias = static_cast<const float *>(bias_dev);
  a.out = static_cast<float *>(output_f32_dev);
  a.n = d.n; a.g = d.g; a.ic = d.ic; a.oc = d.oc; a.ih = d.ih; a.iw = d.iw; a.oh = d.oh; a.ow = d.ow;
  a.kh = d.kh; a.kw = d.kw; a.pad_t = d.pad_t; a.pad_l = d.pad_l; a.sh = d.stride_h; a.sw = d.stride_w;
  a.in_nhwc = d.input_fmt == EHIP_NHWC;
  a.out_nhwc = d.output_fmt == EHIP_NHWC;
  a.w_goihw = d.weights_fmt != EHIP_OIHW16I16O;
  a.with_relu = d.with_relu; a.with_sum = d.with_ip_sum; a.with_bias = d.with_bias;
  a.ic2 = up(d.ic, 16) / 16;
  a.oc2 = up(d.oc, 16) / 16;
  const long long blocks = (long long)d.n * a.oc2 * (((long long)d.oh * d.ow + 15) / 16);
  if (blocks >= (1ll << 31)) return fail(EHIP_UNIMPLEMENTED, "reference convolution: too many outputs");
  HIP_TRY(hipMalloc(reinterpret_cast<void **>(&a.partials), 2 * (size_t)blocks * sizeof(float)));
  hipError_t e = launch_ref_conv_f32(a, (unsigned)blocks);
  std::vector<float> part(2 * (size_t)blocks);
  if (e == hipSuccess) e = hipMemcpy(part.data(), a.partials, part.size() * sizeof(float), hipMemcpyDeviceToHost);
  (void)hipFree(a.partials);
  HIP_TRY(e);
  float lo = part[0], hi = part[1];
  for (size_t b = 1; b < (size_t)blocks; ++b) {
    lo = std::min(lo, part[2 * b]);
    hi = std::max(hi, part[2 * b + 1]);
  }
  *min_out = lo;
  *max_out = hi;
  return EHIP_OK;
}

EHIP_API int ehip_calibrate_output_quant(const ehip_conv_desc_t *desc, float out_min, float out_max, float sum_absmax,
                                         float representation, float *output_scale, float *output_z, float *sum_scale)
{
  if (!desc || !output_scale || !output_z) return fail(EHIP_GENERAL_ERROR, "null argument");
  if (!(representation > 0.0f)) return fail(EHIP_GENERAL_ERROR, "calibration: representation must be positive");
  const float abs_min = out_min > 0 ? out_min : -out_min;
  const float abs_max = out_max > abs_min ? out_max : abs_min;
  if (desc->with_relu || desc->output_type == EHIP_S8) {
    // ReLU output, or a signed code: symmetric scale, zero point 0 (tests/elt_conv_utils.cpp:313-323)
    *output_scale = abs_max / representation;
    *output_z = 0.0f;
  } else {
    // the full range mapped onto the code range (tests/elt_conv_utils.cpp:324-328; the harness adds its
    // 0.000001 as a double, so the two quotients are formed in double and then narrowed)
    const double diff = (double)(out_max - out_min) + 0.000001;
    *output_scale = (float)(diff / representation);
    *output_z = (float)((double)(-out_min * representation) / diff);
  }
  if (desc->with_ip_sum) {
    if (!sum_scale) return fail(EHIP_GENERAL_ERROR, "null argument");
    // the sum operand's own scale over the output scale (tests/elt_conv_utils.cpp:333-345)
    const float sum_operand_scale = sum_absmax / representation;
    *sum_scale = sum_operand_scale / *output_scale;
  }
  return EHIP_OK;
}
