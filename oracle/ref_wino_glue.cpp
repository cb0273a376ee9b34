// TEST INFRASTRUCTURE ONLY -- never linked into, imported by, or called from the product path.
//
// Thin C-ABI driver around two translation units of the reference that compile on their own with
// g++ (headers only, no generated tables), linked from where they lie under /root/reference by
// oracle/Makefile (target `ref`):
//   src/elx_conv_wino_trans_input.cpp    elx_conv_wino_trans_input_t<uint8_t, float|uint8_t, ISA_AVX512, A, 3, 16>
//                                        (tile gather, border tiles, the quantization a * mrepS + mz -> epu32 -> u8)
//                                        and <float, float, ...> (the fp32 transformed input the harness calibrates on)
//   src/elx_conv_wino_trans_weights.cpp  elx_conv_wino_trans_weights_t<int8_t, float, ISA_AVX512, A, 3, 16>
//                                        (U = G g Gt, per-(position, oc) abs-max quantization, scale / shift)
// They pin the Winograd quantization glue of the oracle (orc_wino_trans_input, orc_wino_prepare,
// orc_wino_tinput_range) by the reference's compiled code: which multiply-adds g++ -O2 fuses is decided by
// the compiler, not by this file.  Nothing of the reference is copied; this file only fills elx_param_t
// (the fields those classes read) and re-indexes results into the oracle's plain layouts.
#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "euler.hpp"
#include "el_def.hpp"
#include "elx_conv.hpp"
#include "elx_conv_wino_trans_input.hpp"
#include "elx_conv_wino_trans_weights.hpp"

using namespace euler;

namespace {

constexpr int V = 16;

template <typename T>
T *aligned(size_t count)
{
  void *p = nullptr;
  if (posix_memalign(&p, 64, (count * sizeof(T) + 63) / 64 * 64 + 64) != 0) return nullptr;
  memset(p, 0, (count * sizeof(T) + 63) / 64 * 64 + 64);
  return static_cast<T *>(p);
}

// the fields the two classes and their tile kernels read (src/elx_conv.cpp:15-130 derives them from
// eld_conv_t; the Winograd executor adds ht/wt/nt/t/T/t2/Tr, src/elx_int8_conv_wino.cpp:24-54)
void fill(elx_param_t &ep, int A, int n, int ic, int oc, int ih, int iw, int oh, int ow, int pad_t, int pad_l, int T)
{
  const int M = A - 2;
  ep.g = 1; ep.n = n; ep.ic = ic; ep.oc = oc; ep.ih = ih; ep.iw = iw; ep.oh = oh; ep.ow = ow;
  ep.kh = ep.kw = 3;
  ep.tp = pad_t; ep.lp = pad_l; ep.bp = oh + 2 - ih - pad_t; ep.rp = ow + 2 - iw - pad_l;
  ep.hs = ep.ws = ep.hd = ep.wd = 1;
  ep.V1 = 4; ep.Vx = 4;
  ep.G = 1; ep.IC = (ic + V - 1) / V * V; ep.OC = (oc + V - 1) / V * V;
  ep.G2 = ep.G3 = 1;
  ep.I2 = ep.IC / V; ep.I3 = 1; ep.I4 = 1;
  ep.O = 1; ep.O1 = 1; ep.O2 = 1; ep.O3 = ep.OC / V; ep.O4 = 1;
  ep.Ir = ic % V ? ic % V : V;
  ep.Or = oc % V ? oc % V : V;
  ep.ic234 = ep.IC / V; ep.oc234 = ep.OC / V;   // aliases ic2 / oc2
  ep.ht = (oh + M - 1) / M; ep.wt = (ow + M - 1) / M;
  ep.nt = ep.ht * ep.wt; ep.t = ep.nt * n;
  ep.T = T;
  ep.t2 = (ep.t + T - 1) / T;
  ep.Tr = ep.t % T ? ep.t % T : T;
  ep.input_fmt = nChw16c; ep.weights_fmt = OIhw16i16o; ep.output_fmt = nChw16c;
  ep.streaming_input = ep.streaming_output = 0;
  ep.input_as_blocked = ep.weights_as_blocked = ep.output_as_blocked = false;
  ep.nthreads = 1;
  ep.execution_mode = 0xa161;
  ep.sampling_kind = CALIBRATED;
}

// src/elx_int8_conv_wino.cpp:259-278 (prepare_quant_calibration): reciprocals and ceil of the zero points
void calibrate(elx_param_t &ep, float in_S, float in_z, float tin_S, float tin_z)
{
  ep.input_quant_S = in_S;
  ep.input_quant_z = in_z;
  ep.tinput_quant_S = tin_S;
  ep.tinput_quant_z = tin_z;
  ep.input_quant_repS = 1 / ep.input_quant_S;
  ep.input_quant_z = (float)std::ceil(ep.input_quant_z);
  ep.tinput_quant_repS = 1 / ep.tinput_quant_S;
  ep.tinput_quant_z = (float)std::ceil(ep.tinput_quant_z);
}

template <typename InputType, int A>
int trans_input_u8(elx_param_t &ep, const void *input, uint8_t *tinput_plain)
{
  elx_conv_wino_trans_input_t<uint8_t, InputType, ISA_AVX512, A, 3, V> ti;
  ti.setup(&ep);
  const size_t in_count = (size_t)ep.n * ep.I2 * ep.ih * ep.iw * V;
  InputType *in = aligned<InputType>(in_count);
  uint8_t *blk = aligned<uint8_t>((size_t)A * A * ep.I2 * ep.T * V);
  if (!in || !blk) return 2;
  memcpy(in, input, in_count * sizeof(InputType));
  // the per-t2 form that the fused schedule (a161) calls: one block of Tz tiles, laid out
  // [A][A][I3][I2][Tz][V] (src/elx_conv_wino_trans_input.cpp:599-654)
  for (int t2 = 0; t2 < ep.t2; ++t2) {
    const int Tz = t2 == ep.t2 - 1 ? ep.Tr : ep.T;
    ti.execute(nullptr, blk, nullptr, in, t2, Tz);
    for (int pos = 0; pos < A * A; ++pos)
      for (int c2 = 0; c2 < ep.I2; ++c2)
        memcpy(tinput_plain + (((size_t)pos * ep.I2 + c2) * ep.t + (size_t)t2 * ep.T) * V,
               blk + ((size_t)pos * ep.I2 + c2) * Tz * V, (size_t)Tz * V);
  }
  free(in);
  free(blk);
  return 0;
}

template <int A>
int trans_input_f32(elx_param_t &ep, const float *input, float *tinput_plain)
{
  elx_conv_wino_trans_input_t<float, float, ISA_AVX512, A, 3, V> ti;
  ti.setup(&ep);
  const size_t in_count = (size_t)ep.n * ep.I2 * ep.ih * ep.iw * V;
  float *in = aligned<float>(in_count);
  float *blk = aligned<float>((size_t)A * A * ep.I2 * ep.T * V);
  if (!in || !blk) return 2;
  memcpy(in, input, in_count * sizeof(float));
  // per-t2 form, [A][A][I3][I2][Tz][V] (src/elx_conv_wino_trans_input.cpp:27-59,337-359)
  for (int t2 = 0; t2 < ep.t2; ++t2) {
    const int Tz = t2 == ep.t2 - 1 ? ep.Tr : ep.T;
    ti.execute(blk, in, Tz, t2, 0);
    for (int pos = 0; pos < A * A; ++pos)
      for (int c2 = 0; c2 < ep.I2; ++c2)
        memcpy(tinput_plain + (((size_t)pos * ep.I2 + c2) * ep.t + (size_t)t2 * ep.T) * V,
               blk + ((size_t)pos * ep.I2 + c2) * Tz * V, (size_t)Tz * V * sizeof(float));
  }
  free(in);
  free(blk);
  return 0;
}

template <int A>
int trans_weights_s8(elx_param_t &ep, const float *w_blocked, int8_t *twq, float *tscale, float *tshift)
{
  elx_conv_wino_trans_weights_t<int8_t, float, ISA_AVX512, A, 3, V> tw;
  tw.setup(&ep);
  const int oc2 = ep.O3, ic2 = ep.I2, ocp = oc2 * V, icp = ic2 * V;
  const size_t wn = (size_t)oc2 * ic2 * 9 * V * V;
  float *w = aligned<float>(wn);
  float *tf = aligned<float>((size_t)oc2 * A * A * ic2 * V * V);
  int8_t *ts8 = aligned<int8_t>((size_t)oc2 * A * A * ic2 * V * V);
  float *sc = aligned<float>((size_t)oc2 * A * A * V);
  float *sh = aligned<float>((size_t)oc2 * A * A * V);
  if (!w || !tf || !ts8 || !sc || !sh) return 2;
  memcpy(w, w_blocked, wn * sizeof(float));
  tw.execute(sc, sh, ts8, tf, w, ep.O4);
  // s8: [O4][I4][O3][I3][A][A][O1][I2][V1][O][V oc][Vx]; scale / shift: [O4][I4][O3][A][A][O1][O][V]
  // (src/elx_conv_wino_trans_weights.cpp:437-535) -> [A*A][OCp][ICp], [A*A][OCp]
  for (int o2 = 0; o2 < oc2; ++o2)
    for (int pos = 0; pos < A * A; ++pos) {
      for (int ov = 0; ov < V; ++ov) {
        tscale[(size_t)pos * ocp + o2 * V + ov] = sc[((size_t)o2 * A * A + pos) * V + ov];
        tshift[(size_t)pos * ocp + o2 * V + ov] = sh[((size_t)o2 * A * A + pos) * V + ov];
      }
      for (int i2 = 0; i2 < ic2; ++i2)
        for (int v1 = 0; v1 < 4; ++v1)
          for (int ov = 0; ov < V; ++ov)
            for (int vx = 0; vx < 4; ++vx)
              twq[((size_t)pos * ocp + o2 * V + ov) * icp + i2 * V + v1 * 4 + vx] =
                  ts8[(((((size_t)o2 * A * A + pos) * ic2 + i2) * 4 + v1) * V + ov) * 4 + vx];
    }
  free(w); free(tf); free(ts8); free(sc); free(sh);
  return 0;
}

}  // namespace

extern "C" {

// u8 transformed input [A*A][ICp/16][t][16] of an nChw16c input (f32, or u8 codes with in_u8 != 0), tiles in
// blocks of T (the last block ragged).  tin_S / tin_z are wino_tinput_quant as the user sets it.
int ref_wino_glue_trans_input(int A, int in_u8, int n, int ic, int ih, int iw, int oh, int ow, int pad_t, int pad_l,
    int T, float in_S, float tin_S, float tin_z, const void *input, uint8_t *tinput)
{
  elx_param_t ep;
  fill(ep, A, n, ic, 16, ih, iw, oh, ow, pad_t, pad_l, T);
  calibrate(ep, in_S, 0.0f, tin_S, tin_z);
#define GLUE_TI(AA)                                                                                  \
  case AA:                                                                                           \
    return in_u8 ? trans_input_u8<uint8_t, AA>(ep, input, tinput) : trans_input_u8<float, AA>(ep, input, tinput)
  switch (A) {
    GLUE_TI(4);
    GLUE_TI(5);
    GLUE_TI(6);
  }
#undef GLUE_TI
  return 1;
}

// fp32 transformed input [A*A][ICp/16][t][16] (what the harness takes min / max of,
// tests/elt_conv_utils.cpp:222-262)
int ref_wino_glue_trans_input_f32(int A, int n, int ic, int ih, int iw, int oh, int ow, int pad_t, int pad_l, int T,
    const float *input, float *tinput)
{
  elx_param_t ep;
  fill(ep, A, n, ic, 16, ih, iw, oh, ow, pad_t, pad_l, T);
  calibrate(ep, 1.0f, 0.0f, 1.0f, 0.0f);
  switch (A) {
  case 4: return trans_input_f32<4>(ep, input, tinput);
  case 5: return trans_input_f32<5>(ep, input, tinput);
  case 6: return trans_input_f32<6>(ep, input, tinput);
  }
  return 1;
}

// s8 transformed weights [A*A][OCp][ICp], scale / shift [A*A][OCp] from OIhw16i16o f32 weights
int ref_wino_glue_trans_weights(int A, int ic, int oc, float tin_S, float tin_z, const float *w_blocked, int8_t *twq,
    float *tscale, float *tshift)
{
  elx_param_t ep;
  fill(ep, A, 1, ic, oc, 8, 8, 8, 8, 1, 1, 1);
  calibrate(ep, 1.0f, 0.0f, tin_S, tin_z);
  switch (A) {
  case 4: return trans_weights_s8<4>(ep, w_blocked, twq, tscale, tshift);
  case 5: return trans_weights_s8<5>(ep, w_blocked, twq, tscale, tshift);
  case 6: return trans_weights_s8<6>(ep, w_blocked, twq, tscale, tshift);
  }
  return 1;
}

}  // extern "C"
