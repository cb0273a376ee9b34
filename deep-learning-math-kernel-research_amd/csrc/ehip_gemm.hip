// u8 x s8 -> s32 GEMM on gfx950 matrix cores for the 1x1 convolutions (stride 1 and 2) and for
// the 36 independent GEMMs of the Winograd pipeline, with the requantization epilogue fused.
//
// Replaces elx_int8_conv_direct_1x1_t::__execute_a160_s1/_s2 + gemm_a160_s1/_s2
// (src/elx_int8_conv_direct_1x1_xopt.hpp:20-195, src/elx_int8_conv_direct_1x1.cpp:357-480),
// elx_int8_conv_direct_t::gemm_a160 for K=1 (src/elx_int8_conv_direct.cpp:574-718),
// elx_int8_conv_wino_gemm_t::execute (src/elx_int8_conv_wino_gemm.cpp:23-76) and the
// u8s8 micro-kernel with its epilogue (src/kernel/elk_u8s8_gemm.hxx:168-406).
//
// Mapping.  D[oc][pixel] += W[oc][k] * X[k][pixel] with v_mfma_i32_16x16x64_i8:
//   A operand = weights, one lane = 16 consecutive input channels of one output channel,
//   B operand = activations, one lane = the 16 channels of one nChw16c pixel cell (16 bytes that
//               are contiguous in memory, so no layout change is needed on the way in),
//   D         = lane holds 4 consecutive output channels of one pixel, i.e. one dword of u8/s8
//               output or one float4 of f32 output, and a wave stores 16 pixels x 16 channels as
//               one contiguous run of the nChw16c output.
// The MFMA is signed x signed: activations are remapped u8 -> s8 by flipping the top bit when a
// tile is staged into LDS, and the accumulators start at 128 * sum(weights) per output channel,
// which makes the s32 result identical to the unsigned product.
//
// A workgroup (4 waves) owns OC_T output channels x P_T pixels.  The pixel tile is staged through
// LDS (double buffered, KC units of 16 channels per fill) and shared by the waves that own different
// output channels; every wave streams its own weight rows straight from L2 into registers, one
// k-step ahead of the MFMAs that use them.
#include "ehip_internal.hpp"

namespace ehip {

template <int MO, int NP, int WO, int WPX, int KC>
__global__ __launch_bounds__(kBlock) void k_gemm_u8s8(GemmArgs a)
{
  constexpr int OC_T = WO * MO * 16;
  constexpr int P_T = WPX * NP * 16;
  constexpr int ITEMS = KC * P_T;  // 16-byte cells per LDS fill
  constexpr int NI = (ITEMS + kBlock - 1) / kBlock;
  constexpr int KS = KC / 4;       // MFMA k-steps per fill
  static_assert(WO * WPX == 4, "four waves per workgroup");
  static_assert(KC % 4 == 0, "a k-step is four units");

  __shared__ uint4 lds[2][ITEMS];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int l16 = lane & 15;
  const int lg = lane >> 4;
  const int b = blockIdx.z;
  const int pix0 = blockIdx.x * P_T;
  const int ocw0 = blockIdx.y * OC_T + (wave % WO) * MO * 16;
  const int pw0 = (wave / WO) * NP * 16;
  const int oc_real = a.oc2 * 16;

  // ---- staging plan: which pixel/unit cells this thread copies ---------------------------
  const uint8_t *inb = a.in + (long long)b * a.in_batch_stride;
  long long poff[NI];
  int ucell[NI];
#pragma unroll
  for (int j = 0; j < NI; ++j) {
    const int id = tid + j * kBlock;
    const int p = id % P_T;
    ucell[j] = id / P_T;
    int gp = pix0 + p;
    gp = gp < a.p_total ? gp : a.p_total - 1;
    const int n = gp / a.ohw;
    const int r = gp - n * a.ohw;
    const int oh = r / a.ow;
    const int ow = r - oh * a.ow;
    poff[j] = ((long long)n * a.ic2 * a.ihw + (long long)(oh * a.stride_h) * a.iw + ow * a.stride_w) * 16;
  }
  const long long unit_stride = (long long)a.ihw * 16;
  uint4 stage[NI];
  auto load_stage = [&](int chunk) {
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      if (NI * kBlock == ITEMS || tid + j * kBlock < ITEMS) {
        int u = chunk * KC + ucell[j];
        u = u < a.ic2 ? u : a.ic2 - 1;  // padded units multiply zero weights: any valid cell will do
        stage[j] = *reinterpret_cast<const uint4 *>(inb + poff[j] + (long long)u * unit_stride);
      }
    }
  };
  auto store_stage = [&](int buf) {
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      if (NI * kBlock == ITEMS || tid + j * kBlock < ITEMS) {
        uint4 v = stage[j];
        v.x ^= 0x80808080u; v.y ^= 0x80808080u; v.z ^= 0x80808080u; v.w ^= 0x80808080u;
        lds[buf][tid + j * kBlock] = v;
      }
    }
  };

  // ---- accumulators start at the u8->s8 compensation -------------------------------------
  v4i acc[MO][NP];
#pragma unroll
  for (int mo = 0; mo < MO; ++mo) {
    const v4i c = *reinterpret_cast<const v4i *>(a.ep.comp + (long long)b * a.ocpp + ocw0 + mo * 16 + 4 * lg);
#pragma unroll
    for (int np = 0; np < NP; ++np) acc[mo][np] = c;
  }

  // ---- weights: each wave streams its own rows ---------------------------------------------
  const int8_t *wb = a.w + (long long)b * a.units_pad * a.ocpp * 16 + ((long long)lg * a.ocpp + ocw0 + l16) * 16;
  const long long w_kstep = (long long)4 * a.ocpp * 16;
  auto load_a = [&](v4i (&dst)[MO], int kstep) {
#pragma unroll
    for (int mo = 0; mo < MO; ++mo)
      dst[mo] = *reinterpret_cast<const v4i *>(wb + (long long)kstep * w_kstep + mo * 256);
  };

  const int nchunks = a.units_pad / KC;
  const int nksteps = nchunks * KS;
  v4i a_cur[MO], a_nxt[MO];
  load_stage(0);
  load_a(a_cur, 0);
  int buf = 0;
  for (int c = 0; c < nchunks; ++c) {
    store_stage(buf);
    __syncthreads();
    if (c + 1 < nchunks) load_stage(c + 1);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int kstep = c * KS + ks;
      if (kstep + 1 < nksteps) load_a(a_nxt, kstep + 1);
      const v4i *bl = reinterpret_cast<const v4i *>(&lds[buf][(ks * 4 + lg) * P_T + pw0 + l16]);
#pragma unroll
      for (int np = 0; np < NP; ++np) {
        const v4i bq = bl[np * 16];
#pragma unroll
        for (int mo = 0; mo < MO; ++mo)
          acc[mo][np] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a_cur[mo], bq, acc[mo][np], 0, 0, 0);
      }
#pragma unroll
      for (int mo = 0; mo < MO; ++mo) a_cur[mo] = a_nxt[mo];
    }
    buf ^= 1;
  }

  // ---- epilogue ------------------------------------------------------------------------------
  const float *scale = a.ep.scale + (long long)b * a.ocpp;
  const float *shift = a.ep.shift + (long long)b * a.ocpp;
#pragma unroll
  for (int np = 0; np < NP; ++np) {
    const int gp = pix0 + pw0 + np * 16 + l16;
    if (gp >= a.p_total) continue;
    const int n = gp / a.ohw;
    const int r = gp - n * a.ohw;
#pragma unroll
    for (int mo = 0; mo < MO; ++mo) {
      const int oc = ocw0 + mo * 16 + 4 * lg;
      if (oc >= oc_real) continue;
      const size_t elem = (size_t)b * a.out_batch_stride +
          (((size_t)n * a.oc2 + (oc >> 4)) * a.ohw + r) * 16 + (oc & 15);
      store_quad(a.ep, scale, shift, acc[mo][np], oc, a.out, elem);
    }
  }
}

namespace {
struct Variant {
  const char *name;
  int oc_t, p_t, kc;
  void (*kernel)(GemmArgs);
};
#define V(MO, NP, WO, WPX, KC)                                                                   \
  { "k_gemm_u8s8<" #MO "," #NP "," #WO "," #WPX "," #KC ">", WO * MO * 16, WPX * NP * 16, KC,     \
    k_gemm_u8s8<MO, NP, WO, WPX, KC> }
const Variant kVariants[] = {
    V(4, 4, 4, 1, 8),  // 0: 256 oc x  64 px
    V(2, 4, 4, 1, 8),  // 1: 128 oc x  64 px
    V(4, 2, 4, 1, 8),  // 2: 256 oc x  32 px
    V(2, 2, 4, 1, 4),  // 3: 128 oc x  32 px
    V(4, 1, 4, 1, 4),  // 4: 256 oc x  16 px
    V(4, 4, 2, 2, 8),  // 5: 128 oc x 128 px
    V(2, 4, 2, 2, 8),  // 6:  64 oc x 128 px
    V(1, 4, 4, 1, 4),  // 7:  64 oc x  64 px
};
#undef V
constexpr int kNumVariants = sizeof(kVariants) / sizeof(kVariants[0]);
}  // namespace

const char *gemm_variant_name(int v) { return kVariants[v].name; }
int gemm_variant_chunk(int v) { return kVariants[v].kc; }

// Largest tile that still gives every CU at least two workgroups; ties go to the tile that
// re-reads the pixel tile least (all output channels in one workgroup).
int gemm_pick_variant(int p_total, int oc2, int ic2, int nbatch)
{
  const char *env = getenv("EHIP_GEMM_VARIANT");
  if (env && env[0]) {
    int v = atoi(env);
    if (v >= 0 && v < kNumVariants) return v;
  }
  const int oc = oc2 * 16;
  int best = -1;
  double best_score = -1;
  for (int v = 0; v < kNumVariants; ++v) {
    const Variant &k = kVariants[v];
    if (k.kc > up(ic2, 4) && k.kc > 4) continue;
    const long long wgs = (long long)((p_total + k.p_t - 1) / k.p_t) * ((oc + k.oc_t - 1) / k.oc_t) * nbatch;
    const double util = (double)oc / (double)(((oc + k.oc_t - 1) / k.oc_t) * k.oc_t);
    const double fill = wgs >= 512 ? 1.0 : (double)wgs / 512.0;
    const double tile = (double)k.oc_t * k.p_t / (256.0 * 128.0);
    const double score = util * fill * (0.5 + tile);
    if (score > best_score) { best_score = score; best = v; }
  }
  return best;
}

hipError_t launch_gemm(const GemmArgs &a, int nbatch, int variant, hipStream_t s)
{
  const Variant &k = kVariants[variant];
  dim3 grid((a.p_total + k.p_t - 1) / k.p_t, (a.oc2 * 16 + k.oc_t - 1) / k.oc_t, nbatch);
  hipLaunchKernelGGL(k.kernel, grid, dim3(kBlock), 0, s, a);
  return hipGetLastError();
}

}  // namespace ehip
