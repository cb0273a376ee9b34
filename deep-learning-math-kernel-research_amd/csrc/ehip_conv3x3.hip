// Direct 3x3 stride-1 u8 x s8 -> s32 convolution on gfx950 matrix cores as an implicit GEMM
// (K = 9 taps x IC), requantization epilogue fused.
//
// Replaces elx_int8_conv_direct_t::__execute_c160 + conv_c160
// (src/elx_int8_conv_direct_xopt.hpp:20-110, src/elx_int8_conv_direct.cpp:502-571) and the 3x3
// micro-kernel with its epilogue (src/kernel/elk_u8s8_conv.hxx:190-252,679-901).
//
// A workgroup owns P_T consecutive output pixels (row-major inside one image) x OC_T output
// channels.  The input rows those pixels touch, plus the one-pixel frame, are staged into LDS as
// [unit][row][col][16 bytes]; all nine taps read the same staged tile at shifted positions, so
// each input byte is fetched from memory once per workgroup.  Frame cells outside the image
// hold the u8 value 0: after the u8 -> s8 remap (top bit flipped) a zero activation is -128,
// whose product with a weight is cancelled exactly by the 128 * sum(weights) the accumulators
// start from, so skipped border taps of the reference and zero taps here give the same s32.
// Operand roles, lane layout and epilogue are those of the 1x1 kernel (ehip_gemm.hip); the four
// waves of a workgroup split the output channels and share the staged pixels.
#include "ehip_internal.hpp"

// Development aid (compile with -DEHIP_TRACE): lane 0 of every wave records the shader clock at
// phase boundaries into Conv3x3Args::trace.
#ifdef EHIP_TRACE
#define TRACE_POINT(i)                                                                             \
  do {                                                                                             \
    if (a.trace && lane == 0) a.trace[((size_t)(blockIdx.z * gridDim.x + blockIdx.x) * 4 + wave) * 16 + (i)] = clock64(); \
  } while (0)
#else
#define TRACE_POINT(i) do { } while (0)
#endif

namespace ehip {

// Every global load of the main loop is unconditional (addresses are clamped, unwanted values
// are replaced afterwards): with no branch between a load and its use the compiler can count
// outstanding loads exactly, so waiting for one operand does not drain the prefetches behind it.
template <int MO, int NP, int NS>
__global__ __launch_bounds__(kBlock) void k_conv3x3_u8s8(Conv3x3Args a)
{
  constexpr int OC_T = 4 * MO * 16;
  constexpr int P_T = NP * 16;
  constexpr int SLOTS = NS * kBlock;         // 16-byte cells per LDS buffer (>= cells of one fill)
  extern __shared__ uint4 lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int l16 = lane & 15;
  const int lg = lane >> 4;
  const int n = blockIdx.z;
  const int ohw = a.oh * a.ow;
  const int p0 = blockIdx.x * P_T;
  const int r0 = p0 / a.ow;                  // first output row of the tile
  const int ocw0 = blockIdx.y * OC_T + wave * MO * 16;
  const int oc_real = a.oc2 * 16;
  const int WP2 = a.ow + 2;
  const int cells_per_unit = a.halo_rows * WP2;
  const int items = 4 * cells_per_unit;      // one fill = 4 units = one k-step per tap
  const long long plane = (long long)a.ih * a.iw * 16;
  const uint8_t *inb = a.in + (long long)n * a.ic2 * plane;
  TRACE_POINT(0);

  // ---- staging plan (the same cells for every fill) -------------------------------------------
  int goff[NS];      // byte offset of the cell inside a unit's plane (clamped into the image)
  int gunit[NS];
  bool gin[NS];      // false: frame cell, staged as the u8 value 0
#pragma unroll
  for (int j = 0; j < NS; ++j) {
    int id = tid + j * kBlock;
    id = id < items ? id : items - 1;        // surplus slots re-stage the last cell into spare LDS
    const int u = id / cells_per_unit;
    const int rem = id - u * cells_per_unit;
    const int hr = rem / WP2;
    const int hc = rem - hr * WP2;
    const int ih = r0 - a.pad_t + hr;
    const int iw = hc - a.pad_l;
    gunit[j] = u;
    gin[j] = ih >= 0 && ih < a.ih && iw >= 0 && iw < a.iw;
    const int ihc = ih < 0 ? 0 : (ih >= a.ih ? a.ih - 1 : ih);
    const int iwc = iw < 0 ? 0 : (iw >= a.iw ? a.iw - 1 : iw);
    goff[j] = (ihc * a.iw + iwc) * 16;
  }
  uint4 stage[NS];
  auto load_stage = [&](int chunk) {
#pragma unroll
    for (int j = 0; j < NS; ++j) {
      int u = chunk * 4 + gunit[j];
      u = u < a.ic2 ? u : a.ic2 - 1;         // padded units multiply zero weights
      stage[j] = *reinterpret_cast<const uint4 *>(inb + (long long)u * plane + goff[j]);
    }
  };
  auto store_stage = [&](int buf) {
#pragma unroll
    for (int j = 0; j < NS; ++j) {
      uint4 v = stage[j];
      v.x = gin[j] ? v.x ^ 0x80808080u : 0x80808080u;
      v.y = gin[j] ? v.y ^ 0x80808080u : 0x80808080u;
      v.z = gin[j] ? v.z ^ 0x80808080u : 0x80808080u;
      v.w = gin[j] ? v.w ^ 0x80808080u : 0x80808080u;
      lds[buf * SLOTS + tid + j * kBlock] = v;
    }
  };

  // ---- per-lane pixel cells ----------------------------------------------------------------------
  int cellbase[NP];
#pragma unroll
  for (int np = 0; np < NP; ++np) {
    int p = p0 + np * 16 + l16;
    p = p < ohw ? p : ohw - 1;
    const int r = p / a.ow;
    const int c = p - r * a.ow;
    cellbase[np] = (lg * a.halo_rows + (r - r0)) * WP2 + c;
  }

  // per-channel scale/shift of this lane's channels: requested now, needed in the epilogue
  float4 sc[MO], sh[MO];
#pragma unroll
  for (int mo = 0; mo < MO; ++mo) {
    sc[mo] = *reinterpret_cast<const float4 *>(a.ep.scale + ocw0 + mo * 16 + 4 * lg);
    sh[mo] = *reinterpret_cast<const float4 *>(a.ep.shift + ocw0 + mo * 16 + 4 * lg);
  }

  v4i acc[MO][NP];
#pragma unroll
  for (int mo = 0; mo < MO; ++mo) {
    const v4i c = *reinterpret_cast<const v4i *>(a.ep.comp + ocw0 + mo * 16 + 4 * lg);
#pragma unroll
    for (int np = 0; np < NP; ++np) acc[mo][np] = c;
  }

  // weights [9][units_pad][ocpp][16]
  const int8_t *wb = a.w + ((long long)lg * a.ocpp + ocw0 + l16) * 16;
  const long long w_unit = (long long)a.ocpp * 16;
  const int nchunks = a.units_pad / 4;
  auto load_a = [&](v4i (&dst)[MO], int chunk, int tap) {
    chunk = chunk < nchunks ? chunk : nchunks - 1;   // the last fill re-reads its own operands
    const int8_t *p = wb + ((long long)tap * a.units_pad + chunk * 4) * w_unit;
#pragma unroll
    for (int mo = 0; mo < MO; ++mo) dst[mo] = *reinterpret_cast<const v4i *>(p + mo * 256);
  };

  // Software pipeline (one wave per SIMD has nobody else to hide its latencies behind):
  //   - the weight operands of all nine taps of a fill live in registers; each slot is refilled
  //     with the next fill's operand right after its last use, i.e. a whole fill ahead;
  //   - the pixel operands of tap t+1 are read from LDS while the MFMAs of tap t run;
  //   - the next fill's global loads are in flight during the whole fill.
  v4i a_reg[9][MO];
  load_stage(0);
#pragma unroll
  for (int tap = 0; tap < 9; ++tap) load_a(a_reg[tap], 0, tap);
  TRACE_POINT(1);
  int buf = 0;
  for (int c = 0; c < nchunks; ++c) {
    store_stage(buf);
    TRACE_POINT(2 + 3 * (c < 3 ? c : 3));
    __syncthreads();
    TRACE_POINT(3 + 3 * (c < 3 ? c : 3));
    load_stage(c + 1 < nchunks ? c + 1 : c);
    const v4i *tile = reinterpret_cast<const v4i *>(lds + buf * SLOTS);
    v4i bq[2][NP];
#pragma unroll
    for (int np = 0; np < NP; ++np) bq[0][np] = tile[cellbase[np]];
#pragma unroll
    for (int tap = 0; tap < 9; ++tap) {
      if (tap < 8) {
        const int toff = ((tap + 1) / 3) * WP2 + ((tap + 1) % 3);
#ifdef EHIP_TRACE
        if (a.dbg & 1) {
#pragma unroll
          for (int np = 0; np < NP; ++np) bq[(tap + 1) & 1][np] = bq[tap & 1][np];
        } else
#endif
#pragma unroll
        for (int np = 0; np < NP; ++np) bq[(tap + 1) & 1][np] = tile[cellbase[np] + toff];
      }
      // keep the compiler from sinking these reads next to their use: they must be in flight
      // while the MFMAs below run
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int np = 0; np < NP; ++np)
#pragma unroll
        for (int mo = 0; mo < MO; ++mo)
          acc[mo][np] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a_reg[tap][mo], bq[tap & 1][np], acc[mo][np], 0, 0, 0);
#ifdef EHIP_TRACE
      if (!(a.dbg & 2))
#endif
      load_a(a_reg[tap], c + 1, tap);
      __builtin_amdgcn_sched_barrier(0);
    }
    TRACE_POINT(4 + 3 * (c < 3 ? c : 3));
    buf ^= 1;
  }

  size_t pix[NP];
  bool pvalid[NP];
#pragma unroll
  for (int np = 0; np < NP; ++np) {
    const int p = p0 + np * 16 + l16;
    pvalid[np] = p < ohw;
    pix[np] = ((size_t)n * a.oc2 * ohw + (pvalid[np] ? p : 0)) * 16;
  }
  TRACE_POINT(14);
  int oc_of[MO];
#pragma unroll
  for (int mo = 0; mo < MO; ++mo) oc_of[mo] = ocw0 + mo * 16 + 4 * lg;
  epilogue_dispatch<MO, NP>(a.ep, acc, sc, sh, pix, pvalid, oc_of, oc_real, (size_t)ohw * 16, a.out);
  TRACE_POINT(15);
}

namespace {
struct Variant {
  const char *name;
  int oc_t, p_t, ns;
  void (*kernel)(Conv3x3Args);
};
#define V(MO, NP, NS)                                                                              \
  { "k_conv3x3_u8s8<" #MO "," #NP "," #NS ">", 4 * MO * 16, NP * 16, NS, k_conv3x3_u8s8<MO, NP, NS> }
// every (oc tile, pixel tile) comes with a small and a large staging budget NS (cells per thread
// and fill); the launcher takes the first entry of the chosen tile whose budget fits the layer
const Variant kVariants[] = {
    V(2, 7, 3), V(2, 7, 8),  // 0,1: 128 oc x 112 px (4 rows of 28, 2 rows of 56, 8 rows of 14)
    V(2, 8, 4), V(2, 8, 8),  // 2,3: 128 oc x 128 px
    V(2, 4, 3), V(2, 4, 8),  // 4,5: 128 oc x  64 px
    V(1, 7, 3), V(1, 7, 8),  // 6,7:  64 oc x 112 px
    V(1, 4, 3), V(1, 4, 8),  // 8,9:  64 oc x  64 px
    V(4, 4, 3), V(4, 4, 8),  // 10,11: 256 oc x 64 px
};
#undef V
constexpr int kNumVariants = sizeof(kVariants) / sizeof(kVariants[0]);
}  // namespace

const char *conv3x3_variant_name(int v) { return kVariants[v].name; }
int conv3x3_variant_pixels(int v) { return kVariants[v].p_t; }
int conv3x3_variant_slots(int v) { return kVariants[v].ns * kBlock; }
int conv3x3_num_variants() { return kNumVariants; }

int conv3x3_pick_variant(int oh, int ow, int oc2)
{
  const char *env = getenv("EHIP_CONV3X3_VARIANT");
  if (env && env[0]) {
    int v = atoi(env);
    if (v >= 0 && v < kNumVariants) return v;
  }
  const int oc = oc2 * 16, ohw = oh * ow;
  int best = 0;
  double best_score = -1;
  for (int v = 0; v < kNumVariants; v += 2) {
    const Variant &k = kVariants[v];
    const int tiles = (ohw + k.p_t - 1) / k.p_t;
    const double putil = (double)ohw / ((double)tiles * k.p_t);
    const double outil = (double)oc / (double)(((oc + k.oc_t - 1) / k.oc_t) * k.oc_t);
    const double rows = (k.p_t % ow == 0) ? 1.0 : 0.85;  // whole rows stage no superfluous halo
    const double size = 0.5 + (double)k.oc_t * k.p_t / (128.0 * 128.0);
    const double score = putil * outil * rows * size;
    if (score > best_score) { best_score = score; best = v; }
  }
  return best;
}

hipError_t launch_conv3x3(const Conv3x3Args &a, int n, int variant, size_t lds_bytes, hipStream_t s)
{
  const Variant &k = kVariants[variant];
  const int ohw = a.oh * a.ow;
  dim3 grid((ohw + k.p_t - 1) / k.p_t, (a.oc2 * 16 + k.oc_t - 1) / k.oc_t, n);
  if (lds_bytes > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(k.kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
    if (e != hipSuccess) return e;
  }
  hipLaunchKernelGGL(k.kernel, grid, dim3(kBlock), lds_bytes, s, a);
  return hipGetLastError();
}

}  // namespace ehip
