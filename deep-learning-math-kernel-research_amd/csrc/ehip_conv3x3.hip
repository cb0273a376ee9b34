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

namespace ehip {

constexpr int kMaxStage = 8;  // 16-byte cells a thread may stage per LDS fill

template <int MO, int NP>
__global__ __launch_bounds__(kBlock) void k_conv3x3_u8s8(Conv3x3Args a)
{
  constexpr int OC_T = 4 * MO * 16;
  constexpr int P_T = NP * 16;
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

  // ---- staging plan (the same cells for every fill) -------------------------------------------
  int goff[kMaxStage];   // byte offset of the cell inside the chunk's first plane, -1 = frame
  int gunit[kMaxStage];
#pragma unroll
  for (int j = 0; j < kMaxStage; ++j) {
    const int id = tid + j * kBlock;
    goff[j] = -2;  // not mine
    gunit[j] = 0;
    if (id < items) {
      const int u = id / cells_per_unit;
      const int rem = id - u * cells_per_unit;
      const int hr = rem / WP2;
      const int hc = rem - hr * WP2;
      const int ih = r0 - a.pad_t + hr;
      const int iw = hc - a.pad_l;
      gunit[j] = u;
      goff[j] = (ih >= 0 && ih < a.ih && iw >= 0 && iw < a.iw) ? (ih * a.iw + iw) * 16 : -1;
    }
  }
  uint4 stage[kMaxStage];
  auto load_stage = [&](int chunk) {
#pragma unroll
    for (int j = 0; j < kMaxStage; ++j) {
      if (goff[j] >= 0) {
        int u = chunk * 4 + gunit[j];
        u = u < a.ic2 ? u : a.ic2 - 1;  // padded units multiply zero weights
        stage[j] = *reinterpret_cast<const uint4 *>(inb + (long long)u * plane + goff[j]);
      } else {
        stage[j] = make_uint4(0u, 0u, 0u, 0u);
      }
    }
  };
  auto store_stage = [&](int buf) {
#pragma unroll
    for (int j = 0; j < kMaxStage; ++j) {
      if (goff[j] >= -1) {
        uint4 v = stage[j];
        v.x ^= 0x80808080u; v.y ^= 0x80808080u; v.z ^= 0x80808080u; v.w ^= 0x80808080u;
        lds[buf * items + tid + j * kBlock] = v;
      }
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
    const int8_t *p = wb + ((long long)tap * a.units_pad + chunk * 4) * w_unit;
#pragma unroll
    for (int mo = 0; mo < MO; ++mo) dst[mo] = *reinterpret_cast<const v4i *>(p + mo * 256);
  };

  v4i a_cur[MO], a_nxt[MO];
  load_stage(0);
  load_a(a_cur, 0, 0);
  int buf = 0;
  for (int c = 0; c < nchunks; ++c) {
    store_stage(buf);
    __syncthreads();
    if (c + 1 < nchunks) load_stage(c + 1);
    const v4i *tile = reinterpret_cast<const v4i *>(lds + buf * items);
#pragma unroll
    for (int tap = 0; tap < 9; ++tap) {
      if (tap < 8) load_a(a_nxt, c, tap + 1);
      else if (c + 1 < nchunks) load_a(a_nxt, c + 1, 0);
      const int toff = (tap / 3) * WP2 + (tap % 3);
#pragma unroll
      for (int np = 0; np < NP; ++np) {
        const v4i bq = tile[cellbase[np] + toff];
#pragma unroll
        for (int mo = 0; mo < MO; ++mo)
          acc[mo][np] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a_cur[mo], bq, acc[mo][np], 0, 0, 0);
      }
#pragma unroll
      for (int mo = 0; mo < MO; ++mo) a_cur[mo] = a_nxt[mo];
    }
    buf ^= 1;
  }

#pragma unroll
  for (int np = 0; np < NP; ++np) {
    const int p = p0 + np * 16 + l16;
    if (p >= ohw) continue;
#pragma unroll
    for (int mo = 0; mo < MO; ++mo) {
      const int oc = ocw0 + mo * 16 + 4 * lg;
      if (oc >= oc_real) continue;
      const size_t elem = (((size_t)n * a.oc2 + (oc >> 4)) * ohw + p) * 16 + (oc & 15);
      store_quad(a.ep, a.ep.scale, a.ep.shift, acc[mo][np], oc, a.out, elem);
    }
  }
}

namespace {
struct Variant {
  const char *name;
  int oc_t, p_t;
  void (*kernel)(Conv3x3Args);
};
#define V(MO, NP) { "k_conv3x3_u8s8<" #MO "," #NP ">", 4 * MO * 16, NP * 16, k_conv3x3_u8s8<MO, NP> }
const Variant kVariants[] = {
    V(2, 7),  // 0: 128 oc x 112 px (4 rows of 28, 2 rows of 56, 8 rows of 14)
    V(2, 8),  // 1: 128 oc x 128 px
    V(2, 4),  // 2: 128 oc x  64 px
    V(1, 7),  // 3:  64 oc x 112 px
    V(1, 4),  // 4:  64 oc x  64 px
    V(4, 4),  // 5: 256 oc x  64 px
};
#undef V
constexpr int kNumVariants = sizeof(kVariants) / sizeof(kVariants[0]);
}  // namespace

const char *conv3x3_variant_name(int v) { return kVariants[v].name; }
int conv3x3_variant_pixels(int v) { return kVariants[v].p_t; }

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
  for (int v = 0; v < kNumVariants; ++v) {
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
