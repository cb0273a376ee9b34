// 1x1 u8 x s8 -> s32 convolution with MANY input channels on gfx950 matrix cores: the pixel tile is
// resident, the weights stream.
//
// Replaces, for blocked activations, elx_int8_conv_direct_1x1_t::__execute_a160_s1 / _s2 + gemm_a160_s1 / _s2
// (src/elx_int8_conv_direct_1x1_xopt.hpp:20-195, src/elx_int8_conv_direct_1x1.cpp:357-480) and the u8s8 GEMM
// micro-kernel with its epilogue (src/kernel/elk_u8s8_gemm.hxx:168-406).
//
// Why a second 1x1 kernel.  A layer like 1024 -> 256 at 14 x 14 is a short, wide GEMM whose activations
// come from HBM exactly once.  The general kernel (ehip_gemm.hip) walks K in fills of 128 channels with two
// fills in flight: every fill waits a full trip to HBM, eight times in a row.  Here a workgroup asks for
// its WHOLE pixel tile -- P_T pixels x all input channels -- in one go, with loads that write LDS
// directly (global_load_lds_dwordx4: no registers held while they fly, so all of them can be in flight
// at once), pays the trip to HBM once, and then only streams weights, which sit in L2, through a register
// ring straight into the MFMA A operand.  Every wave owns its own TM x 32 output channels (no weight row is
// loaded twice by a workgroup) and all of the tile's TN x 32 pixels.
//
// The u8 -> s8 remap (top bit of every activation byte flipped, 128 * sum(w) added back through the
// accumulators' start value) happens when an operand is read from LDS, since the loads bypass registers.
#include <type_traits>

#include "ehip_internal.hpp"

// Development aid (compile with -DEHIP_TRACE): lane 0 of every wave records the wall clock at phase boundaries.
#ifdef EHIP_TRACE
#define TRACE_POINT(i)                                                                             \
  do {                                                                                             \
    if (a.trace && lane == 0) a.trace[((size_t)blockIdx.x * 4 + wave) * 16 + (i)] = wall_clock64(); \
  } while (0)
#else
#define TRACE_POINT(i) do { } while (0)
#endif

namespace ehip {

// 16 bytes per lane from global memory straight into LDS: lane i's piece lands at lds_dst + 16 i
// (lds_dst is wave-uniform).  The builtin exists in the device pass only.
__device__ __forceinline__ void load_to_lds_16(const void *gsrc, void *lds_dst)
{
#if defined(__HIP_DEVICE_COMPILE__)
  __builtin_amdgcn_global_load_lds(gsrc, (__attribute__((address_space(3))) void *)lds_dst, 16, 0, 0);
#else
  (void)gsrc;
  (void)lds_dst;
#endif
}
__device__ __forceinline__ void wait_all_loads()
{
#if defined(__HIP_DEVICE_COMPILE__)
  __builtin_amdgcn_s_waitcnt(0x0f70);   // vmcnt(0), the other counters untouched
#endif
}

// The same load written as assembly.  The compiler cannot tell which part of LDS an LDS-writing load
// touches, and makes the first LDS read behind such loads wait for ALL of them; this form it does not see as
// a memory instruction at all.  The caller waits for these loads itself (wait_loads_but) and must not rely
// on the compiler's own waits to cover them: those then wait for a few older loads more than they need,
// never for fewer, because the wave's loads complete in issue order.
__device__ __forceinline__ void load_to_lds_16_unseen(const void *gsrc, void *lds_dst)
{
#if defined(__HIP_DEVICE_COMPILE__)
  const unsigned m = __builtin_amdgcn_readfirstlane((unsigned)(size_t)(__attribute__((address_space(3))) void *)lds_dst);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(m), "v"(gsrc) : "memory", "m0");
#else
  (void)gsrc;
  (void)lds_dst;
#endif
}
// vmcnt(n): at most n of the wave's vector-memory loads still in flight.  n is a constant after unrolling.
__device__ __forceinline__ void wait_loads_but(int n)
{
#if defined(__HIP_DEVICE_COMPILE__)
#define EHIP_W(N) case N: __builtin_amdgcn_s_waitcnt(0x0f70 | (N & 15) | ((N >> 4) << 14)); break;
  switch (n) {
    EHIP_W(0) EHIP_W(1) EHIP_W(2) EHIP_W(3) EHIP_W(4) EHIP_W(5) EHIP_W(6) EHIP_W(7) EHIP_W(8) EHIP_W(9) EHIP_W(10)
    EHIP_W(11) EHIP_W(12) EHIP_W(13) EHIP_W(14) EHIP_W(15) EHIP_W(16) EHIP_W(17) EHIP_W(18) EHIP_W(19) EHIP_W(20)
    EHIP_W(21) EHIP_W(22) EHIP_W(23) EHIP_W(24) EHIP_W(25) EHIP_W(26) EHIP_W(27) EHIP_W(28) EHIP_W(29) EHIP_W(30)
    EHIP_W(31) EHIP_W(32)
    default: __builtin_amdgcn_s_waitcnt(0x0f70); break;
  }
#undef EHIP_W
#else
  (void)n;
#endif
}

// NKS > 0: the layer has exactly NKS k-steps (pairs of 16-channel units): the K loop is straight-line code
// and every wait names the load it needs.  NKS == 0: a loop over blocks of eight k-steps.
// NHWC: nhwc input.  A pixel's channel vector is contiguous in memory, so the tile is kept pixel-major in LDS,
// [P_T pixels][units_pad + 1 cells]: the odd row length spreads the 16 pixels a 16-byte operand read serves per
// clock over all banks.  A wave-load still fills 64 consecutive LDS cells; its lane i fetches whatever cell
// 64 j + i of that layout is (the pad cell and padded units repeat a real unit: they multiply zero weights or
// nothing).  The whole tile is waited for before the K loop (no unit order to consume it in).
// What a wave's first instructions need -- the three pointers its first loads go through and the geometry
// their addresses are made of -- is passed as leading scalar arguments, which the dispatcher preloads into scalar
// registers with the wave (the file is compiled with -amdgpu-kernarg-preload-count=16); the rest of the argument
// block is loaded as usual while those loads fly.  geom = stride_h | stride_w << 8 | dense << 16 | oc2 << 20.
#define EHIP_RES_HEAD                                                                                                  \
  const uint8_t *in, const int8_t *w, const int *comp, int nx, int ny, int p_total, int ohw, unsigned ohw_magic, int ihw, \
      int ic2, int units_pad, int ocpp, unsigned geom
template <int TM, int TN, int NKS, bool NHWC = false>
__global__ __launch_bounds__(kBlock, 1) void k_gemm1x1_res(EHIP_RES_HEAD, GemmArgs rest)
{
  GemmArgs a = rest;
  a.in = in; a.w = w; a.ep.comp = comp; a.nx = nx; a.ny = ny; a.p_total = p_total; a.ohw = ohw; a.ohw_magic = ohw_magic;
  a.ihw = ihw; a.ic2 = ic2; a.units_pad = units_pad; a.ocpp = ocpp;
  a.stride_h = (int)(geom & 0xffu); a.stride_w = (int)((geom >> 8) & 0xffu); a.oc2 = (int)(geom >> 20);
  constexpr int OC_T = 4 * TM * 32;
  constexpr int P_T = TN * 32;
  // Weight ring: k-steps requested ahead.  A kernel launch starts with cold L2s, and in a layer of ONE
  // generation of workgroups every workgroup asks for the same weight lines at the same time: each request
  // then takes a trip to the memory-side cache, not to L2, and a ring of eight k-steps is four such trips
  // in a row.  Where the wave's whole weight slice fits in registers (NKS x TM <= 32 operands) it is
  // requested up front, next to the pixel tile: one trip.
  constexpr int R = (NKS > 0 && NKS * TM <= 32) ? NKS : 8;
  extern __shared__ v4i lds[];         // [units][P_T]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31;
  const int lh = lane >> 5;
  // channel blocks of one pixel tile follow each other on ONE XCD (the first pulls the pixels into that
  // XCD's L2, the others find them there); an XCD takes a contiguous eighth of the pixel tiles
  const int xcd = blockIdx.x & 7, seq = blockIdx.x >> 3;
  const int by = seq % a.ny;
  const int bx = xcd * ((a.nx + 7) >> 3) + seq / a.ny;
  if (bx >= a.nx) return;   // whole workgroup
  const int pix0 = bx * P_T;
  const int oc0 = by * OC_T + wave * TM * 32;   // the wave's first channel
  const int oc_real = a.oc2 * 16;
  const int nks = a.units_pad >> 1;
  const bool dense = (geom >> 16) & 1u;   // stride 1 and the output plane is the input plane
  TRACE_POINT(0);

  // ---- the whole pixel tile, all units, straight into LDS -----------------------------------------------
  // A wave-load moves 64 consecutive pixels of one unit (1 KB): lane i's 16 bytes land at the wave-uniform
  // LDS address + 16 i.  Pixel halves of 64 (P_T / 64) x units are dealt to the four waves round-robin.
  constexpr int HALVES = P_T / 64 > 0 ? P_T / 64 : 1;
  constexpr int LPW = P_T >= 64 ? 64 : P_T;   // pixels per wave-load (32-pixel tiles: the upper lanes repeat)
  const int U1 = a.units_pad + 1;   // nhwc: cells per staged pixel
  // byte offset of output pixel gp's first input cell in an nhwc tensor (clamped past the end)
  auto nhwc_pixel = [&](int gp) -> long long {
    gp = gp < a.p_total ? gp : a.p_total - 1;
    const int n = a.ohw == a.p_total ? 0 : fastdiv_any(gp, a.ohw, a.ohw_magic);
    const int r = gp - n * a.ohw;
    long long sp = r;
    if (!dense) {
      const int oh = fastdiv(r, a.ow, a.ow_magic);
      sp = (long long)oh * a.stride_h * a.iw + (long long)(r - oh * a.ow) * a.stride_w;
    }
    return ((long long)n * a.ihw + sp) * a.ic2 * 16;
  };
  auto request_tile_nhwc = [&]() {
    const int cells = P_T * U1;
    for (int c0 = wave * 64; c0 < cells; c0 += 256) {   // wave-uniform
      const int c = c0 + lane;
      int p = fastdiv(c, U1, a.u1_magic);
      int u = c - p * U1;
      p = p < P_T ? p : P_T - 1;            // the last load runs past the tile: into the allocation's slack
      u = u < a.ic2 ? u : a.ic2 - 1;
      load_to_lds_16(a.in + nhwc_pixel(pix0 + p) + u * 16, lds + c0);
    }
  };
  const uint8_t *src[HALVES];
#pragma unroll
  for (int h = 0; h < HALVES; ++h) {
    int gp = pix0 + h * 64 + (lane % LPW);
    gp = gp < a.p_total ? gp : a.p_total - 1;   // pixels behind the end are computed and not stored
    const int n = a.ohw == a.p_total ? 0 : fastdiv_any(gp, a.ohw, a.ohw_magic);
    const int r = gp - n * a.ohw;
    long long sp = r;
    if (!dense) {
      const int oh = fastdiv(r, a.ow, a.ow_magic);
      sp = (long long)oh * a.stride_h * a.iw + (long long)(r - oh * a.ow) * a.stride_w;
    }
    src[h] = a.in + ((long long)n * a.ic2 * a.ihw + sp) * 16;
  }
  const long long unit_stride = (long long)a.ihw * 16;
  auto request_tile = [&]() {   // in unit order: what lands first is what the K loop needs first
    const int items = a.units_pad * HALVES;
    for (int it = wave; it < items; it += 4) {
      const int u = it / HALVES, h = it - u * HALVES;
      const int uc = u < a.ic2 ? u : a.ic2 - 1;   // the padded unit multiplies zero weights: any data will do
#pragma unroll
      for (int hh = 0; hh < HALVES; ++hh)
        if (hh == h)
          load_to_lds_16(src[hh] + (long long)uc * unit_stride, lds + (size_t)u * P_T + h * 64);
    }
  };
  // PIPE (the wave's whole weight slice fits in registers and is requested up front, BEFORE the tile, and
  // nothing else is loaded until the K loop is over): the tile is consumed as it arrives.  Loads complete in
  // issue order, so the weights (from L2) are there first; the K loop then waits for eight units (four
  // k-steps) of the tile at a time -- its own share by count, everybody else's by a barrier -- instead of
  // for all 64 KB before its first MFMA.
  constexpr bool PIPE = !NHWC && NKS > 0 && R == NKS && NKS % 4 == 0;
  constexpr int LPC = 2 * HALVES;            // loads of one wave per chunk: 8 units x HALVES dealt to four waves
  constexpr int TILE_LOADS = NKS * HALVES / 2;   // of one wave, all chunks (PIPE)
  auto request_tile_unseen = [&]() {
#pragma unroll
    for (int j = 0; j < TILE_LOADS; ++j) {
      const int it = wave + 4 * j;
      const int u = it / HALVES, h = it - u * HALVES;
      const int uc = u < a.ic2 ? u : a.ic2 - 1;
      const uint8_t *p = src[0];
#pragma unroll
      for (int hh = 1; hh < HALVES; ++hh) p = hh == h ? src[hh] : p;
      load_to_lds_16_unseen(p + (long long)uc * unit_stride, lds + (size_t)u * P_T + h * 64);
    }
  };
  if (NHWC) request_tile_nhwc();
  else if (!PIPE) request_tile();

  // ---- the accumulators start from the compensation ------------------------------------------------
  const long long cidx = oc0 + 16 * lh;   // the lane's 16 channels of tile 0
  v16i acc[TM][TN];
#pragma unroll
  for (int mt = 0; mt < TM; ++mt) {
    v4i c4[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) c4[q] = *reinterpret_cast<const v4i *>(a.ep.comp + cidx + 32 * mt + 4 * q);
#pragma unroll
    for (int nt = 0; nt < TN; ++nt)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[mt][nt][v] = c4[v >> 2][v & 3];
  }


  TRACE_POINT(1);
  // ---- weights [units_pad][ocpp][16]: lane = packed row l32 of unit 2 ks + lh, tile mt 32 rows on --------
  const int8_t *wb = a.w + ((long long)lh * a.ocpp + oc0 + l32) * 16;
  const long long w_step = (long long)a.ocpp * 32;   // two units
  v4i a_reg[R][TM];
  auto load_a = [&](int slot, int ks) {
    const int8_t *p = wb + (long long)ks * w_step;
#pragma unroll
    for (int mt = 0; mt < TM; ++mt) a_reg[slot][mt] = *reinterpret_cast<const v4i *>(p + mt * 512);
  };
#pragma unroll
  for (int k = 0; k < R; ++k) load_a(k, k < nks ? k : nks - 1);

  // the in-place sum's operand is requested now, with everything else, and used in the epilogue
  uint8_t *cell[TN];
  bool pv[TN];
  v4i old[TM][TN];
  const size_t tile_stride = a.out_nhwc ? (size_t)32 : (size_t)2 * a.ohw * 16;   // to the next 32 channels' cell
#pragma unroll
  for (int nt = 0; nt < TN; ++nt) {
    const int gp = pix0 + nt * 32 + l32;
    pv[nt] = gp < a.p_total;
    const int gpc = pv[nt] ? gp : 0;
    const int n = a.ohw == a.p_total ? 0 : fastdiv_any(gpc, a.ohw, a.ohw_magic);
    const int r = gpc - n * a.ohw;
    cell[nt] = static_cast<uint8_t *>(a.out) +
        (a.out_nhwc ? (size_t)gpc * oc_real + (oc0 + 16 * lh) : (((size_t)n * a.oc2 + (oc0 >> 4) + lh) * a.ohw + r) * 16);
    if (a.lean & 4) {
#pragma unroll
      for (int mt = 0; mt < TM; ++mt) {
        const bool ok = pv[nt] && oc0 + 16 * lh + 32 * mt < oc_real;
        old[mt][nt] = *reinterpret_cast<const v4i *>(ok ? cell[nt] + (size_t)mt * tile_stride : cell[nt]);
      }
    }
  }

  LeanConsts lk[TM];
  OcConsts k0;
  auto load_epilogue_consts = [&]() {
    if (a.lean) {
#pragma unroll
      for (int mt = 0; mt < TM; ++mt) load_lean_consts(lk[mt], a.ep, cidx + 32 * mt);
    } else {
      load_consts(k0, a.ep, cidx);
    }
  };

  auto next_chunk = [&](int c) {   // units 8 c .. 8 c + 7 of the tile are in LDS, everybody's share
    wait_loads_but(TILE_LOADS - (c + 1) * LPC);
    __syncthreads();
  };
  if (PIPE) {
    load_epilogue_consts();   // nothing may be requested behind the tile
    request_tile_unseen();
    TRACE_POINT(2);
    next_chunk(0);
  } else {
    // the tile has landed (every wave waits for its own loads, the barrier for everybody else's)
    wait_all_loads();
    TRACE_POINT(2);
    __syncthreads();
  }
  TRACE_POINT(3);

  // ---- K loop: one memory instruction behind each MFMA ---------------------------------------------------
  v4i bq[2][TN];
  const v4i *tile = NHWC ? lds + l32 * U1 + lh : lds + lh * P_T + l32;
  // (raw bytes: the u8 -> s8 flip of the top bits happens right before the operand's first use.  Next to the
  // read it would make the wave wait for the read it has just issued; as a pass over the whole tile in LDS it
  // was measured to cost more than it saves.  With one wave per SIMD the flip still sits between a read and
  // the MFMA that waits for it -- 51 instead of 34 clocks per MFMA -- which a second workgroup on the CU
  // hides: the 64-pixel tiles, two workgroups per CU, are the fast ones.)
  auto read_b = [&](int par, int ks, int nt) {
    bq[par][nt] = NHWC ? tile[nt * 32 * U1 + 2 * ks] : tile[(size_t)ks * 2 * P_T + nt * 32];
  };
  // k-step ks out of operand buffer par; the operands of k-step ks + 1 are read on the way, the ring slot
  // is refilled with the weights of k-step ks + R behind the last MFMA
  auto kstep = [&](int par, int slot, int ks, bool read_next, bool load_next) {
#pragma unroll
    for (int mt = 0; mt < TM; ++mt)
#pragma unroll
      for (int nt = 0; nt < TN; ++nt) {
        if (mt == 0) bq[par][nt] ^= (int)0x80808080;
        acc[mt][nt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a_reg[slot][mt], bq[par][nt], acc[mt][nt], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        if (mt == 0 && read_next) read_b(par ^ 1, ks + 1, nt);
        if (mt == TM - 1 && nt == TN - 1 && load_next) load_a(slot, ks + R);
        __builtin_amdgcn_sched_barrier(0);
      }
  };
#pragma unroll
  for (int nt = 0; nt < TN; ++nt) read_b(0, 0, nt);
  if (NKS > 0) {
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
      if (!PIPE && ks == (NKS > R ? NKS - R : 0)) load_epilogue_consts();
      if (PIPE && (ks + 1) % 4 == 0 && ks + 1 < NKS) next_chunk((ks + 1) / 4);   // k-step ks reads the operands of ks + 1
      kstep(ks & 1, ks % R, ks, ks + 1 < NKS, ks + R < NKS);
    }
  } else {
    // blocks of R k-steps (nks is a multiple of R or the tail is peeled below)
    int ks0 = 0;
    for (; ks0 + 2 * R <= nks; ks0 += R) {
#pragma unroll
      for (int k = 0; k < R; ++k) kstep(k & 1, k, ks0 + k, true, true);
    }
    load_epilogue_consts();
    // last one or two blocks: requests stop at the end of K
    for (; ks0 < nks; ks0 += R) {
#pragma unroll
      for (int k = 0; k < R; ++k)
        if (ks0 + k < nks) kstep(k & 1, k, ks0 + k, ks0 + k + 1 < nks, ks0 + k + R < nks);
    }
  }

  TRACE_POINT(5);
  // ---- epilogue ---------------------------------------------------------------------------------------
  if (a.lean) {
    lean_store<TM, TN>(a.lean, a.ep, acc, lk, cell, pv, oc0 + 16 * lh, oc_real, tile_stride, old);
    TRACE_POINT(15);
    return;
  }
  size_t pix[TN];
  bool pvalid[TN];
#pragma unroll
  for (int nt = 0; nt < TN; ++nt) {
    const int gp = pix0 + nt * 32 + l32;
    pvalid[nt] = gp < a.p_total;
    const int gpc = pvalid[nt] ? gp : 0;
    const int n = a.ohw == a.p_total ? 0 : fastdiv_any(gpc, a.ohw, a.ohw_magic);
    pix[nt] = ((size_t)n * a.oc2 * a.ohw + (gpc - n * a.ohw)) * 16;
  }
  const size_t pixT[TN][2] = {};
  const bool validT[TN][2] = {};
  epilogue_wave<TM, TN, false, true>(a.ep, acc, k0, cidx, oc0 + 16 * lh, pix, pvalid, oc_real, (size_t)a.ohw * 16, a.out,
                                     nullptr, pixT, validT);
}

namespace {
typedef void (*res_kernel_t)(EHIP_RES_HEAD, GemmArgs);
struct ResVariant {
  const char *name;
  int oc_t, p_t;
  res_kernel_t generic;
  res_kernel_t unrolled[3];   // exactly 8, 16, 32 k-steps
  res_kernel_t generic_nhwc;  // nhwc input (64-pixel tiles only), or null
  res_kernel_t unrolled_nhwc[3];
};
hipError_t res_enqueue(const LaunchPlan<GemmArgs> &plan, hipStream_t s)
{
  const GemmArgs &a = plan.args;
  const bool dense = a.stride_h == 1 && a.stride_w == 1 && a.iw == a.ow;
  const unsigned geom = (unsigned)a.stride_h | (unsigned)a.stride_w << 8 | (dense ? 1u << 16 : 0u) | (unsigned)a.oc2 << 20;
  hipLaunchKernelGGL(reinterpret_cast<res_kernel_t>(plan.kernel), plan.grid, plan.block, plan.lds, s, a.in, a.w, a.ep.comp,
                     a.nx, a.ny, a.p_total, a.ohw, a.ohw_magic, a.ihw, a.ic2, a.units_pad, a.ocpp, geom, a);
  return hipGetLastError();
}
#define RV(TM, TN)                                                                                           \
  { "k_gemm1x1_res<" #TM "," #TN ">", 4 * TM * 32, TN * 32, k_gemm1x1_res<TM, TN, 0>,                        \
    {k_gemm1x1_res<TM, TN, 8>, k_gemm1x1_res<TM, TN, 16>, k_gemm1x1_res<TM, TN, 32>}, nullptr, {nullptr, nullptr, nullptr} }
#define RVN(TM, TN)                                                                                          \
  { "k_gemm1x1_res<" #TM "," #TN ">", 4 * TM * 32, TN * 32, k_gemm1x1_res<TM, TN, 0>,                        \
    {k_gemm1x1_res<TM, TN, 8>, k_gemm1x1_res<TM, TN, 16>, k_gemm1x1_res<TM, TN, 32>}, k_gemm1x1_res<TM, TN, 0, true>, \
    {k_gemm1x1_res<TM, TN, 8, true>, k_gemm1x1_res<TM, TN, 16, true>, k_gemm1x1_res<TM, TN, 32, true>} }
const ResVariant kRes[] = {
    RV(1, 4),    // 0: 128 oc x 128 px
    RVN(1, 2),   // 1: 128 oc x  64 px
    RV(2, 4),    // 2: 256 oc x 128 px
    RVN(2, 2),   // 3: 256 oc x  64 px
};
#undef RV
#undef RVN
constexpr int kNumRes = sizeof(kRes) / sizeof(kRes[0]);
constexpr size_t kResLds = 160 * 1024;

}  // namespace

namespace {
// LDS of a workgroup: [units][P_T] cells, or (nhwc input) [P_T][units + 1] rounded up to whole wave-loads
size_t res_lds_bytes(const GemmArgs &a, int p_t)
{
  return a.in_nhwc ? (size_t)up((a.units_pad + 1) * p_t, 64) * 16 : (size_t)a.units_pad * p_t * 16;
}
}  // namespace

// -1: the layer is not one for this kernel
int gemm1x1_res_pick(const GemmArgs &a, int nbatch)
{
  const char *env = getenv("EHIP_GEMM1X1_RES");
  if (env && env[0] == '0') return -1;
  if (nbatch != 1 || a.kh * a.kw > 1 || a.ep.shift_tab) return -1;
  if (a.stride_h > 255 || a.stride_w > 255 || a.oc2 >= 4096) return -1;   // what the kernel's packed leading argument holds
  // nhwc output: through the lean epilogue only (a lane's 16 bytes are contiguous there as well; the general
  // epilogue of this kernel addresses blocked cells)
  if (a.out_nhwc && !lean_mode(a.ep, false)) return -1;
  if (a.ic2 <= 8 || (a.units_pad & 1)) return -1;   // few channels: the weights-in-registers kernel
  if (env && env[0] >= '1' && env[0] <= '4') {
    const int v = env[0] - '1';
    if (a.in_nhwc && !kRes[v].generic_nhwc) return -1;
    return res_lds_bytes(a, kRes[v].p_t) <= kResLds ? v : -1;
  }
  const int oc = a.oc2 * 16;
  int best = -1;
  double best_score = 0;
  for (int v = 0; v < kNumRes; ++v) {
    const ResVariant &k = kRes[v];
    if (res_lds_bytes(a, k.p_t) > kResLds || (a.in_nhwc && !k.generic_nhwc)) continue;
    const int gx = (a.p_total + k.p_t - 1) / k.p_t, gy = (oc + k.oc_t - 1) / k.oc_t;
    const long long wgs = (long long)gx * gy;
    const int per_cu = (int)(kResLds / res_lds_bytes(a, k.p_t));   // resident workgroups
    const long long slots = 256ll * (per_cu > 2 ? 2 : per_cu);
    const long long rounds = (wgs + slots - 1) / slots;
    const double util = ((double)oc / ((double)gy * k.oc_t)) * ((double)a.p_total / ((double)gx * k.p_t));
    const double fill = (double)wgs / (double)(rounds * slots);
    // Measured (1024 -> 256 at 14 x 14 and 512 -> 1024 stride 2, N = 64): the 128 x 64 tile, two workgroups
    // per CU that hide each other's load, flip and epilogue phases, 8.6 / 17.5 us; 128 x 128 10.8 / 19.4 us;
    // the 256-channel tiles (a wave owns 64 channels, twice the registers) 9.0-14.4 / 22.5-25.9 us.
    static const double pref[] = {0.95, 1.10, 0.70, 0.85};
    double score = util * (0.5 + 0.5 * fill) * pref[v] * (per_cu >= 2 ? 1.0 : 0.9);
    // 1024 input channels, whole 256-channel tiles, enough of them for three quarters of the CUs: the
    // 256 x 64 tile pulls every pixel tile through L2 half as often (1024 -> 256 at 14 x 14, N = 64: 8.1 against
    // 9.0 us, 1024 -> 512: 12.2 against 15.4 us); with 512 channels its weights-in-registers form needs too
    // many registers and loses (512 -> 1024 stride 2: 23.9 against 15.2 us)
    if (v == 3 && a.units_pad == 64 && oc % 256 == 0 && wgs >= 192) score = 2.0;
    // up to 512 input channels and about one and a half workgroups of the 128 x 128 tile per CU (where the 128 x 64
    // tile needs twice as many): measured at N = 64 with 392-400 of them, 512 -> 128 at 28 x 28 7.9 against 9.1 us,
    // 512 -> 512 at 14 x 14 7.5 against 8.4 us, 256 -> 512 at 14 x 14 6.1 against 6.7 us, 512 -> 2048 at 7 x 7 9.3
    // against 10.0 us; with 196-294 or 784 and more of them the 64-pixel tile stays ahead by 5-30 %
    if (v == 0 && a.units_pad <= 32 && wgs >= 352 && wgs <= 448 && util >= 0.95) score = 1.9;
    // fewer than 3/4 of the tile's channels real (64 output channels): the general kernel's 64-channel tiles
    // win (256 -> 64 at 56 x 56, N = 64: 13.4 against 17.1 us)
    if (util < 0.75) continue;
    if (score > best_score) { best_score = score; best = v; }
  }
  return best;
}

const char *gemm1x1_res_name(int v) { return kRes[v].name; }

hipError_t launch_gemm1x1_res(const GemmArgs &a0, int v, hipStream_t s, LaunchPlan<GemmArgs> *plan)
{
  const ResVariant &k = kRes[v];
  GemmArgs a = a0;
  a.lean = lean_mode(a.ep, false);
  a.nx = (a.p_total + k.p_t - 1) / k.p_t;
  a.ny = (a.oc2 * 16 + k.oc_t - 1) / k.oc_t;
  const int nks = a.units_pad / 2;
  res_kernel_t kernel = a.in_nhwc ? k.generic_nhwc : k.generic;
  const char *env = getenv("EHIP_GEMM1X1_UNROLL");
  if (!(env && env[0] == '0')) {
    const res_kernel_t *un = a.in_nhwc ? k.unrolled_nhwc : k.unrolled;
    if (nks == 8) kernel = un[0];
    else if (nks == 16) kernel = un[1];
    else if (nks == 32) kernel = un[2];
  }
  if (!kernel) return hipErrorInvalidValue;
  a.u1_magic = div_magic(a.units_pad + 1);
  const size_t lds_bytes = res_lds_bytes(a, k.p_t);
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)lds_bytes);
  if (e != hipSuccess) return e;
  dim3 grid(8 * a.ny * ((a.nx + 7) / 8));
  if (a.stride_h > 255 || a.stride_w > 255 || a.oc2 >= 4096) return hipErrorInvalidValue;   // geom's fields
  LaunchPlan<GemmArgs> local;
  LaunchPlan<GemmArgs> *p = plan ? plan : &local;
  p->kernel = reinterpret_cast<void (*)(GemmArgs)>(kernel);
  p->grid = grid;
  p->block = dim3(kBlock);
  p->lds = (unsigned)lds_bytes;
  p->args = a;
  p->enqueue = res_enqueue;
  p->name = k.name;   // (nhwc output: the handle could not tell at creation whether the lean epilogue applies)
  return plan_first_launch(p, s);
}

}  // namespace ehip
