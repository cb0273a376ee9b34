// u8 x s8 -> s32 GEMM on gfx950 matrix cores for the 1x1 convolutions (stride 1 and 2) and for
// the 36 independent GEMMs of the Winograd pipeline, with the requantization epilogue fused.
//
// Replaces elx_int8_conv_direct_1x1_t::__execute_a160_s1/_s2 + gemm_a160_s1/_s2
// (src/elx_int8_conv_direct_1x1_xopt.hpp:20-195, src/elx_int8_conv_direct_1x1.cpp:357-480),
// elx_int8_conv_direct_t::gemm_a160 for K=1 (src/elx_int8_conv_direct.cpp:574-718),
// elx_int8_conv_wino_gemm_t::execute (src/elx_int8_conv_wino_gemm.cpp:23-76) and the
// u8s8 micro-kernel with its epilogue (src/kernel/elk_u8s8_gemm.hxx:168-406).
//
// Mapping.  D[oc][pixel] += W[oc][k] * X[k][pixel] with v_mfma_i32_32x32x32_i8:
//   A operand = weights: lane l holds 16 consecutive input channels (unit 2*kstep + l/32) of
//               packed row l%32 (rows are packed in the order that makes a lane's results 16
//               consecutive output channels, see packed_row_of_oc),
//   B operand = activations: lane l holds the 16 channels of one nChw16c pixel cell (pixel l%32,
//               unit 2*kstep + l/32) -- 16 bytes that are contiguous in memory, so no layout
//               change is needed on the way in,
//   D         = lane l holds, for pixel l%32, 16 consecutive output channels (16*(l/32) .. +15 of
//               the 32-row tile): one 16-byte cell of u8/s8 output, four float4 of f32 output.
// The MFMA is signed x signed: activations are remapped u8 -> s8 by flipping the top bit when a
// tile is staged into LDS, and 128 * sum(weights) per output channel is added to the sums,
// which makes the s32 result identical to the unsigned product (the epilogue adds that term).
//
// A workgroup (4 waves, WM x WN) owns OC_T output channels x P_T pixels; a wave owns TM x TN MFMA
// tiles of 32 x 32.  Both operands go global -> registers -> LDS (double buffered, KC units of 16
// channels per fill; the loads of fill c+1 are in flight while fill c is multiplied) and every
// wave reads its operands from LDS one k-step ahead of the MFMAs that use them.  Two workgroups
// share a CU, so one can multiply while the other waits at its barrier.
#include "ehip_internal.hpp"

// Development aid (compile with -DEHIP_TRACE): lane 0 of every wave records the shader clock at
// phase boundaries into GemmArgs::trace.
#ifdef EHIP_TRACE
#define TRACE_POINT(i)                                                                             \
  do {                                                                                             \
    if (a.trace && lane == 0)                                                                      \
      a.trace[((size_t)(blockIdx.y * gridDim.x + blockIdx.x) * 4 + wave) * 16 + (i)] = wall_clock64(); \
  } while (0)
#else
#define TRACE_POINT(i) do { } while (0)
#endif

namespace ehip {

template <int WM, int WN, int TM, int TN, int KC, int D, bool NHWC, int CONV>
__global__ __launch_bounds__(kBlock, 2) void k_gemm_u8s8(GemmArgs a)
{
  static_assert(!(NHWC && CONV == 1), "nhwc kh x kw input works the tap out per cell");
  constexpr int OC_T = WM * TM * 32;
  constexpr int P_T = WN * TN * 32;
  constexpr int KS = KC / 2;               // MFMA k-steps per fill
  constexpr int A_CELLS = OC_T * KC;       // 16-byte cells per fill
  constexpr int B_CELLS = P_T * KC;
  constexpr int NA = A_CELLS / kBlock;
  constexpr int NB = B_CELLS / kBlock;
  constexpr int BU = kBlock / P_T;         // units covered by one pass of the workgroup over B
  static_assert(WM * WN == 4, "four waves per workgroup");
  static_assert(KC % 2 == 0, "a k-step is two units");
  static_assert(A_CELLS % kBlock == 0 && B_CELLS % kBlock == 0, "whole passes of the workgroup");
  static_assert(kBlock % P_T == 0 && OC_T <= kOcTile, "tile limits");
  static_assert(2 * (A_CELLS + B_CELLS) >= 4 * 256, "the epilogue borrows 256 LDS cells per wave");

  __shared__ v4i lds[2 * (A_CELLS + B_CELLS)];
  v4i(*lds_a)[A_CELLS] = reinterpret_cast<v4i(*)[A_CELLS]>(lds);                  // [buf][unit][row]
  v4i(*lds_b)[B_CELLS] = reinterpret_cast<v4i(*)[B_CELLS]>(lds + 2 * A_CELLS);    // [buf][unit][pixel]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform: what depends on it stays scalar
  const int l32 = lane & 31;
  const int lh = lane >> 5;
  // Workgroups go to the 8 XCDs round-robin by their linear index.  The channel blocks of one pixel
  // block are numbered so that they follow each other on ONE XCD: the first one pulls the pixels
  // into that XCD's L2, the others find them there.  An XCD takes a contiguous eighth of the pixel
  // blocks: in the kh x kw form neighbouring pixel blocks share input rows.
  const int b = blockIdx.y;
  const int xcd = blockIdx.x & 7, seq = blockIdx.x >> 3;
  const int by = seq % a.ny;
  const int bx = xcd * ((a.nx + 7) >> 3) + seq / a.ny;
  if (bx >= a.nx) return;   // whole workgroup (grid padded to a multiple of 8 pixel blocks)
  const int pix0 = bx * P_T;
  const int oc0 = by * OC_T;
  const int mw0 = (wave % WM) * TM * 32;   // wave's first row / pixel inside the workgroup tile
  const int pw0 = (wave / WM) * TN * 32;
  const int oc_real = a.oc2 * 16;
  const bool dense = !CONV && a.stride_h == 1 && a.stride_w == 1 && a.iw == a.ow;
  TRACE_POINT(0);

  // ---- staging plan ---------------------------------------------------------------------------
  // Byte offset of output pixel gp's first input cell (unit 0); nhwc: the pixel's channel vector.
  // kh x kw form (CONV): the cell under tap (0, 0), which may lie outside the image, and the set of
  // taps that fall inside it.
  long long safe_off = 0;   // a cell of the same image that every unit offset keeps in bounds
  auto input_pixel = [&](int gp, unsigned long long &tapmask) -> long long {
    gp = gp < a.p_total ? gp : a.p_total - 1;
    const int n = a.ohw == a.p_total ? 0 : fastdiv_any(gp, a.ohw, a.ohw_magic);
    const int r = gp - n * a.ohw;
    long long sp;   // pixel index inside the image
    if (dense) {
      sp = r;
    } else {
      const int oh = fastdiv(r, a.ow, a.ow_magic);
      const int ow = r - oh * a.ow;
      const int ih0 = oh * a.stride_h - (CONV ? a.pad_t : 0), iw0 = ow * a.stride_w - (CONV ? a.pad_l : 0);
      sp = (long long)ih0 * a.iw + iw0;
      if (CONV) {
        tapmask = 0;
        for (int kh = 0; kh < a.kh; ++kh)
          for (int kw = 0; kw < a.kw; ++kw)
            if (ih0 + kh >= 0 && ih0 + kh < a.ih && iw0 + kw >= 0 && iw0 + kw < a.iw) tapmask |= 1ull << (kh * a.kw + kw);
        safe_off = (long long)n * a.ic2 * a.ihw * 16;
      }
    }
    return NHWC ? ((long long)n * a.ihw + sp) * a.ic2 * 16 : ((long long)n * a.ic2 * a.ihw + sp) * 16;
  };
  // B, blocked input: a thread always copies the same pixel (tid % P_T), units tid / P_T + j * BU of
  // a fill (a unit's pixels are contiguous).  B, nhwc input: cell id = tid + j * 256 -> pixel
  // id / KC, unit id % KC (a pixel's units are contiguous: KC lanes read 16 * KC consecutive bytes).
  constexpr int NPIX = NHWC ? NB : 1;
  const uint8_t *inb[NPIX];
  unsigned long long tapmask[NPIX];   // CONV: the taps of the thread's pixel(s) that fall inside the image
#pragma unroll
  for (int j = 0; j < NPIX; ++j) {
    tapmask[j] = 0;
    inb[j] = a.in + (long long)b * a.in_batch_stride +
        input_pixel(pix0 + (NHWC ? (tid + j * kBlock) / KC : tid % P_T), tapmask[j]);
  }
  // bytes between horizontally adjacent taps of a pixel: a cell (blocked), a whole channel vector (nhwc)
  const long long tap_stride = NHWC ? (long long)a.ic2 * 16 : 16;
  const uint8_t *safe = a.in + safe_off;
  const int bu0 = NHWC ? tid % KC : tid / P_T;
  const long long unit_stride = NHWC ? 16 : (long long)a.ihw * 16;
  // A: cell id = tid + j * 256 -> unit id / OC_T, row id % OC_T; rows of a unit are contiguous.
  const int8_t *wb = a.w + (long long)b * a.units_pad * a.ocpp * 16 + (long long)oc0 * 16;
  const long long w_unit = (long long)a.ocpp * 16;

  v4i sta[D][NA], stb[D][NB];   // D fills in flight (global -> registers), see the main loop
  unsigned stz[D];              // CONV: bit j = cell j of the fill belongs to a tap outside the image
  // All global loads of the main loop are unconditional (indices clamped): without branches
  // between a load and its use the compiler counts outstanding loads exactly.
  // CONV: the K axis is [tap][unit] with the ic2 real units per tap and nothing in between (a layer
  // with few input channels would otherwise multiply mostly padding); the packed weights are
  // contiguous in that order, zero behind the last real unit, and the input cell of tap (kh, kw)
  // sits (kh * iw + kw) cells behind the one of tap (0, 0).  Cells of taps outside the image read a
  // safe cell and are replaced by u8 0 on the way to LDS, which contributes nothing -- the
  // reference skips such taps.
  auto load_stage = [&](int chunk, int d) {
#pragma unroll
    for (int j = 0; j < NA; ++j) {
      const int id = tid + j * kBlock;
      sta[d][j] = *reinterpret_cast<const v4i *>(wb + (long long)(chunk * KC + id / OC_T) * w_unit + (id % OC_T) * 16);
    }
    if (CONV == 1) {
      // ic2 is a multiple of KC: the whole fill belongs to one tap (scalar arithmetic)
      const int tap = fastdiv(chunk * KC, a.ic2, a.ic2_magic);
      const int ub = chunk * KC - tap * a.ic2;
      const int kh = fastdiv(tap, a.kw, a.kw_magic);
      const bool inside = (tapmask[0] >> tap) & 1;
      stz[d] = inside ? 0u : ~0u;
      const uint8_t *src = inside ? inb[0] + (long long)(kh * a.iw + (tap - kh * a.kw)) * 16 : safe;
#pragma unroll
      for (int j = 0; j < NB; ++j)
        stb[d][j] = *reinterpret_cast<const v4i *>(src + (long long)(ub + bu0 + j * BU) * unit_stride);
      return;
    }
    if (CONV) stz[d] = 0u;
#pragma unroll
    for (int j = 0; j < NB; ++j) {
      int u = chunk * KC + bu0 + (NHWC ? 0 : j * BU);
      const uint8_t *src = inb[NHWC ? j : 0];
      if (CONV) {   // any ic2: the tap is worked out per cell
        u = u < a.k_real ? u : a.k_real - 1;   // behind the last real unit the weights are zero
        const int tap = fastdiv(u, a.ic2, a.ic2_magic);
        u -= tap * a.ic2;
        const int kh = fastdiv(tap, a.kw, a.kw_magic);
        const bool inside = (tapmask[NHWC ? j : 0] >> tap) & 1;
        stz[d] |= inside ? 0u : 1u << j;
        src = inside ? inb[NHWC ? j : 0] + (long long)(kh * a.iw + (tap - kh * a.kw)) * tap_stride : safe;
      } else {
        u = u < a.ic2 ? u : a.ic2 - 1;  // padded units multiply zero weights: any valid cell will do
      }
      stb[d][j] = *reinterpret_cast<const v4i *>(src + (long long)u * unit_stride);
    }
  };
  // LDS keeps B as [unit][pixel].  The nhwc plan writes one pixel's KC units from neighbouring
  // lanes, which would all land in the same banks: there pixel p of unit u sits at p ^ (2u & 15),
  // a permutation inside every aligned group of 16 pixels that spreads those writes over all banks
  // and leaves the reads (32 consecutive pixels of one unit) conflict free.
  auto store_stage = [&](int buf, int d) {
#pragma unroll
    for (int j = 0; j < NA; ++j) lds_a[buf][tid + j * kBlock] = sta[d][j];
#pragma unroll
    for (int j = 0; j < NB; ++j) {
      const int id = tid + j * kBlock;
      const int cell = NHWC ? (id % KC) * P_T + ((id / KC) ^ ((2 * (id % KC)) & 15)) : id;
      const v4i x = (CONV && ((stz[d] >> j) & 1u)) ? v4i{0, 0, 0, 0} : stb[d][j];
      lds_b[buf][cell] = x ^ (int)0x80808080;
    }
  };

  // The accumulators start from the compensation 128 * sum(weights) of their channel instead of zero
  // (requested before the first fill's loads, so it costs the epilogue nothing).
  const long long cidx = (long long)b * a.ocpp + oc0 + mw0 + 16 * lh;   // the lane's 16 channels of tile 0
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

  // ---- main loop ------------------------------------------------------------------------------
  v4i opa[2][TM], opb[2][TN];
  auto read_ops = [&](int buf, int ks, int slot) {
    const v4i *pa = &lds_a[buf][(2 * ks + lh) * OC_T + mw0 + l32];
    const v4i *pb = &lds_b[buf][(2 * ks + lh) * P_T + pw0 + (NHWC ? l32 ^ ((4 * ks + 2 * lh) & 15) : l32)];
#pragma unroll
    for (int mt = 0; mt < TM; ++mt) opa[slot][mt] = pa[mt * 32];
#pragma unroll
    for (int nt = 0; nt < TN; ++nt) opb[slot][nt] = pb[nt * 32];
  };
  // The scheduling barriers keep the compiler from sinking the operand prefetch next to its use.
  auto multiply = [&](int buf) {
    read_ops(buf, 0, 0);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      if (ks + 1 < KS) read_ops(buf, ks + 1, (ks + 1) & 1);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int mt = 0; mt < TM; ++mt)
#pragma unroll
        for (int nt = 0; nt < TN; ++nt)
          acc[mt][nt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(opa[ks & 1][mt], opb[ks & 1][nt], acc[mt][nt], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  const int nchunks = a.k_units / KC;
  // The layers this kernel serves are small: what a workgroup waits for is the latency of its
  // global loads, not their bandwidth.  So D fills are kept in flight in registers: the loads of
  // fill c + D are issued when fill c moves to LDS.  The launcher picks D so that it divides the
  // number of fills; the last D fills are peeled and prefetch nothing.
  const int ngroups = nchunks / D;
#pragma unroll
  for (int d = 0; d < D; ++d) load_stage(d, d);
  TRACE_POINT(1);
  int buf = 0;
  for (int g = 0; g + 1 < ngroups; ++g) {
#pragma unroll
    for (int d = 0; d < D; ++d) {
      store_stage(buf, d);
      if (g == 0 && d == 0) TRACE_POINT(2);
      __syncthreads();
      if (g == 0 && d == 0) TRACE_POINT(3);
      load_stage((g + 1) * D + d, d);
      multiply(buf);
      if (g == 0 && d == 0) TRACE_POINT(4);
      buf ^= 1;
    }
  }
  TRACE_POINT(5);
  OcConsts k0;
  LeanConsts lk[TM];
#pragma unroll
  for (int d = 0; d < D; ++d) {
    store_stage(buf, d);
    __syncthreads();
    // the epilogue's per-channel constants travel while the last fill is multiplied
    if (d == D - 1) {
      if (a.lean) {
#pragma unroll
        for (int mt = 0; mt < TM; ++mt) load_lean_consts(lk[mt], a.ep, cidx + 32 * mt);
      } else {
        load_consts(k0, a.ep, cidx);
      }
    }
    multiply(buf);
    buf ^= 1;
  }
  TRACE_POINT(6);

  if (a.lean) {   // u8 / s8 with ReLU bounds, per-channel shift: no output-type switch
    // the lane's 16 bytes: its pixel's cell in 16-channel block (oc0 + mw0) / 16 + lh, or (nhwc) channels
    // oc0 + mw0 + 16 lh .. + 15 of its pixel's vector; the next 32-channel tile is two blocks / 32 bytes on
    uint8_t *cell[TN];
    bool pv[TN];
#pragma unroll
    for (int nt = 0; nt < TN; ++nt) {
      const int gp = pix0 + pw0 + nt * 32 + l32;
      pv[nt] = gp < a.p_total;
      const int gpc = pv[nt] ? gp : 0;
      if (a.out_nhwc) {
        cell[nt] = static_cast<uint8_t *>(a.out) + (size_t)gpc * oc_real + (oc0 + mw0 + 16 * lh);
      } else {
        const int n = a.ohw == a.p_total ? 0 : fastdiv_any(gpc, a.ohw, a.ohw_magic);
        const int r = gpc - n * a.ohw;
        cell[nt] = static_cast<uint8_t *>(a.out) + (size_t)b * a.out_batch_stride +
            (((size_t)n * a.oc2 + ((oc0 + mw0) >> 4) + lh) * a.ohw + r) * 16;
      }
    }
    // (non-temporal stores for blocked output only: in nhwc a line's pieces come from several waves)
    if (a.out_nhwc) lean_store<TM, TN>(a.lean, a.ep, acc, lk, cell, pv, oc0 + mw0 + 16 * lh, oc_real, (size_t)32);
    else lean_store<TM, TN, true>(a.lean, a.ep, acc, lk, cell, pv, oc0 + mw0 + 16 * lh, oc_real, (size_t)2 * a.ohw * 16);
    TRACE_POINT(15);
    return;
  }

  // ---- epilogue ------------------------------------------------------------------------------
  // element offset of output pixel gp's cell in 16-channel block 0 (nhwc: its channel vector)
  auto pixel_offset = [&](int gp, bool &valid) -> size_t {
    valid = gp < a.p_total;
    const int gpc = valid ? gp : 0;
    if (a.out_nhwc) return (size_t)gpc * oc_real;
    const int n = a.ohw == a.p_total ? 0 : fastdiv_any(gpc, a.ohw, a.ohw_magic);
    const int r = gpc - n * a.ohw;
    return (size_t)b * a.out_batch_stride + ((size_t)n * a.oc2 * a.ohw + r) * 16;
  };
  size_t pix[TN], pixT[TN][2];
  bool pvalid[TN], validT[TN][2];
  int cls[TN];
#pragma unroll
  for (int nt = 0; nt < TN; ++nt) {
    cls[nt] = 0;
    if (CONV && a.ep.shift_tab) {   // border class of the lane's pixel
      int gp = pix0 + pw0 + nt * 32 + l32;
      gp = gp < a.p_total ? gp : a.p_total - 1;
      const int r = gp - (a.ohw == a.p_total ? 0 : fastdiv_any(gp, a.ohw, a.ohw_magic)) * a.ohw;
      const int oh = fastdiv(r, a.ow, a.ow_magic);
      cls[nt] = a.cls_h[oh] * a.ncls_w + a.cls_w[r - oh * a.ow];
    }
    pix[nt] = pixel_offset(pix0 + pw0 + nt * 32 + l32, pvalid[nt]);
    pixT[nt][0] = pixel_offset(pix0 + pw0 + nt * 32 + (lane >> 2), validT[nt][0]);
    pixT[nt][1] = pixel_offset(pix0 + pw0 + nt * 32 + (lane >> 2) + 16, validT[nt][1]);
  }
  // 4-byte outputs are exchanged through a wave-private 4 KB patch of the (now idle) operand LDS
  v4i *xlds = nullptr;
  if ((a.ep.out_type == EHIP_F32 || a.ep.out_type == EHIP_S32) && !a.out_nhwc) {
    __syncthreads();   // every wave has read its last operands
    xlds = lds + wave * 256;
  }
  TRACE_POINT(14);
  epilogue_wave<TM, TN, CONV != 0, true>(a.ep, acc, k0, cidx, oc0 + mw0 + 16 * lh, pix, pvalid, oc_real,
                                         a.out_nhwc ? (size_t)16 : (size_t)a.ohw * 16, a.out, xlds, pixT, validT, cls);
  TRACE_POINT(15);
}

// ---- 1x1 layers with few input channels: weights stay in registers ---------------------------
// With K <= 128 a workgroup of the kernel above multiplies for a few hundred clocks and spends the
// rest of its life on start-up, barriers and its epilogue -- and such a layer needs thousands of
// them.  Here nothing is shared: a wave loads the weights of its 32 output channels ONCE into
// registers (KS operands of one 32-channel tile), then walks over 32-pixel tiles: the tile's activations go straight
// from memory into MFMA operands (a lane's operand is one 16-byte cell, blocked or nhwc), the next
// tile's are in flight while this one is multiplied, and the results leave through the same
// epilogue.  No LDS (apart from the 4 KB exchange patch of 4-byte outputs), no barrier.
// The four waves of a workgroup split into a.sk_wo tiles of 32 channels (1, 2 or 4) times
// 4 / a.sk_wo pixel tiles of TNW x 32 pixels; waves of different channel groups walk the same tiles at the same time,
// so the activations reach the CU once.  grid: (workgroups over pixel tiles, 4-wave channel blocks).
// What a wave's first loads need -- the two pointers and the geometry their addresses are made of -- is passed as
// leading scalar arguments, which the dispatcher preloads into scalar registers with the wave (the file is compiled
// with -amdgpu-kernarg-preload-count=16); the rest of the argument block is loaded as usual meanwhile.
// geom = stride_h | stride_w << 8 | dense << 16 | in_nhwc << 17 | out_nhwc << 18 | sk_wo << 20.
#define EHIP_SMALLK_HEAD                                                                                             \
  const uint8_t *in, const int8_t *w, int p_total, int ohw, unsigned ohw_magic, int ihw, int ic2, int ocpp, int oc2, \
      unsigned geom, int iw, int ow, unsigned ow_magic
template <int TNW, int KS>
__global__ __launch_bounds__(kBlock, 2) void k_gemm_smallk_u8s8(EHIP_SMALLK_HEAD, GemmArgs rest)
{
  GemmArgs a = rest;
  a.in = in; a.w = w; a.p_total = p_total; a.ohw = ohw; a.ohw_magic = ohw_magic; a.ihw = ihw; a.ic2 = ic2; a.ocpp = ocpp;
  a.oc2 = oc2; a.iw = iw; a.ow = ow; a.ow_magic = ow_magic;
  a.stride_h = (int)(geom & 0xffu); a.stride_w = (int)((geom >> 8) & 0xffu);
  a.in_nhwc = (int)((geom >> 17) & 1u); a.out_nhwc = (int)((geom >> 18) & 1u); a.sk_wo = (int)(geom >> 20);
  __shared__ v4i xpatch[4 * 256];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform: what depends on it stays scalar
  const int l32 = lane & 31;
  const int lh = lane >> 5;
  const int wo = wave % a.sk_wo, wp = wave / a.sk_wo, wpn = 4 / a.sk_wo;
  const int oc0 = (blockIdx.y * a.sk_wo + wo) * 32;
  const int oc_real = a.oc2 * 16;
  const bool dense = a.stride_h == 1 && a.stride_w == 1 && a.iw == a.ow;
  const long long unit_stride = a.in_nhwc ? 16 : (long long)a.ihw * 16;

  // weights: packed [unit][OCpp rows][16]; lane = row l32 of the wave's tile, unit 2 ks + lh
  v4i wreg[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks)
    wreg[ks] = *reinterpret_cast<const v4i *>(a.w + ((long long)(2 * ks + lh) * a.ocpp + oc0 + l32) * 16);

  // byte offset of output pixel gp's first input cell (clamped past the end)
  auto input_pixel = [&](int gp) -> long long {
    gp = gp < a.p_total ? gp : a.p_total - 1;
    const int n = a.ohw == a.p_total ? 0 : fastdiv_any(gp, a.ohw, a.ohw_magic);
    const int r = gp - n * a.ohw;
    long long sp;
    if (dense) {
      sp = r;
    } else {
      const int oh = fastdiv(r, a.ow, a.ow_magic);
      sp = (long long)(oh * a.stride_h) * a.iw + (r - oh * a.ow) * a.stride_w;
    }
    return a.in_nhwc ? ((long long)n * a.ihw + sp) * a.ic2 * 16 : ((long long)n * a.ic2 * a.ihw + sp) * 16;
  };
  auto pixel_offset = [&](int gp, bool &valid) -> size_t {
    valid = gp < a.p_total;
    const int gpc = valid ? gp : 0;
    if (a.out_nhwc) return (size_t)gpc * oc_real;
    const int n = a.ohw == a.p_total ? 0 : fastdiv_any(gpc, a.ohw, a.ohw_magic);
    return ((size_t)n * a.oc2 * a.ohw + (gpc - n * a.ohw)) * 16;
  };
  // the lane's units: 2 ks + lh, clamped to the real ones (padded units multiply zero weights)
  int ucl[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) ucl[ks] = 2 * ks + lh < a.ic2 ? 2 * ks + lh : a.ic2 - 1;

  // a wave-tile is TNW x 32 consecutive pixels
  const int ntiles = (a.p_total + 32 * TNW - 1) / (32 * TNW);
  const int tstep = wpn * gridDim.x;
  int tile = wpn * blockIdx.x + wp;
  v4i breg[TNW][KS];
  auto load_b = [&](int t) {
#pragma unroll
    for (int nt = 0; nt < TNW; ++nt) {
      const uint8_t *src = a.in + input_pixel((t * TNW + nt) * 32 + l32);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) breg[nt][ks] = *reinterpret_cast<const v4i *>(src + (long long)ucl[ks] * unit_stride);
    }
  };
  if (tile < ntiles) load_b(tile);
  const long long cidx = oc0 + 16 * lh;
  // the per-channel constants of the wave's tile stay in registers for all its pixel tiles (fetched
  // per tile they would cost the vector-memory path more than the activations do)
  OcConsts k0;
  load_consts(k0, a.ep, cidx);
  // Lean epilogue (a.lean, decided by the launcher: u8 / s8 output, ReLU, per-channel shift): these
  // layers produce an output value per 32-128 multiply-adds, so the epilogue's instructions per value, not
  // the multiplies, are what a tile costs; the lean form takes 3-4 of them where the general one takes ~10.
  // Its accumulators start from the compensation instead of zero.
  LeanConsts lk[1];
  v16i acc0;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc0[v] = 0;
  if (a.lean) {
    load_lean_consts(lk[0], a.ep, cidx);
#pragma unroll
    for (int v = 0; v < 16; ++v) acc0[v] = k0.comp[v >> 2][v & 3];
  }
  v4i *xlds = ((a.ep.out_type == EHIP_F32 || a.ep.out_type == EHIP_S32) && !a.out_nhwc) ? xpatch + wave * 256 : nullptr;
  for (; tile < ntiles; tile += tstep) {
    v16i acc[1][TNW];
#pragma unroll
    for (int nt = 0; nt < TNW; ++nt) acc[0][nt] = acc0;
    v4i bcur[TNW][KS];
#pragma unroll
    for (int nt = 0; nt < TNW; ++nt)
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) bcur[nt][ks] = breg[nt][ks] ^ (int)0x80808080;
    // next tile's activations travel during this tile's multiplies and epilogue (the last wave-tile
    // re-reads its own)
    load_b(tile + tstep < ntiles ? tile + tstep : tile);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int nt = 0; nt < TNW; ++nt)
        acc[0][nt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wreg[ks], bcur[nt][ks], acc[0][nt], 0, 0, 0);
    size_t pix[TNW], pixT[TNW][2];
    bool pvalid[TNW], validT[TNW][2];
    if (a.lean) {   // the lane's 16 bytes: its pixel in 16-channel block (oc0 / 16) + lh, or of its nhwc vector
      uint8_t *cell[TNW];
#pragma unroll
      for (int nt = 0; nt < TNW; ++nt) {
        const size_t px = pixel_offset((tile * TNW + nt) * 32 + l32, pvalid[nt]);
        cell[nt] = static_cast<uint8_t *>(a.out) + px +
            (a.out_nhwc ? (size_t)(oc0 + 16 * lh) : ((size_t)(oc0 >> 4) + lh) * a.ohw * 16);
      }
      if (a.out_nhwc) lean_store<1, TNW>(a.lean, a.ep, acc, lk, cell, pvalid, oc0 + 16 * lh, oc_real, (size_t)32);
      else lean_store<1, TNW, true>(a.lean, a.ep, acc, lk, cell, pvalid, oc0 + 16 * lh, oc_real, (size_t)2 * a.ohw * 16);
      continue;
    }
#pragma unroll
    for (int nt = 0; nt < TNW; ++nt) {
      const int p0 = (tile * TNW + nt) * 32;
      pix[nt] = pixel_offset(p0 + l32, pvalid[nt]);
      pixT[nt][0] = pixel_offset(p0 + (lane >> 2), validT[nt][0]);
      pixT[nt][1] = pixel_offset(p0 + (lane >> 2) + 16, validT[nt][1]);
    }
    epilogue_wave<1, TNW>(a.ep, acc, k0, cidx, oc0 + 16 * lh, pix, pvalid, oc_real,
                          a.out_nhwc ? (size_t)16 : (size_t)a.ohw * 16, a.out, xlds, pixT, validT);
  }
}

// The same walk for the lean epilogue's cases (u8 / s8 output, ReLU, per-channel shift), with OCW
// tiles of 32 output channels per wave instead of one.  A layer like 64 -> 256 at 56 x 56 writes four
// times the bytes it reads; with one channel tile per wave every activation cell is pulled from L2 once
// per channel tile (eight times), which then outweighs the output.  Here a wave keeps the weights of all
// its OCW tiles in registers (OCW x KS <= 8 operands), reads a pixel tile once and produces OCW x 32
// channels from it.  Scale, shift and the accumulators' start values (the u8 -> s8 compensation) of the
// wave's channels sit in a wave-private piece of LDS -- in registers they would take 48 per tile -- and every
// lane of a half-wave reads the same 16 bytes of them (a broadcast).
template <int KS, int OCW>
__global__ __launch_bounds__(kBlock, 2) void k_gemm_smallk_lean(EHIP_SMALLK_HEAD, GemmArgs rest)
{
  GemmArgs a = rest;
  a.in = in; a.w = w; a.p_total = p_total; a.ohw = ohw; a.ohw_magic = ohw_magic; a.ihw = ihw; a.ic2 = ic2; a.ocpp = ocpp;
  a.oc2 = oc2; a.iw = iw; a.ow = ow; a.ow_magic = ow_magic;
  a.stride_h = (int)(geom & 0xffu); a.stride_w = (int)((geom >> 8) & 0xffu);
  a.in_nhwc = (int)((geom >> 17) & 1u); a.out_nhwc = (int)((geom >> 18) & 1u); a.sk_wo = (int)(geom >> 20);
  __shared__ float4 cst_lds[4 * OCW * 24];   // [wave][tile][scale | shift | compensation][8 cells of 4 channels]
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform: what depends on it stays scalar
  const int l32 = lane & 31;
  const int lh = lane >> 5;
  const int wo = wave % a.sk_wo, wp = wave / a.sk_wo, wpn = 4 / a.sk_wo;
  const int oc0 = (blockIdx.y * a.sk_wo + wo) * OCW * 32;
  const int oc_real = a.oc2 * 16;
  const bool dense = a.stride_h == 1 && a.stride_w == 1 && a.iw == a.ow;
  const long long unit_stride = (long long)a.ihw * 16;

  v4i wreg[OCW][KS];
#pragma unroll
  for (int ot = 0; ot < OCW; ++ot)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      wreg[ot][ks] = *reinterpret_cast<const v4i *>(a.w + ((long long)(2 * ks + lh) * a.ocpp + oc0 + 32 * ot + l32) * 16);
  float4 *cst = cst_lds + wave * (OCW * 24);
  for (int i = lane; i < OCW * 24; i += 64) {
    const int ot = i / 24, r = i - 24 * ot, arr = r >> 3, c = r & 7;
    const float *src = arr == 0 ? a.ep.scale : (arr == 1 ? a.ep.shift : reinterpret_cast<const float *>(a.ep.comp));
    cst[i] = *reinterpret_cast<const float4 *>(src + oc0 + 32 * ot + 4 * c);
  }

  auto input_pixel = [&](int gp) -> long long {
    gp = gp < a.p_total ? gp : a.p_total - 1;
    const int n = a.ohw == a.p_total ? 0 : fastdiv_any(gp, a.ohw, a.ohw_magic);
    const int r = gp - n * a.ohw;
    long long sp;
    if (dense) {
      sp = r;
    } else {
      const int oh = fastdiv(r, a.ow, a.ow_magic);
      sp = (long long)(oh * a.stride_h) * a.iw + (r - oh * a.ow) * a.stride_w;
    }
    return a.in_nhwc ? ((long long)n * a.ihw + sp) * a.ic2 * 16 : ((long long)n * a.ic2 * a.ihw + sp) * 16;
  };
  int ucl[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) ucl[ks] = 2 * ks + lh < a.ic2 ? 2 * ks + lh : a.ic2 - 1;
  const long long ustride = a.in_nhwc ? 16 : unit_stride;

  const int ntiles = (a.p_total + 31) / 32;
  const int tstep = wpn * gridDim.x;
  int tile = wpn * blockIdx.x + wp;
  v4i breg[KS];
  auto load_b = [&](int t) {
    const uint8_t *src = a.in + input_pixel(t * 32 + l32);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) breg[ks] = *reinterpret_cast<const v4i *>(src + (long long)ucl[ks] * ustride);
  };
  if (tile < ntiles) load_b(tile);
  __builtin_amdgcn_wave_barrier();   // the constants are the wave's own: its LDS writes are done before its reads
  for (; tile < ntiles; tile += tstep) {
    v4i bcur[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) bcur[ks] = breg[ks] ^ (int)0x80808080;
    load_b(tile + tstep < ntiles ? tile + tstep : tile);
    // the lane's cell of 16-channel block (oc0 / 16) + lh
    const int gp = tile * 32 + l32;
    bool pvalid[1] = {gp < a.p_total};
    const int gpc = pvalid[0] ? gp : 0;
    const int n = a.ohw == a.p_total ? 0 : fastdiv_any(gpc, a.ohw, a.ohw_magic);
    uint8_t *const cell0 = static_cast<uint8_t *>(a.out) +
        (a.out_nhwc ? (size_t)gpc * oc_real + (oc0 + 16 * lh)
                    : (((size_t)n * a.oc2 + (oc0 >> 4) + lh) * a.ohw + (gpc - n * a.ohw)) * 16);
    const size_t tile_stride = a.out_nhwc ? (size_t)32 : (size_t)2 * a.ohw * 16;
    // The multiplies of tile ot + 1 are issued before the epilogue of tile ot and run behind it; the
    // scheduling barriers keep the compiler from pulling all OCW tiles' constants and accumulators up front
    // (it then runs out of registers).
    v16i acc2[2];
    auto multiply = [&](int ot) {
      const float4 *k = cst + ot * 24 + 4 * lh;
      v16i x;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const float4 c = k[16 + q];
        x[4 * q + 0] = __float_as_int(c.x);
        x[4 * q + 1] = __float_as_int(c.y);
        x[4 * q + 2] = __float_as_int(c.z);
        x[4 * q + 3] = __float_as_int(c.w);
      }
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) x = __builtin_amdgcn_mfma_i32_32x32x32_i8(wreg[ot][ks], bcur[ks], x, 0, 0, 0);
      acc2[ot & 1] = x;
    };
    multiply(0);
#pragma unroll
    for (int ot = 0; ot < OCW; ++ot) {
      if (ot + 1 < OCW) multiply(ot + 1);
      __builtin_amdgcn_sched_barrier(0);
      const float4 *k = cst + ot * 24 + 4 * lh;
      LeanConsts lk[1];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        lk[0].sc[q] = k[q];
        lk[0].sh[q] = k[8 + q];
      }
      v16i acc[1][1];
      acc[0][0] = acc2[ot & 1];
      uint8_t *cell[1] = {cell0 + (size_t)ot * tile_stride};
      if (a.out_nhwc) lean_store<1, 1>(a.lean, a.ep, acc, lk, cell, pvalid, oc0 + 32 * ot + 16 * lh, oc_real, tile_stride);
      else lean_store<1, 1, true>(a.lean, a.ep, acc, lk, cell, pvalid, oc0 + 32 * ot + 16 * lh, oc_real, tile_stride);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
}

namespace {
struct Variant {
  const char *name;
  int oc_t, p_t, kc;
  // [blocked | nhwc | blocked kh x kw, ic2 % KC == 0 | blocked kh x kw, any ic2 | nhwc kh x kw][prefetch depth 1, 2, 4]
  // (null: not built)
  void (*kernel[5][3])(GemmArgs);
};
// depth 4 only where four fills of staging fit in 96 registers
template <int WM, int WN, int TM, int TN, int KC, bool NHWC>
constexpr void (*deep_or_null())(GemmArgs)
{
  if constexpr (4 * ((WM * TM + WN * TN) * 32 * KC / kBlock) * 4 <= 96) return k_gemm_u8s8<WM, WN, TM, TN, KC, 4, NHWC, 0>;
  else return nullptr;
}
#define V(WM, WN, TM, TN, KC)                                                                    \
  { "k_gemm_u8s8<" #WM "," #WN "," #TM "," #TN "," #KC ">", WM * TM * 32, WN * TN * 32, KC,       \
    { { k_gemm_u8s8<WM, WN, TM, TN, KC, 1, false, 0>, k_gemm_u8s8<WM, WN, TM, TN, KC, 2, false, 0>,                 \
        deep_or_null<WM, WN, TM, TN, KC, false>() },                                                              \
      { k_gemm_u8s8<WM, WN, TM, TN, KC, 1, true, 0>, k_gemm_u8s8<WM, WN, TM, TN, KC, 2, true, 0>,                   \
        deep_or_null<WM, WN, TM, TN, KC, true>() },                                                               \
      { k_gemm_u8s8<WM, WN, TM, TN, KC, 1, false, 1>, k_gemm_u8s8<WM, WN, TM, TN, KC, 2, false, 1>, nullptr },      \
      { k_gemm_u8s8<WM, WN, TM, TN, KC, 1, false, 2>, k_gemm_u8s8<WM, WN, TM, TN, KC, 2, false, 2>, nullptr },      \
      { k_gemm_u8s8<WM, WN, TM, TN, KC, 1, true, 2>, k_gemm_u8s8<WM, WN, TM, TN, KC, 2, true, 2>, nullptr } } }
const Variant kVariants[] = {
    V(2, 2, 2, 2, 8),  // 0: 128 oc x 128 px
    V(2, 2, 2, 1, 8),  // 1: 128 oc x  64 px
    V(4, 1, 2, 2, 8),  // 2: 256 oc x  64 px
    V(2, 2, 1, 1, 8),  // 3:  64 oc x  64 px
    V(4, 1, 2, 1, 8),  // 4: 256 oc x  32 px
    V(2, 2, 1, 2, 8),  // 5:  64 oc x 128 px
    V(2, 2, 1, 1, 4),  // 6:  64 oc x  64 px, short K
};
#undef V
constexpr int kNumVariants = sizeof(kVariants) / sizeof(kVariants[0]);
}  // namespace

const char *gemm_variant_name(int v) { return kVariants[v].name; }
int gemm_variant_chunk(int v) { return kVariants[v].kc; }
int gemm_num_variants() { return kNumVariants; }

// Score = useful fraction of the padded tile grid x how well the grid fills the chip (two
// workgroups per CU) x operand reuse of the tile.
int gemm_pick_variant(int p_total, int oc2, int ic2, int nbatch, int stride)
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
    const int gx = (p_total + k.p_t - 1) / k.p_t, gy = (oc + k.oc_t - 1) / k.oc_t;
    const long long wgs = (long long)gx * gy * nbatch;
    const double util = ((double)oc / ((double)gy * k.oc_t)) * ((double)p_total / ((double)gx * k.p_t)) *
                        ((double)ic2 / (double)up(ic2, k.kc));
    const long long rounds = (wgs + 511) / 512;
    const double fill = (double)wgs / (double)(rounds * 512);
    double reuse = (double)k.oc_t * k.p_t / (double)(k.oc_t + k.p_t) / 64.0;  // 1.0 for 128 x 128
    // a strided 1x1 gathers its pixels in 16-byte pieces: the more channels share one gather the better
    if (stride > 1) reuse *= (double)k.oc_t / 128.0;
    const double score = util * fill * (0.25 + reuse);
    if (score > best_score) { best_score = score; best = v; }
  }
  return best;
}

namespace {
typedef void (*smallk_kernel_t)(EHIP_SMALLK_HEAD, GemmArgs);
template <int KS>
smallk_kernel_t smallk_kernel(int tnw)
{
  (void)tnw;   // (two pixel tiles per iteration cost more in occupancy than they gain in overlap: one)
  return k_gemm_smallk_u8s8<1, KS>;
}
hipError_t smallk_enqueue(const LaunchPlan<GemmArgs> &plan, hipStream_t s)
{
  const GemmArgs &a = plan.args;
  const bool dense = a.stride_h == 1 && a.stride_w == 1 && a.iw == a.ow;
  const unsigned geom = (unsigned)a.stride_h | (unsigned)a.stride_w << 8 | (dense ? 1u << 16 : 0u) | (a.in_nhwc ? 1u << 17 : 0u) |
      (a.out_nhwc ? 1u << 18 : 0u) | (unsigned)a.sk_wo << 20;
  hipLaunchKernelGGL(reinterpret_cast<smallk_kernel_t>(plan.kernel), plan.grid, plan.block, plan.lds, s, a.in, a.w, a.p_total,
                     a.ohw, a.ohw_magic, a.ihw, a.ic2, a.ocpp, a.oc2, geom, a.iw, a.ow, a.ow_magic, a);
  return hipGetLastError();
}
hipError_t smallk_launch(LaunchPlan<GemmArgs> *plan, smallk_kernel_t kernel, dim3 grid, const GemmArgs &a, hipStream_t s)
{
  if (a.stride_h > 255 || a.stride_w > 255) return hipErrorInvalidValue;   // geom's fields
  LaunchPlan<GemmArgs> local;
  LaunchPlan<GemmArgs> *p = plan ? plan : &local;
  p->kernel = reinterpret_cast<void (*)(GemmArgs)>(kernel);
  p->grid = grid;
  p->block = dim3(kBlock);
  p->lds = 0;
  p->args = a;
  p->enqueue = smallk_enqueue;
  return plan_first_launch(p, s);
}
}  // namespace

// 1x1 layers with at most 8 input units (128 channels): the weights-in-registers kernel.  The channel
// rows past the last real block are zero rows of the packed weights (OCpp is a multiple of 256).
bool gemm_smallk_applies(int ic2, int taps, int nbatch)
{
  const char *env = getenv("EHIP_GEMM_SMALLK");
  if (env && env[0] == '0') return false;
  return nbatch == 1 && taps <= 1 && ic2 <= 8;
}

hipError_t launch_gemm_smallk(const GemmArgs &a0, hipStream_t s, LaunchPlan<GemmArgs> *plan = nullptr)
{
  GemmArgs a = a0;
  a.lean = lean_mode(a.ep, false);   // blocked and nhwc output alike
  const int ks = a.ic2 <= 2 ? 1 : (a.ic2 <= 4 ? 2 : 4);
  const int oc_tiles = (a.oc2 * 16 + 31) / 32;
  // one tile of 32 channels per wave (its constants then stay in registers) x two tiles of 32 pixels
  const int groups = oc_tiles;
  a.sk_wo = groups >= 4 ? 4 : (groups >= 2 ? 2 : 1);
  const int ny = (groups + a.sk_wo - 1) / a.sk_wo;
  const int tnw = 1;   // (two pixel tiles per iteration cost more in occupancy than they gain in overlap)
  const int ntiles = (a.p_total + 32 * tnw - 1) / (32 * tnw);
  const int wpn = 4 / a.sk_wo;
  // one resident set of workgroups, so that a wave amortises its weights over many tiles
  int nx = (ntiles + wpn - 1) / wpn;
  const int wgs = 768;   // three workgroups per CU: what the register budget of the one-tile form admits, and the measured optimum
  const int cap = (wgs + ny - 1) / ny;
  if (nx > cap) nx = cap;
  smallk_kernel_t kernel = ks == 1 ? smallk_kernel<1>(tnw) : (ks == 2 ? smallk_kernel<2>(tnw) : smallk_kernel<4>(tnw));
  // lean epilogue and blocked activations: several channel tiles per wave.  Measured at N = 64 (64 -> 256 and
  // 64 -> 128 at 56 x 56, 128 -> 512 at 28 x 28, 128 -> 128 at 56 x 56, 32 -> 64 at 112 x 112): four tiles per
  // wave up to 64 input channels, two above (more weights in registers cost a resident workgroup), 20-25 %
  // faster than one; eight tiles lose again.
  int ocw = ks == 4 ? 2 : 4;
  while (ocw > 1 && ocw > oc_tiles) ocw >>= 1;
  if (a.lean && ocw > 1) {
    const int groups2 = (oc_tiles + ocw - 1) / ocw;
    a.sk_wo = groups2 >= 4 ? 4 : (groups2 >= 2 ? 2 : 1);
    const int ny2 = (groups2 + a.sk_wo - 1) / a.sk_wo;
    const int wpn2 = 4 / a.sk_wo;
    const int ntiles2 = (a.p_total + 31) / 32;
    int nx2 = (ntiles2 + wpn2 - 1) / wpn2;
    // one resident set: four workgroups per CU with the weights of up to 32 channels per lane, else three
    const int wgs2 = ks == 1 ? 1024 : 768;
    const int cap2 = (wgs2 + ny2 - 1) / ny2;
    if (nx2 > cap2) nx2 = cap2;
    smallk_kernel_t lk = nullptr;
    if (ks == 1) lk = ocw == 4 ? k_gemm_smallk_lean<1, 4> : k_gemm_smallk_lean<1, 2>;
    else if (ks == 2) lk = ocw == 4 ? k_gemm_smallk_lean<2, 4> : k_gemm_smallk_lean<2, 2>;
    else lk = k_gemm_smallk_lean<4, 2>;
    if (plan) {
      static const char *const names[3][2] = {{"k_gemm_smallk_lean<1,2>", "k_gemm_smallk_lean<1,4>"},
                                              {"k_gemm_smallk_lean<2,2>", "k_gemm_smallk_lean<2,4>"},
                                              {"k_gemm_smallk_lean<4,2>", "k_gemm_smallk_lean<4,2>"}};
      plan->name = names[ks == 1 ? 0 : (ks == 2 ? 1 : 2)][ocw == 4 ? 1 : 0];
    }
    return smallk_launch(plan, lk, dim3(nx2, ny2), a, s);
  }
  return smallk_launch(plan, kernel, dim3(nx, ny), a, s);
}

hipError_t launch_gemm(const GemmArgs &a0, int nbatch, int variant, hipStream_t s, LaunchPlan<GemmArgs> *plan)
{
  if (plan && plan->valid) {   // everything but the tensors is as on the first launch
    return plan_relaunch(*plan, [&](GemmArgs &x) { x.in = a0.in; x.out = a0.out; }, s);
  }
  if (gemm1x1_wres_applies(a0, nbatch)) return launch_gemm1x1_wres(a0, s, plan);
  if (gemm_smallk_applies(a0.ic2, a0.kh * a0.kw, nbatch)) return launch_gemm_smallk(a0, s, plan);
  {
    const int rv = gemm1x1_res_pick(a0, nbatch);
    if (rv >= 0) return launch_gemm1x1_res(a0, rv, s, plan);
  }
  const Variant &k = kVariants[variant];
  GemmArgs a = a0;
  a.lean = lean_mode(a.ep, false);   // blocked and nhwc output alike
  a.nx = (a.p_total + k.p_t - 1) / k.p_t;
  a.ny = (a.oc2 * 16 + k.oc_t - 1) / k.oc_t;
  dim3 grid(8 * a.ny * ((a.nx + 7) / 8), nbatch);
  // prefetch depth: must divide the number of fills.  Measured on the configured layers depth 2 is
  // as good as it gets (depth 4 costs registers and gains nothing).
  const int taps = a.kh * a.kw > 1 ? a.kh * a.kw : 1;
  a.k_real = taps * a.units_pad;   // kh x kw: units_pad is the ic2 real units of a tap
  a.k_units = up(a.k_real, k.kc);
  a.ic2_magic = div_magic(a.ic2);
  a.kw_magic = div_magic(a.kw > 0 ? a.kw : 1);
  const int nchunks = a.k_units / k.kc;
  int dl = 1;
  if (taps > 1 && (taps > 64 || nbatch != 1)) return hipErrorInvalidValue;
  const int fmt = taps > 1 ? (a.in_nhwc ? 4 : (a.ic2 % k.kc == 0 ? 2 : 3)) : (a.in_nhwc ? 1 : 0);
  while (dl > 0 && (nchunks % (1 << dl) != 0 || !k.kernel[fmt][dl])) --dl;
  return plan_launch(plan, k.kernel[fmt][dl], grid, dim3(kBlock), 0, a, s);
}

}  // namespace ehip
