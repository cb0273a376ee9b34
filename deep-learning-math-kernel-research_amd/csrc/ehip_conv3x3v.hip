// Direct 3x3 stride-1 u8 x s8 -> s32 convolution on gfx950 matrix cores as an implicit GEMM
// (K = 9 taps x IC) over "virtual rows", requantization epilogue fused.
//
// Replaces elx_int8_conv_direct_t::__execute_c160 + conv_c160
// (src/elx_int8_conv_direct_xopt.hpp:20-110, src/elx_int8_conv_direct.cpp:502-571) and the 3x3
// micro-kernel with its epilogue (src/kernel/elk_u8s8_conv.hxx:190-252,679-901).
//
// Virtual rows.  An image is addressed as if every row were VW = ow + 2 cells wide (the input row
// with its left/right frame): virtual cell v = r * VW + c.  Output pixel v then reads, for tap
// (kh, kw), input cell v + kh * VW + kw -- one constant offset per tap for ANY run of consecutive
// virtual pixels, whatever its alignment to the image rows.  So a workgroup takes P_T consecutive
// virtual pixels (a multiple of the 32-pixel MFMA tile, not of the row width), stages the
// P_T + 2 * VW + 2 input cells they touch for ALL input channels into LDS once, and all nine taps of
// all channel pairs read that one staged run at shifted positions.  Two of every VW virtual pixels
// are the frame columns: they are computed and not stored.
//
// Frame cells hold the u8 value 0: after the u8 -> s8 remap (top bit flipped) a zero activation is
// -128, whose product with a weight is cancelled exactly by the 128 * sum(weights) the accumulators
// start from, so skipped border taps of the reference and zero taps here give the same s32.
//
// Stride 2 (template S = 2): the staged input of a unit is de-interleaved into four phase planes,
// plane (pr, pc)[r][c] = in[2 r + pr - pad_t][2 c + pc - pad_l], each addressed by virtual rows of VW = ow + 1
// cells.  Tap (kh, kw) of output pixel v then reads plane (kh & 1, kw & 1) at v + (kh >> 1) * VW + (kw >> 1):
// again one constant offset per tap, so the K loop is the stride-1 loop with another offset table, and only the
// staging plan (which input cell goes where) differs.  One of every VW virtual pixels is a frame column.
//
// MFMA mapping as in the 1x1 kernel (v_mfma_i32_32x32x32_i8; A = weights in packed row order,
// B = pixels, a lane's D = 16 consecutive output channels of one pixel).  A wave owns TM x TN tiles of 32 x 32; its
// weight operands (9 taps x TM) live in registers and every slot is refilled with the next channel
// pair's operand right after its last use, i.e. nine taps ahead; pixel operands come from LDS one
// tap ahead.  Two workgroups share a CU.
#include <type_traits>

#include "ehip_internal.hpp"

// Development aid (compile with -DEHIP_TRACE): lane 0 of every wave records the shader clock at
// phase boundaries into Conv3x3Args::trace.
#ifdef EHIP_TRACE
#define TRACE_POINT(i)                                                                             \
  do {                                                                                             \
    if (a.trace && lane == 0) a.trace[((size_t)tile_id * 4 + wave) * 16 + (i)] = wall_clock64(); \
  } while (0)
#else
#define TRACE_POINT(i) do { } while (0)
#endif

namespace ehip {

// PAIRS > 0: the layer has exactly PAIRS pairs of 16-channel units and they are staged in one fill; the
// whole K loop is then straight-line code.  The weight operands are requested nine taps ahead of their
// use; inside a loop the compiler waits for ALL outstanding loads at the loop's head (its counter model
// does not survive the back edge), which exposes a full trip to L2 once per pair.  Unrolled, every wait
// names exactly the load it needs.
//
// SP ("strided pixels"): lane l32 of pixel tile nt owns virtual pixel TN * l32 + nt of the wave's run
// instead of 32 * nt + l32.  The pixel operand of tap (kh, kw) and tile nt is then the staged run read
// at offset kh * VW + (nt + kw) with a lane stride of TN cells -- it depends on nt + kw only, so one
// kernel row needs TN + 2 operand reads for its 3 * TN pixel operands (18 instead of 36 per channel
// pair at TN = 4), and they are requested a whole kernel row (3 * TM * TN MFMAs) ahead of their use.
// The staged cells of a unit are stored by residue: cell c at (c % TN) * R + c / TN, which makes the
// strided read a read of consecutive 16-byte slots; R is chosen so that neighbouring cells written by
// neighbouring threads land in different banks.
constexpr int conv3x3v_unit_stride(int cells, int tn, bool sp)
{
  if (!sp || tn == 1) return cells;
  int r = (cells + tn - 1) / tn;
  const int want = tn == 4 ? 2 : 4;   // R * 16 bytes = 32 (TN 4) or 64 (TN 2) modulo 128
  while (r % 8 != want) ++r;
  return r * tn;
}

template <int WM, int WN, int TM, int TN, int CT, int NPASS, int PAIRS, bool SP, bool SL, int S>
__device__ __forceinline__ void conv3x3v_body(const Conv3x3Args &a)
{
  static_assert(!SL || (PAIRS > 0 && !SP && TM == 1 && TN == 4), "split last pair: straight-line form, 32 channels x 4 tiles");
  static_assert(S == 1 || (S == 2 && !SP && (CT * NPASS) % 4 == 0), "stride 2: four phase planes per staged unit");
  constexpr int PS = CT * NPASS / 4;   // stride 2: staged cells per phase plane
  constexpr int OC_T = WM * TM * 32;
  constexpr int P_T = WN * TN * 32;
  constexpr int STRIDE = conv3x3v_unit_stride(CT * NPASS, TN, SP);   // LDS cells per unit
  constexpr int RSP = STRIDE / TN;
  static_assert(!SP || TN == 2 || TN == 4, "strided pixels: two or four pixel tiles per wave");
  // where staged cell c of a unit lives
  auto slot = [](int c) { return SP ? (c % TN) * RSP + c / TN : c; };
  constexpr int G = kBlock / CT;       // thread groups that split the units of a fill
  static_assert(WM * WN == 4, "four waves per workgroup");
  static_assert(kBlock % CT == 0, "cells per pass");
  extern __shared__ v4i lds[];         // [chunk_units][STRIDE]
#ifdef EHIP_TRACE
  const long long t_entry = wall_clock64();
#endif

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform: what depends on it stays scalar
  const int l32 = lane & 31;
  const int lh = lane >> 5;
  // Workgroups go round the eight XCDs (block b runs on XCD b % 8), each XCD with an L2 of its own.
  // Tiles are numbered pixel tile first, then channel tile, then image, and XCD x takes the x-th
  // eighth of that sequence: neighbouring pixel tiles share two rows of input, the channel tiles of an
  // image share all of it, and what one of them has pulled into the XCD's L2 the others find there
  // instead of fetching it from HBM again through another XCD.
  const int tile_id = (blockIdx.x & 7) * a.tiles_per_xcd + (blockIdx.x >> 3);
  if (tile_id >= a.tiles) return;   // whole workgroup
  const int n = tile_id / (a.gx * a.gy);
  const int txy = tile_id - n * (a.gx * a.gy);
  const int ty = txy / a.gx;
  const int v0 = (txy - ty * a.gx) * P_T;
  const int oc0 = ty * OC_T;
  const int mw0 = (wave % WM) * TM * 32;
  const int pw0 = (wave / WM) * TN * 32;
  const int oc_real = a.oc2 * 16;
  const int VW = a.vw;
  const int ohw = a.oh * a.ow;
  const long long plane = (long long)a.ih * a.iw * 16;
  const uint8_t *inb = a.in + (long long)n * a.ic2 * plane;
  TRACE_POINT(0);
#ifdef EHIP_TRACE
  if (a.trace && lane == 0) {   // wall clock at the wave's first instruction and once the arguments are in
    a.trace[((size_t)tile_id * 4 + wave) * 16 + 0] = t_entry;
    a.trace[((size_t)tile_id * 4 + wave) * 16 + 1] = wall_clock64();
  }
#endif

  // ---- staging plan: the same cells for every fill ------------------------------------------
  const int ug = tid / CT;
  int goff[NPASS];
  bool gin[NPASS];
#pragma unroll
  for (int p = 0; p < NPASS; ++p) {
    int ih, iw;
    if (S == 2) {
      const int cell = tid % CT + p * CT;   // plane q = cell / PS, cell j of it
      const int q = cell / PS, v = v0 + cell - q * PS;
      const int r = fastdiv(v, VW, a.vw_magic);
      const int c = v - r * VW;
      ih = 2 * r + (q >> 1) - a.pad_t;
      iw = 2 * c + (q & 1) - a.pad_l;
    } else {
      const int v = v0 + tid % CT + p * CT;
      const int r = fastdiv(v, VW, a.vw_magic);
      const int c = v - r * VW;
      ih = r - a.pad_t;
      iw = c - a.pad_l;
    }
    gin[p] = ih >= 0 && ih < a.ih && iw >= 0 && iw < a.iw;
    goff[p] = gin[p] ? (ih * a.iw + iw) * 16 : 0;
  }

  // ---- weights [9][units_pad][ocpp][16]: lane = packed row l32 of unit 2 * pair + lh ---------
  const int8_t *wb = a.w + ((long long)lh * a.ocpp + oc0 + mw0 + l32) * 16;
  const long long w_unit = (long long)a.ocpp * 16;
  const long long w_tap = (long long)a.units_pad * w_unit;
  v4i a_reg[9][TM];
  auto load_a = [&](int tap, int pair) {
    const int8_t *p = wb + tap * w_tap + (long long)(2 * pair) * w_unit;
#pragma unroll
    for (int mt = 0; mt < TM; ++mt) a_reg[tap][mt] = *reinterpret_cast<const v4i *>(p + mt * 512);
  };

  // All global loads are unconditional (clamped indices, unwanted values replaced afterwards).
  // `first`: the weight operands of pair 0 are requested right behind the first batch of pixel
  // loads -- loads return in order, and the pixels are needed first (LDS store, barrier).
  const int nk = a.chunk_units / G;    // units per thread and pass
  constexpr int SB = 8;                // loads in flight per thread: one round trip for up to 8 units
  auto stage = [&](int chunk, bool first) {
#pragma unroll
    for (int p = 0; p < NPASS; ++p) {
      for (int k0 = 0; k0 < nk; k0 += SB) {
        v4i t[SB];
#pragma unroll
        for (int j = 0; j < SB; ++j) {
          const int k = k0 + j < nk ? k0 + j : nk - 1;
          int u = chunk * a.chunk_units + ug + G * k;
          u = u < a.ic2 ? u : a.ic2 - 1;   // padded units multiply zero weights
          t[j] = *reinterpret_cast<const v4i *>(inb + (long long)u * plane + goff[p]);
        }
        if (first && p == 0 && k0 == 0) {
#pragma unroll
          for (int tap = 0; tap < 9; ++tap) load_a(tap, 0);
        }
#pragma unroll
        for (int j = 0; j < SB; ++j) {
          if (k0 + j < nk) {
            const v4i x = t[j] ^ (int)0x80808080;
            const v4i z = {(int)0x80808080, (int)0x80808080, (int)0x80808080, (int)0x80808080};
            lds[(ug + G * (k0 + j)) * STRIDE + slot(tid % CT + p * CT)] = gin[p] ? x : z;
          }
        }
      }
    }
  };

  // The first fill: nothing else is live yet, so the loads of ALL passes travel together, up to 16
  // per thread -- a workgroup's staging time is the number of round trips, not the number of cells
  // (a 3-pass tile of a 224-wide image: three trips before, one now).
  auto stage_first = [&](auto kb) {
    constexpr int KB = decltype(kb)::value;   // units per thread and round trip
    for (int k0 = 0; k0 < nk; k0 += KB) {
      v4i t[NPASS][KB];
#pragma unroll
      for (int p = 0; p < NPASS; ++p)
#pragma unroll
        for (int j = 0; j < KB; ++j) {
          const int k = k0 + j < nk ? k0 + j : nk - 1;
          int u = ug + G * k;
          u = u < a.ic2 ? u : a.ic2 - 1;   // padded units multiply zero weights
          t[p][j] = *reinterpret_cast<const v4i *>(inb + (long long)u * plane + goff[p]);
        }
      if (k0 == 0) {
#pragma unroll
        for (int tap = 0; tap < 9; ++tap) load_a(tap, 0);
      }
#pragma unroll
      for (int p = 0; p < NPASS; ++p)
#pragma unroll
        for (int j = 0; j < KB; ++j) {
          if (k0 + j < nk) {
            const v4i x = t[p][j] ^ (int)0x80808080;
            const v4i z = {(int)0x80808080, (int)0x80808080, (int)0x80808080, (int)0x80808080};
            lds[(ug + G * (k0 + j)) * STRIDE + slot(tid % CT + p * CT)] = gin[p] ? x : z;
          }
        }
    }
  };

  v16i acc[TM][TN];
  // one channel pair (32 input channels) x nine taps; `last` = nothing left to prefetch
  // Issue order matters more than bandwidth here: a wave issues in order, an MFMA occupies the matrix
  // pipe for 32 clocks, and an LDS read or a global load takes the wave's issue slot for several clocks.
  // Four reads issued in a row between two groups of MFMAs leave the pipe idle behind them (measured:
  // 46 instead of 32 clocks per MFMA); ONE memory instruction behind EACH MFMA hides in its shadow
  // (34 clocks).  So every MFMA is followed by at most one pixel-operand read for the next tap, and the
  // tap's last MFMA by the weight request for the next channel pair; sched_barrier pins that order.
  v4i bq[2][TN];
  auto read_b = [&](int par, int pl, int tap, int nt) {
    const v4i *tile = lds + (2 * pl + lh) * STRIDE + pw0 + l32;
    const int kh = tap / 3, kw = tap % 3;
    bq[par][nt] = tile[nt * 32 + (S == 2 ? ((kh & 1) * 2 + (kw & 1)) * PS + (kh >> 1) * VW + (kw >> 1) : kh * VW + kw)];
  };
  // one tap of one channel pair out of operand buffer par; next_pl >= 0: the operands of (next_pl,
  // next_tap) are read into the other buffer on the way
  auto tap_mfmas = [&](int par, int tap, int pair, bool last, int next_pl, int next_tap) {
#pragma unroll
    for (int mt = 0; mt < TM; ++mt)
#pragma unroll
      for (int nt = 0; nt < TN; ++nt) {
        acc[mt][nt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a_reg[tap][mt], bq[par][nt], acc[mt][nt], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        if (mt == 0 && next_pl >= 0) read_b(par ^ 1, next_pl, next_tap, nt);
        if (mt == TM - 1 && nt == TN - 1 && !last) load_a(tap, pair + 1);
        __builtin_amdgcn_sched_barrier(0);
      }
  };
  // loop form: the operands of a pair's first tap are read at its start
  auto pair_taps = [&](int pl, int pair, bool last) {
#pragma unroll
    for (int nt = 0; nt < TN; ++nt) read_b(0, pl, 0, nt);
#pragma unroll
    for (int tap = 0; tap < 9; ++tap) tap_mfmas(tap & 1, tap, pair, last, tap < 8 ? pl : -1, tap + 1);
  };

  // strided pixels: LDS slot offsets of the TN + 2 operands of each kernel row (wave-uniform)
  int soff[3][TN + 2];
  if (SP) {
#pragma unroll
    for (int kh = 0; kh < 3; ++kh)
#pragma unroll
      for (int o = 0; o < TN + 2; ++o) {
        const int b = kh * VW + o;   // pw0 is a multiple of TN
        soff[kh][o] = (b % TN) * RSP + b / TN + pw0 / TN;
      }
  }
  v4i q[2][TN + 2];
  // operands of kernel row kh of the pair staged at pl, into buffer par
  auto load_q = [&](int par, int pl, int kh) {
    const v4i *ub = lds + (2 * pl + lh) * STRIDE + l32;
#pragma unroll
    for (int o = 0; o < TN + 2; ++o) q[par][o] = ub[soff[kh][o]];
  };
  // one kernel row of one channel pair: 3 taps x TM x TN MFMAs out of buffer par; next_pl >= 0: the
  // TN + 2 operands of row (next_pl, next_kh) are read into the other buffer, one behind each MFMA
  auto row_taps = [&](int par, int kh, int pair, bool last, int next_pl, int next_kh) {
    int issued = 0;
#pragma unroll
    for (int kw = 0; kw < 3; ++kw) {
      const int tap = kh * 3 + kw;
#pragma unroll
      for (int mt = 0; mt < TM; ++mt)
#pragma unroll
        for (int nt = 0; nt < TN; ++nt) {
          acc[mt][nt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a_reg[tap][mt], q[par][nt + kw], acc[mt][nt], 0, 0, 0);
          __builtin_amdgcn_sched_barrier(0);
          if (next_pl >= 0 && issued < TN + 2) {
            const v4i *ub = lds + (2 * next_pl + lh) * STRIDE + l32;
            q[par ^ 1][issued] = ub[soff[next_kh][issued]];
            ++issued;
          }
          if (mt == TM - 1 && nt == TN - 1 && !last) load_a(tap, pair + 1);
          __builtin_amdgcn_sched_barrier(0);
        }
    }
  };
  // generic loop form: the operands of a pair's first row are requested at its start
  auto pair_taps_sp = [&](int pl, int pair, bool last) {
    load_q(0, pl, 0);
#pragma unroll
    for (int kh = 0; kh < 3; ++kh) row_taps(kh & 1, kh, pair, last, kh < 2 ? pl : -1, kh + 1);
  };

  const int ppc = a.chunk_units / 2;
  const int nchunks = a.units_pad / a.chunk_units;
  const long long cidx = oc0 + mw0 + 16 * lh;   // the lane's 16 channels of tile 0
  OcConsts k0;
  // The accumulators start from the compensation 128 * sum(weights) of their channel instead of zero:
  // it is requested before the staging loads and costs the epilogue nothing.
#pragma unroll
  for (int mt = 0; mt < TM; ++mt) {
    v4i c4[4];
#pragma unroll
    for (int qq = 0; qq < 4; ++qq) c4[qq] = *reinterpret_cast<const v4i *>(a.ep.comp + cidx + 32 * mt + 4 * qq);
#pragma unroll
    for (int nt = 0; nt < TN; ++nt)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[mt][nt][v] = c4[v >> 2][v & 3];
  }
  // Lean epilogue (a.lean, decided by the launcher): u8 / s8 output, ReLU with bounds 0 <= lo <= hi, no
  // sum -- the case of every direct 3x3 layer of the tuned networks.  Scale and shift of the lane's
  // channels travel during the last channel pair; a value then costs a convert, a multiply-add, a
  // clamp (none when the bounds are exactly the u8 code range) and a byte pack.
  LeanConsts lk[TM];
  auto load_epilogue_consts = [&]() {
    if (a.lean) {
#pragma unroll
      for (int mt = 0; mt < TM; ++mt) load_lean_consts(lk[mt], a.ep, cidx + 32 * mt);
    } else {
      load_consts(k0, a.ep, cidx);
    }
  };
  // as few loads per trip as cover the fill (unused slots repeat the last unit's load), at most 16
  constexpr int KBMAX = NPASS == 1 ? 16 : (NPASS == 2 ? 8 : 4);
  if (nk <= 2) stage_first(std::integral_constant<int, 2>());
  else if (nk <= 4 || KBMAX == 4) stage_first(std::integral_constant<int, 4>());
  else if (nk <= 8 || KBMAX == 8) stage_first(std::integral_constant<int, (KBMAX < 8 ? KBMAX : 8)>());
  else stage_first(std::integral_constant<int, KBMAX>());
  TRACE_POINT(2);
  __syncthreads();
  TRACE_POINT(3);
  if (PAIRS > 0 && SP) {
    // straight line over the 3 * PAIRS kernel rows, each one's operands requested a row ahead
    load_q(0, 0, 0);
#pragma unroll
    for (int st = 0; st < 3 * PAIRS; ++st) {
      const int pl = st / 3, kh = st % 3;
      if (st == 3 * PAIRS - 3) load_epilogue_consts();
      row_taps(st & 1, kh, pl, pl == PAIRS - 1, st + 1 < 3 * PAIRS ? (st + 1) / 3 : -1, (st + 1) % 3);
    }
  } else if (PAIRS > 0) {
    // straight line over the 9 * PAIRS taps, each one's pixel operands read during the tap before
#pragma unroll
    for (int nt = 0; nt < TN; ++nt) read_b(0, 0, 0, nt);
    constexpr int LAST0 = 9 * (PAIRS - 1);   // first tap of the last channel pair
#pragma unroll
    for (int st = 0; st < LAST0; ++st) tap_mfmas(st & 1, st % 9, st / 9, false, (st + 1) / 9, (st + 1) % 9);
    load_epilogue_consts();
    // Split last pair (a wave of 32 channels x four pixel tiles, lean epilogue without the sum): with one
    // workgroup per CU nothing hides the epilogue -- a convert, a multiply-add and a byte pack per value, a
    // sixth of the kernel's time for 128 input channels.  So the last channel pair is multiplied tile pair by
    // tile pair instead of tap by tap: tiles 0 and 1 through all nine taps (their accumulators alternate, so
    // no MFMA waits for the one before), then tiles 2 and 3, and behind each of THEIR eighteen MFMAs goes a
    // piece of the epilogue of tiles 0 and 1.  All nine weight operands of the last pair are in registers by then.
    // (SL: a kernel of its own, launched only for such epilogues.)
    if constexpr (SL) {
      constexpr int P0 = LAST0 & 1;   // operand buffer of the last pair's first tap
      uint8_t *outb = static_cast<uint8_t *>(a.out) + ((size_t)n * a.oc2 + ((oc0 + mw0) >> 4)) * ohw * 16;
      uint8_t *cell[TN];
      bool pv[TN];
      auto locate = [&](int nt) {
        const int v = v0 + pw0 + nt * 32 + l32;
        const int r = fastdiv(v, VW, a.vw_magic);
        const int c = v - r * VW;
        pv[nt] = r < a.oh && c < a.ow && (int)cidx < oc_real;
        cell[nt] = outb + (unsigned)(lh * ohw + (pv[nt] ? r * a.ow + c : 0)) * 16u;
      };
      const bool s8 = a.ep.out_type == EHIP_S8;
      const float hi = s8 ? __builtin_fminf(a.ep.hi, 127.0f) : a.ep.hi;
      auto last_pair = [&](auto clampc) {
        constexpr bool CLAMP = decltype(clampc)::value;
        auto pack = [&](int tile, int q) -> int {   // four values of tile `tile`: arithmetic of lean_store_typed
          const float sc[4] = {lk[0].sc[q].x, lk[0].sc[q].y, lk[0].sc[q].z, lk[0].sc[q].w};
          const float sh[4] = {lk[0].sh[q].x, lk[0].sh[q].y, lk[0].sh[q].z, lk[0].sh[q].w};
          unsigned pk = 0;
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            float f = __builtin_fmaf((float)acc[0][tile][4 * q + j], sc[j], sh[j]);
            if (CLAMP) f = __builtin_amdgcn_fmed3f(f, a.ep.lo, hi);
            pk = __builtin_amdgcn_cvt_pk_u8_f32(f, j, pk);
          }
          return (int)pk;
        };
        // tiles 0 and 1; where they go is worked out behind the first MFMAs
#pragma unroll
        for (int tap = 0; tap < 9; ++tap)
#pragma unroll
          for (int nt = 0; nt < 2; ++nt) {
            const int par = (P0 + tap) & 1;
            acc[0][nt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a_reg[tap][0], bq[par][nt], acc[0][nt], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            if (tap < 8) read_b(par ^ 1, PAIRS - 1, tap + 1, nt);
            if (2 * tap + nt < TN) locate(2 * tap + nt);
            __builtin_amdgcn_sched_barrier(0);
          }
        // tiles 2 and 3, with the epilogue of tiles 0 and 1 in their shadow
        v4i outv[2];
#pragma unroll
        for (int tap = 0; tap < 9; ++tap)
#pragma unroll
          for (int nt = 2; nt < 4; ++nt) {
            const int par = (P0 + tap) & 1;
            acc[0][nt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a_reg[tap][0], bq[par][nt], acc[0][nt], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            if (tap < 8) read_b(par ^ 1, PAIRS - 1, tap + 1, nt);
            const int k = 2 * tap + (nt - 2);   // 0 .. 17
            if (k < 8) outv[k >> 2][k & 3] = pack(k >> 2, k & 3);
            if (k == 8 && pv[0]) store_out16<false>(cell[0], outv[0]);
            if (k == 9 && pv[1]) store_out16<false>(cell[1], outv[1]);
            __builtin_amdgcn_sched_barrier(0);
          }
        TRACE_POINT(5);
#pragma unroll
        for (int tile = 2; tile < 4; ++tile) {
          v4i o;
#pragma unroll
          for (int q = 0; q < 4; ++q) o[q] = pack(tile, q);
          if (pv[tile]) store_out16<false>(cell[tile], o);
        }
      };
      if (a.lean & 2) last_pair(std::false_type());
      else last_pair(std::true_type());
      TRACE_POINT(15);
      return;
    } else {
#pragma unroll
      for (int st = LAST0; st < 9 * PAIRS; ++st)
        tap_mfmas(st & 1, st % 9, PAIRS - 1, true, st + 1 < 9 * PAIRS ? PAIRS - 1 : -1, (st + 1) % 9);
    }
  } else
  for (int chunk = 0; chunk < nchunks; ++chunk) {
    if (chunk) {
      __syncthreads();
      stage(chunk, false);
      __syncthreads();
    }
    const int npl = chunk + 1 < nchunks ? ppc : ppc - 1;
    for (int pl = 0; pl < npl; ++pl) {
      if (SP) pair_taps_sp(pl, chunk * ppc + pl, false);
      else pair_taps(pl, chunk * ppc + pl, false);
    }
    TRACE_POINT(4);
    if (chunk + 1 == nchunks) {
      // the epilogue's per-channel constants travel while the last pair is multiplied
      load_epilogue_consts();
      if (SP) pair_taps_sp(ppc - 1, chunk * ppc + ppc - 1, true);
      else pair_taps(ppc - 1, chunk * ppc + ppc - 1, true);
    }
  }
  TRACE_POINT(5);

  // ---- epilogue ------------------------------------------------------------------------------
  if (a.lean) {
    // the lane's 16 channels are block lh of the wave's first two; everything else about the address is scalar
    uint8_t *outb = static_cast<uint8_t *>(a.out) + ((size_t)n * a.oc2 + ((oc0 + mw0) >> 4)) * ohw * 16;
    uint8_t *cell[TN];
    bool pv[TN];
#pragma unroll
    for (int nt = 0; nt < TN; ++nt) {
      const int v = SP ? v0 + pw0 + TN * l32 + nt : v0 + pw0 + nt * 32 + l32;
      const int r = fastdiv(v, VW, a.vw_magic);
      const int c = v - r * VW;
      pv[nt] = r < a.oh && c < a.ow;
      cell[nt] = outb + (unsigned)(lh * ohw + (pv[nt] ? r * a.ow + c : 0)) * 16u;
    }
    lean_store<TM, TN>(a.lean, a.ep, acc, lk, cell, pv, (int)cidx, oc_real, (size_t)2 * ohw * 16);
    TRACE_POINT(15);
    return;
  }
  size_t pix[TN];
  bool pvalid[TN];
#pragma unroll
  for (int nt = 0; nt < TN; ++nt) {
    const int v = SP ? v0 + pw0 + TN * l32 + nt : v0 + pw0 + nt * 32 + l32;
    const int r = fastdiv(v, VW, a.vw_magic);
    const int c = v - r * VW;
    pvalid[nt] = r < a.oh && c < a.ow;
    pix[nt] = ((size_t)n * a.oc2 * ohw + (pvalid[nt] ? r * a.ow + c : 0)) * 16;
  }
  TRACE_POINT(14);
  const size_t pixT[TN][2] = {};
  const bool validT[TN][2] = {};
  epilogue_wave<TM, TN, false, true>(a.ep, acc, k0, cidx, (int)cidx, pix, pvalid, oc_real, (size_t)ohw * 16, a.out, nullptr,
                                     pixT, validT);
  TRACE_POINT(15);
}

// The kernel proper.  What the first instructions of a wave need -- the input pointer and the geometry the
// staging addresses are made of -- is passed as leading scalar arguments, which the dispatcher preloads into
// scalar registers with the wave (the file is compiled with -amdgpu-kernarg-preload-count=16): the wave
// starts computing addresses at once instead of after a round trip to the kernel-argument memory (~0.5 us,
// of a 6 us kernel).  The rest of the argument block is loaded as usual while the staging loads fly.
#define EHIP_CONV3X3V_HEAD                                                                                            \
  const uint8_t *in, int ih, int iw, int oh, int ow, int pad_t, int pad_l, int ic2, int chunk_units, int vw,         \
      unsigned vw_magic, int gx, int gy, int tiles, int tiles_per_xcd
template <int WM, int WN, int TM, int TN, int CT, int NPASS, int PAIRS = 0, bool SP = false, bool SL = false, int S = 1>
__global__ __launch_bounds__(kBlock, 2) void k_conv3x3v_u8s8(EHIP_CONV3X3V_HEAD, Conv3x3Args rest)
{
  Conv3x3Args a = rest;
  a.in = in; a.ih = ih; a.iw = iw; a.oh = oh; a.ow = ow; a.pad_t = pad_t; a.pad_l = pad_l; a.ic2 = ic2;
  a.chunk_units = chunk_units; a.vw = vw; a.vw_magic = vw_magic; a.gx = gx; a.gy = gy; a.tiles = tiles;
  a.tiles_per_xcd = tiles_per_xcd;
  conv3x3v_body<WM, WN, TM, TN, CT, NPASS, PAIRS, SP, SL, S>(a);
}

namespace {
typedef void (*conv3x3v_kernel_t)(EHIP_CONV3X3V_HEAD, Conv3x3Args);
inline hipError_t conv3x3v_enqueue(conv3x3v_kernel_t kernel, dim3 grid, unsigned lds, const Conv3x3Args &a, hipStream_t s)
{
  hipLaunchKernelGGL(kernel, grid, dim3(kBlock), lds, s, a.in, a.ih, a.iw, a.oh, a.ow, a.pad_t, a.pad_l, a.ic2, a.chunk_units,
                     a.vw, a.vw_magic, a.gx, a.gy, a.tiles, a.tiles_per_xcd, a);
  return hipGetLastError();
}
struct Variant {
  const char *name;
  int oc_t, p_t, cells;   // cells: staged cells per unit a tile may span
  int ustride;            // LDS cells between units
  conv3x3v_kernel_t kernel;
  conv3x3v_kernel_t unrolled[3];   // straight-line K loop for layers of exactly 2, 4, 8 unit pairs, or null
  conv3x3v_kernel_t split[3];      // the same with the last pair split (lean epilogue without the sum), or null
  int stride;                      // 1, or 2: the staged unit is four phase planes of cells / 4 cells each
};
#define V(WM, WN, TM, TN, CT, NPASS)                                                              \
  { "k_conv3x3v_u8s8<" #WM "," #WN "," #TM "," #TN "," #CT "," #NPASS ">", WM * TM * 32, WN * TN * 32, \
    CT * NPASS, CT * NPASS, k_conv3x3v_u8s8<WM, WN, TM, TN, CT, NPASS>, {nullptr, nullptr, nullptr}, {nullptr, nullptr, nullptr}, 1 }
#define VU(WM, WN, TM, TN, CT, NPASS)                                                             \
  { "k_conv3x3v_u8s8<" #WM "," #WN "," #TM "," #TN "," #CT "," #NPASS ">", WM * TM * 32, WN * TN * 32, \
    CT * NPASS, CT * NPASS, k_conv3x3v_u8s8<WM, WN, TM, TN, CT, NPASS>,                            \
    {k_conv3x3v_u8s8<WM, WN, TM, TN, CT, NPASS, 2>, k_conv3x3v_u8s8<WM, WN, TM, TN, CT, NPASS, 4>,  \
     k_conv3x3v_u8s8<WM, WN, TM, TN, CT, NPASS, 8>}, {nullptr, nullptr, nullptr}, 1 }
#define VU2(WM, WN, TM, TN, CT, NPASS) /* straight-line form for two unit pairs only (64 input channels) */ \
  { "k_conv3x3v_u8s8<" #WM "," #WN "," #TM "," #TN "," #CT "," #NPASS ">", WM * TM * 32, WN * TN * 32, \
    CT * NPASS, CT * NPASS, k_conv3x3v_u8s8<WM, WN, TM, TN, CT, NPASS>,                            \
    {k_conv3x3v_u8s8<WM, WN, TM, TN, CT, NPASS, 2>, nullptr, nullptr}, {nullptr, nullptr, nullptr}, 1 }
#define VK(WM, WN, TM, TN, CT, NPASS)                                                             \
  { "k_conv3x3v_u8s8<" #WM "," #WN "," #TM "," #TN "," #CT "," #NPASS ">", WM * TM * 32, WN * TN * 32, \
    CT * NPASS, CT * NPASS, k_conv3x3v_u8s8<WM, WN, TM, TN, CT, NPASS>,                            \
    {k_conv3x3v_u8s8<WM, WN, TM, TN, CT, NPASS, 2>, k_conv3x3v_u8s8<WM, WN, TM, TN, CT, NPASS, 4>,  \
     k_conv3x3v_u8s8<WM, WN, TM, TN, CT, NPASS, 8>},                                               \
    {k_conv3x3v_u8s8<WM, WN, TM, TN, CT, NPASS, 2, false, true>, k_conv3x3v_u8s8<WM, WN, TM, TN, CT, NPASS, 4, false, true>, \
     k_conv3x3v_u8s8<WM, WN, TM, TN, CT, NPASS, 8, false, true>}, 1 }
#define V2(WM, WN, TM, TN, CT, NPASS) /* stride 2; straight-line forms for two and four unit pairs */ \
  { "k_conv3x3v_u8s8<" #WM "," #WN "," #TM "," #TN "," #CT "," #NPASS ",s2>", WM * TM * 32, WN * TN * 32, \
    CT * NPASS, CT * NPASS, k_conv3x3v_u8s8<WM, WN, TM, TN, CT, NPASS, 0, false, false, 2>,       \
    {k_conv3x3v_u8s8<WM, WN, TM, TN, CT, NPASS, 2, false, false, 2>, k_conv3x3v_u8s8<WM, WN, TM, TN, CT, NPASS, 4, false, false, 2>, \
     nullptr}, {nullptr, nullptr, nullptr}, 2 }
#define VS(WM, WN, TM, TN, CT, NPASS)                                                             \
  { "k_conv3x3v_u8s8<" #WM "," #WN "," #TM "," #TN "," #CT "," #NPASS ",sp>", WM * TM * 32, WN * TN * 32, \
    CT * NPASS, conv3x3v_unit_stride(CT * NPASS, TN, true), k_conv3x3v_u8s8<WM, WN, TM, TN, CT, NPASS, 0, true>, \
    {k_conv3x3v_u8s8<WM, WN, TM, TN, CT, NPASS, 2, true>, k_conv3x3v_u8s8<WM, WN, TM, TN, CT, NPASS, 4, true>, \
     k_conv3x3v_u8s8<WM, WN, TM, TN, CT, NPASS, 8, true>}, {nullptr, nullptr, nullptr}, 1 }
const Variant kVariants[] = {
    V(2, 2, 2, 1, 128, 1),  // 0: 128 oc x  64 px, rows up to  31 cells
    V(2, 2, 2, 1, 256, 1),  // 1: 128 oc x  64 px, rows up to  95 cells
    VU(2, 2, 2, 2, 256, 1), // 2: 128 oc x 128 px, rows up to  63 cells
    V(2, 2, 2, 2, 256, 3),  // 3: 128 oc x 128 px, rows up to 319 cells
    VU(1, 4, 2, 1, 256, 1), // 4:  64 oc x 128 px, rows up to  63 cells
    V(1, 4, 2, 1, 256, 3),  // 5:  64 oc x 128 px, rows up to 319 cells
    V(1, 4, 1, 1, 256, 1),  // 6:  32 oc x 128 px, rows up to  63 cells
    V(1, 4, 1, 1, 256, 3),  // 7:  32 oc x 128 px, rows up to 319 cells
    VU(4, 1, 1, 1, 128, 1), // 8: 128 oc x  32 px, rows up to  47 cells
    VK(4, 1, 1, 4, 256, 1), // 9: 128 oc x 128 px, rows up to  63 cells, every wave all pixels
    VU(4, 1, 1, 2, 128, 1), // 10: 128 oc x 64 px, rows up to  31 cells, every wave all pixels
    V(1, 4, 2, 2, 256, 3),  // 11:  64 oc x 256 px, rows up to 255 cells
    VU2(2, 2, 1, 4, 256, 3), // 12:  64 oc x 256 px, rows up to 255 cells, a wave = 32 oc x 128 px
    VK(4, 1, 1, 4, 256, 2), // 13: 128 oc x 128 px, rows up to 191 cells, every wave all pixels
    V(4, 1, 1, 4, 256, 4),  // 14: 128 oc x 128 px, rows up to 447 cells, every wave all pixels
    VS(4, 1, 1, 4, 256, 1), // 15: as 9, strided pixels
    VS(4, 1, 1, 2, 128, 1), // 16: as 10, strided pixels
    VS(2, 2, 2, 2, 256, 1), // 17: as 2, strided pixels
    VS(4, 1, 1, 4, 256, 2), // 18: as 13, strided pixels
    VS(2, 2, 2, 4, 256, 2), // 19: 128 oc x 256 px, rows up to 127 cells, a wave = 64 oc x 128 px, strided pixels
    V2(4, 1, 1, 2, 128, 3), // 20: stride 2, 128 oc x  64 px, output rows up to 29 pixels, every wave all pixels
    V2(4, 1, 1, 4, 128, 5), // 21: stride 2, 128 oc x 128 px, output rows up to 29 pixels, every wave all pixels
    V2(4, 1, 1, 2, 256, 2), // 22: stride 2, 128 oc x  64 px, output rows up to 61 pixels
    V2(1, 4, 2, 1, 128, 5), // 23: stride 2,  64 oc x 128 px, output rows up to 29 pixels
};
#undef V
#undef VU
#undef VK
#undef VU2
#undef VS
#undef V2
constexpr int kNumVariants = sizeof(kVariants) / sizeof(kVariants[0]);
constexpr int kLdsBudget = 64 * 1024;
}  // namespace

const char *conv3x3v_variant_name(int v) { return kVariants[v].name; }
int conv3x3v_num_variants() { return kNumVariants; }
bool conv3x3v_fits(int v, int ow, int stride)
{
  if (kVariants[v].stride != stride) return false;
  if (stride == 2) return kVariants[v].p_t + (ow + 1) + 2 <= kVariants[v].cells / 4;   // a phase plane: tile + a row + a cell
  return kVariants[v].p_t + 2 * (ow + 2) + 2 <= kVariants[v].cells;
}

// units of 16 input channels staged per LDS fill: all of them if they fit the budget
int conv3x3v_chunk_units(int v, int ic2)
{
  // (stride 2: four pairs per fill, 48 to 80 KB, so that 128 / 256 / 512 input channels are whole fills)
  if (kVariants[v].stride == 2) return ic2 < 8 ? up(ic2, 2) : 8;
  int cu = (kLdsBudget / (kVariants[v].ustride * 16)) & ~1;
  const int all = up(ic2, 2);
  return cu < all ? cu : all;
}

// -1: no variant fits the row width
int conv3x3v_pick_variant(int n, int oh, int ow, int oc2, int stride)
{
  const char *env = getenv("EHIP_CONV3X3V_VARIANT");
  if (env && env[0]) {
    int v = atoi(env);
    if (v >= 0 && v < kNumVariants && conv3x3v_fits(v, ow, stride)) return v;
    return -1;
  }
  if (stride == 2) {
    // fewest computed pixels first, then the chip's fill
    int best = -1;
    double best_score = -1;
    for (int v = 0; v < kNumVariants; ++v) {
      if (!conv3x3v_fits(v, ow, 2)) continue;
      const Variant &k = kVariants[v];
      const int oc = oc2 * 16;
      if (oc > 64 && k.oc_t < 128) continue;
      const int gx = (oh * (ow + 1) + k.p_t - 1) / k.p_t, gy = (oc + k.oc_t - 1) / k.oc_t;
      const long long wgs = (long long)gx * gy * n;
      const double util = (double)(oh * ow) / ((double)gx * k.p_t) * (double)oc / ((double)gy * k.oc_t);
      const double fill = wgs >= 256 ? 1.0 : (double)wgs / 256.0;
      const double big = (k.p_t >= 128 && wgs >= 440) ? 1.15 : 1.0;   // enough work: amortise the weights (as below)
      const double score = util * fill * big;
      if (score > best_score) { best_score = score; best = v; }
    }
    return best;
  }
  // Measured on MI355X (3x3 128 -> 128 @28x28, N = 32 .. 512): a workgroup's time is the time to
  // pull its weights through the CU's vector-memory path, so tiles whose four waves own disjoint
  // channels (no weight row loaded twice: variants 8-10, 13) win; among those the 64-pixel tile while
  // the grid is small (more workgroups to spread over the chip), the 128-pixel tile once it is not.
  // Wide rows (VGG's 224 and 112) make the halo of 2 virtual rows the larger part of a staged tile:
  // there the 256-pixel tiles (11, 12) and the two-pass 128-channel tile (13) are 1.3-1.8 x faster
  // than the 128-pixel tiles with three passes.
  const int oc = oc2 * 16, vpx = oh * (ow + 2);
  static const double pref[] = {0.80, 0.78, 0.92, 0.90, 1.0, 0.95, 1.0, 0.95, 0.85, 1.12, 0.95, 0.97, 1.14, 0.93, 0.85,
                                0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0};
  int best = -1;
  double best_score = -1;
  for (int pass = 0; pass < 2 && best < 0; ++pass)   // second pass: any channel tile that fits the rows
  for (int v = 0; v < kNumVariants; ++v) {
    if (!conv3x3v_fits(v, ow, 1)) continue;
    const Variant &k = kVariants[v];
    if (pass == 0) {
      if (oc > 64 && k.oc_t < 128) continue;
      // (64 channels: the 128-channel tile whose waves own 32 channels each, half of them idle, is within a
      // few percent of the best 64-channel tile -- 64 -> 64 at 56 x 56, N = 64: 19.1 us against 16.8 us for
      // variant 12 and 19.4 us for variant 4 -- and wins where 256-pixel tiles waste too many pixels)
      if (oc <= 64 && oc > 32 && k.oc_t != 64 && v != 9) continue;
      if (oc <= 32 && k.oc_t != 32) continue;
    }
    const int gx = (vpx + k.p_t - 1) / k.p_t, gy = (oc + k.oc_t - 1) / k.oc_t;
    const long long wgs = (long long)gx * gy * n;
    const double util = (double)(oh * ow) / ((double)gx * k.p_t);
    const double fill = wgs >= 256 ? 1.0 : (double)wgs / 256.0;
    const double big = (k.p_t >= 128 && wgs >= 440) ? 1.15 : 1.0;   // enough work: amortise the weights
    const double score = util * fill * big * pref[v];
    if (score > best_score) { best_score = score; best = v; }
  }
  return best;
}

hipError_t launch_conv3x3v(const Conv3x3Args &a0, int n, int variant, hipStream_t s, LaunchPlan<Conv3x3Args> *plan)
{
  if (plan && plan->valid) {   // everything but the tensors is as on the first launch
    Conv3x3Args local = plan->args;   // a copy: the kept plan is only read (executes from several threads or streams)
    local.in = a0.in;
    local.out = a0.out;
    // (the plan keeps this kernel's pointer under the one-argument type of its slot)
    return conv3x3v_enqueue(reinterpret_cast<conv3x3v_kernel_t>(plan->kernel), plan->grid, plan->lds, local, s);
  }
  const Variant &k = kVariants[variant];
  Conv3x3Args a = a0;
  const size_t lds_bytes = (size_t)a.chunk_units * k.ustride * 16;
  a.gx = (a.oh * a.vw + k.p_t - 1) / k.p_t;
  a.gy = (a.oc2 * 16 + k.oc_t - 1) / k.oc_t;
  const long long tiles = (long long)a.gx * a.gy * n;
  if (tiles >= (1ll << 30)) {
    set_error("direct 3x3: too many tiles");
    return hipErrorInvalidValue;
  }
  a.tiles = (int)tiles;
  a.tiles_per_xcd = (a.tiles + 7) / 8;
  a.lean = lean_mode(a.ep, false);
  dim3 grid(8 * a.tiles_per_xcd, 1, 1);
  conv3x3v_kernel_t kernel = k.kernel;
  if (a.units_pad == a.chunk_units) {   // one fill holds every unit
    const int pairs = a.units_pad / 2;
    const int slot = pairs == 2 ? 0 : (pairs == 4 ? 1 : (pairs == 8 ? 2 : -1));
    const char *env = getenv("EHIP_CONV3X3V_UNROLL");
    if (slot >= 0 && k.unrolled[slot] && !(env && env[0] == '0')) {
      kernel = k.unrolled[slot];
      // (the split form needs 238 registers against 164: two workgroups per CU instead of three, which costs
      // more than the split gains once a CU gets more than two -- C2 at N = 512: 63.7 against 61.1 us; at its
      // own N = 32, one workgroup per CU: 6.12 against 6.54 us)
      const char *sl = getenv("EHIP_CONV3X3V_SPLIT_LAST");
      const bool want = sl && sl[0] ? sl[0] != '0' : a.tiles <= 512;
      if (k.split[slot] && (a.lean & 1) && !(a.lean & 4) && want) kernel = k.split[slot];
    }
  }
  if (lds_bytes > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
    if (e != hipSuccess) return e;
  }
  const hipError_t e = conv3x3v_enqueue(kernel, grid, (unsigned)lds_bytes, a, s);
  if (plan && e == hipSuccess) {   // kept only once the first launch has gone out
    plan->kernel = reinterpret_cast<void (*)(Conv3x3Args)>(kernel);
    plan->grid = grid;
    plan->block = dim3(kBlock);
    plan->lds = (unsigned)lds_bytes;
    plan->args = a;
    plan->valid = true;
  }
  return e;
}

}  // namespace ehip
