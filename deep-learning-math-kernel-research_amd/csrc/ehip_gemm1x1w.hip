// 1x1 u8 x s8 -> s32 convolution on gfx950 matrix cores with the WEIGHTS resident in registers and the
// pixels streamed through LDS: the form for layers of 256 to 1024 input channels in blocked layout whose
// epilogue is the lean one (u8 / s8 output, ReLU, optional in-place sum).
//
// Replaces, for those layers, elx_int8_conv_direct_1x1_t::__execute_a160_s1 / _s2 + gemm_a160_s1 / _s2
// (src/elx_int8_conv_direct_1x1_xopt.hpp:20-195, src/elx_int8_conv_direct_1x1.cpp:357-480) and the u8s8 GEMM
// micro-kernel with its epilogue (src/kernel/elk_u8s8_gemm.hxx:168-406).
//
// A workgroup owns 4 x TM x 32 output channels (TM x 32 per wave, all their weights in registers: at most 128
// registers per lane) and a contiguous run of 32-pixel tiles, which it walks.  The number of runs is chosen so
// that (channel blocks) x (runs) is twice the number of CUs: two workgroups share a CU and fill each other's
// stalls, every CU gets the same share whatever the pixel count, and the bytes a CU pulls from L2 are the weights
// of its channels once plus its own pixels -- the resident-tile kernel pulled the weights once per 64 pixels.
// Tiles arrive by loads that write LDS directly (no registers held while they fly), a few tiles ahead, into a
// ring of stages; the in-place sum's operand comes the same way, so after the prologue a wave issues no load that
// returns into registers.  Per tile there is one barrier, two k-steps before the end of the tile's K loop: by
// then every wave has seen its share of the next tile land, and nobody reads the stage of the tile before any
// more; that stage is refilled over the first k-steps of the next tile, a load per k-step.
// The K loop is straight-line code: TM MFMAs per k-step against one pixel operand, the operand of k-step + 2 read
// from LDS and the u8 -> s8 flip of k-step + 1 behind them.
#include "ehip_internal.hpp"

#ifdef EHIP_TRACE
#define TRACE_POINT(i)                                                                             \
  do {                                                                                             \
    if (a.trace && lane == 0) a.trace[((size_t)blockIdx.x * NW + wave) * 16 + (i)] = wall_clock64(); \
  } while (0)
#else
#define TRACE_POINT(i) do { } while (0)
#endif

namespace ehip {

namespace {

// 16 bytes per lane from global memory straight into LDS: lane i's piece lands at lds_addr + 16 i (lds_addr is
// wave-uniform, a byte address in LDS); the global address is a wave-uniform 64-bit base plus a 32-bit offset per
// lane.  Written as assembly the compiler does not see a memory instruction: it cannot tell which part of LDS such a
// load touches and would make every later LDS read wait for all of them.  The caller waits by count (wait_vm) and
// separates writers from readers with barriers.
__device__ __forceinline__ void dma16(const void *sbase, unsigned voff, unsigned lds_addr)
{
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(lds_addr), "v"(voff), "s"(sbase) : "memory", "m0");
#else
  (void)sbase;
  (void)voff;
  (void)lds_addr;
#endif
}
// at most n of the wave's vector-memory operations still in flight (loads complete in issue order; stores
// count as well, which only makes the wait longer than needed, never shorter)
__device__ __forceinline__ void wait_vm(int n)
{
#if defined(__HIP_DEVICE_COMPILE__)
#define EHIP_W(N) case N: asm volatile("s_waitcnt vmcnt(" #N ")" ::: "memory"); break;
  switch (n) {
    EHIP_W(0) EHIP_W(1) EHIP_W(2) EHIP_W(3) EHIP_W(4) EHIP_W(5) EHIP_W(6) EHIP_W(8) EHIP_W(9) EHIP_W(10) EHIP_W(12) EHIP_W(15)
    EHIP_W(16) EHIP_W(18) EHIP_W(20) EHIP_W(24) EHIP_W(25) EHIP_W(30) EHIP_W(32) EHIP_W(36) EHIP_W(40)
    default: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
  }
#undef EHIP_W
#else
  (void)n;
#endif
}

struct PixInfo {
  unsigned in_off;    // byte offset of the pixel's cell in input unit 0 (the launcher checks that tensors stay below 4 GB)
  unsigned out_off;   // byte offset of the pixel's output cell in channel 0 (blocked: 16-channel block 0)
  bool valid;
};

}  // namespace

// geom = stride_h | stride_w << 8 | dense << 16 | nb << 20 (channel blocks of 4 x TM x 32)
// (the leading arguments are what the first tile's loads, the per-channel constants and the weight loads need: they
// arrive in scalar registers with the wave, while the rest of the argument block is still being fetched;
// owiw = ow | iw << 16; consts = [3][ocpp]: scale, shift, compensation, one allocation)
#define EHIP_WRES_HEAD                                                                                                  \
  const uint8_t *in, const int8_t *w, const float *consts, int p_total, int ohw, unsigned ohw_magic, int ihw, int ocpp, \
      unsigned geom, int nreg, unsigned owiw, unsigned ow_magic
// NW waves per workgroup: four, two workgroups per CU; or eight in one workgroup per CU, which then share ONE copy
// of every pixel tile (1024 input channels, where a wave can only hold the weights of 32 channels: eight waves own
// the 256 channels that four own with fewer input channels)
template <int NKS, int TM, int SUM, int NW>   // SUM: 0 none, 1 the old output is u8, 2 it is s8
__global__ __launch_bounds__(NW * 64, NW == 8 ? 1 : 2) void k_gemm1x1_wres(EHIP_WRES_HEAD, GemmArgs rest)
{
  GemmArgs a = rest;
  a.in = in; a.w = w; a.p_total = p_total; a.ohw = ohw; a.ohw_magic = ohw_magic;
  a.ihw = ihw; a.ic2 = 2 * NKS; a.ocpp = ocpp; a.ow = (int)(owiw & 0xffffu); a.iw = (int)(owiw >> 16); a.ow_magic = ow_magic;
  constexpr int stage_bytes = NKS * 1024 + (SUM ? NW * TM * 1024 : 0);
  a.stride_h = (int)(geom & 0xffu); a.stride_w = (int)((geom >> 8) & 0xffu);
  const bool dense = (geom >> 16) & 1u;
  const int nb = (int)(geom >> 20);
  extern __shared__ v4i lds[];
  constexpr int OCW = TM * 32;   // channels of a wave

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31;
  const int lh = lane >> 5;
  // the channel blocks of one run follow each other on ONE XCD (the first pulls the pixels into that XCD's L2,
  // the others find them there); an XCD takes a contiguous eighth of the runs
  const int xcd = blockIdx.x & 7, seq = blockIdx.x >> 3;
  // (the other order -- a channel block's runs next to each other, the blocks of a run 16 workgroups apart -- measured
  // 14.7 against 13.1 us on the 512 -> 1024 stride-2 layer)
  const int by = seq % nb;
  const int reg = xcd * ((nreg + 7) >> 3) + seq / nb;
  if (reg >= nreg) return;   // whole workgroup
  // runs of whole tiles: the first (ntiles_all % nreg) runs are one tile longer
  const int ntiles_all = (p_total + 31) >> 5;
  const int tq = ntiles_all / nreg, tr = ntiles_all - tq * nreg;
  const int tile0 = reg * tq + (reg < tr ? reg : tr);
  const int ntiles = tq + (reg < tr ? 1 : 0);
  if (ntiles == 0) return;
  const int p0 = tile0 * 32;
  const int ocw = by * (NW * OCW) + wave * OCW;   // the wave's first channel
  const int oc_lane = ocw + 16 * lh;             // the lane's 16 channels of tile 0 (tile mt: + 32 mt)
  const int oc_real = a.oc2 * 16;
  const unsigned lds_base = (unsigned)(size_t)(__attribute__((address_space(3))) void *)lds;
  constexpr int stage_cells = stage_bytes >> 4;
  // The weights fill the vector registers: the per-channel constants (scale, shift, compensation) of the wave's
  // channels live in a wave-private piece of LDS behind the stages, [3][OCW] dwords, channel c of the wave at
  // index c: a lane's four consecutive channels are one 16-byte read, the same for half a wave.
  TRACE_POINT(0);

  auto pix_info = [&](int tt, bool with_out = true) -> PixInfo {
    PixInfo pi;
    const int gp = p0 + 32 * tt + l32;
    pi.valid = gp < a.p_total;
    const int gpc = pi.valid ? gp : a.p_total - 1;
    const int n = a.ohw == a.p_total ? 0 : fastdiv_any(gpc, a.ohw, a.ohw_magic);
    const int r = gpc - n * a.ohw;
    int sp = r;
    if (!dense) {
      const int oh = fastdiv(r, a.ow, a.ow_magic);
      sp = oh * a.stride_h * a.iw + (r - oh * a.ow) * a.stride_w;
    }
    pi.in_off = ((unsigned)n * (unsigned)(a.ic2 * a.ihw) + (unsigned)sp) * 16u;
    pi.out_off = with_out ? (a.out_nhwc ? (unsigned)gpc * (unsigned)(a.oc2 * 16) : ((unsigned)n * (unsigned)(a.oc2 * a.ohw) + (unsigned)r) * 16u) : 0u;
    return pi;
  };
  // byte offset, from the pixel's out_off, of the lane's cell in the wave's tile mt
  const unsigned tile_stride = a.out_nhwc ? 32u : 2u * (unsigned)a.ohw * 16u;
  const unsigned lane_cell = a.out_nhwc ? (unsigned)oc_lane : (unsigned)(oc_lane >> 4) * (unsigned)a.ohw * 16u;
  const unsigned unit_stride = (unsigned)a.ihw * 16u;

  // tile tt of the run into stage st: k-step j's operand is one wave-load (lane = unit 2 j + lh, pixel l32)
  // landing at st + 1 KB * j; the waves take one in NW.  With the sum, the wave's own TM cells per lane
  // follow at st + 1 KB * (NKS + TM wave + mt), lane i's at + 16 i.  A tile's loads are issued one by one (load d of
  // the wave's LPT), so that they can be spread over the k-steps of a K loop.
  constexpr int LPT = NKS / NW + (SUM ? TM : 0);   // loads of one wave per tile
  unsigned pend_in = 0, pend_out = 0, pend_sb = 0;
  auto issue_setup = [&](int tt, int st) {
    const PixInfo pi = pix_info(tt);
    pend_in = pi.in_off + (unsigned)lh * unit_stride;
    pend_out = pi.out_off + lane_cell;
    pend_sb = lds_base + (unsigned)st * (unsigned)stage_bytes;
  };
  auto issue_load = [&](int d) {
    if (d < NKS / NW) {
      const int j = wave + NW * d;
      dma16(a.in + (size_t)(2 * j) * unit_stride, pend_in, pend_sb + 1024u * (unsigned)j);
    } else if (SUM) {
      const int mt = d - NKS / NW;
      // (a tile of channels behind the real ones reads the cell of tile 0: any readable address will do)
      const bool ok = oc_lane + 32 * mt < oc_real;
      dma16(a.out, ok ? pend_out + mt * tile_stride : pend_out - lane_cell, pend_sb + 1024u * (unsigned)(NKS + TM * wave + mt));
    }
  };
  auto issue_tile = [&](int tt, int st) {
    issue_setup(tt, st);
#pragma unroll
    for (int d = 0; d < LPT; ++d) issue_load(d);
  };

  // ---- prologue ------------------------------------------------------------------------------------------------
  // First what the leading arguments alone can address: the first tile's pixels and the weights.  The rest of the
  // argument block (output pointer, constants, ring depth) is still on its way from memory then.
  {
    const PixInfo pi = pix_info(0, false);
    pend_in = pi.in_off + (unsigned)lh * unit_stride;
    pend_sb = lds_base;
#pragma unroll
    for (int d = 0; d < NKS / NW; ++d) issue_load(d);
  }
  // the per-channel constants next (into registers now, into LDS once the weights are in): the first tile's epilogue
  // is what waits for them, and behind the weights they would arrive a trip to memory later
  const int cl_idx = lane < OCW ? lane : OCW - 1;
  const float c_sc = consts[ocw + cl_idx];
  const float c_sh = consts[ocpp + ocw + cl_idx];
  const int c_comp = reinterpret_cast<const int *>(consts)[2 * ocpp + ocw + cl_idx];
  TRACE_POINT(1);
  // weights [units][ocpp][16]: lane = packed row l32 of unit 2 ks + lh; tile mt 32 rows on
  const int8_t *wb = a.w + ((long long)lh * a.ocpp + ocw + l32) * 16;
  const long long w_step = (long long)a.ocpp * 32;   // two units
  v4i areg[NKS][TM];
#pragma unroll
  for (int ks = 0; ks < NKS; ++ks)
#pragma unroll
    for (int mt = 0; mt < TM; ++mt) areg[ks][mt] = *reinterpret_cast<const v4i *>(wb + ks * w_step + mt * 512);
  // Then what needs the argument block: the first tile's sum operand, the second tile.  (The compiler's waits for the weights cover
  // the few loads it does not know of that follow them: the last k-steps of the first tile wait for the second
  // tile, which the tile's barrier waits for anyway.)
  const int nbuf = a.wr_nbuf;
  float *const cl_f = reinterpret_cast<float *>(lds + (size_t)nbuf * stage_cells) + wave * (3 * OCW);
  if (SUM) {
    issue_setup(0, 0);
#pragma unroll
    for (int d = NKS / NW; d < LPT; ++d) issue_load(d);
  }
  if (ntiles > 1) issue_tile(1, 1);
  // (the other tiles that fit in the ring are asked for from the first tile's K loop: queued here, ahead of the
  // first loads of the CU's other workgroup, they delayed its start by more than they gained -- 256 -> 512 stride 2 at
  // 56 x 56 13.8 against 13.4 us.  Stage nbuf - 1 stays free for the tile that the second tile's K loop asks for.)
  const int npre = nbuf > 3 ? nbuf - 2 : 1;   // tiles 1 .. npre are in flight when the first tile ends
  // the lane's constants of tile mt, channels 4 q .. 4 q + 3, out of LDS
  auto cl_read = [&](int arr, int mt, int q) -> float4 {
    return *reinterpret_cast<const float4 *>(cl_f + OCW * arr + 32 * mt + 16 * lh + 4 * q);
  };
  const bool out_s8 = a.ep.out_type == EHIP_S8;
  const float hi = out_s8 ? __builtin_fminf(a.ep.hi, 127.0f) : a.ep.hi;
  const float lo = a.ep.lo;
  const float sum_scale = a.ep.sum_scale;

  // tile 0 has landed once the first weights have (loads complete in issue order): the first operand read
  // depends on them, then a barrier for the other waves' shares
  v4i bq[4];
  {
    int dep = 0;
    asm volatile("" : "+v"(dep) : "v"(areg[0][0]));
    __syncthreads();
    const v4i *tb0 = lds + lane + dep;
    bq[0] = tb0[0];
    bq[1] = tb0[64];
    bq[0] ^= (int)0x80808080;
  }
  TRACE_POINT(2);

  // One tile: K loop and epilogue.  The first tile is a copy of its own: only there are loads that the compiler
  // knows of (weights, constants) still in flight, and its waits for them must not be part of the other tiles' code.
  auto tile_step = [&](auto first_tag, int t, int st) {
    constexpr bool FIRST = decltype(first_tag)::value;
    const int stn = st + 1 == nbuf ? 0 : st + 1;   // the next tile's stage
    const v4i *tb = lds + (size_t)st * stage_cells + lane;
    const v4i *tbn = lds + (size_t)stn * stage_cells + lane;
    // tile t + nbuf - 2 goes into the stage that the barrier of tile t - 1 has freed (tile t - 2's), a load per k-step
    const bool issue = !FIRST && nbuf >= 3 && t + nbuf - 2 < ntiles;
    if (issue) issue_setup(t + nbuf - 2, st < 2 ? st + nbuf - 2 : st - 2);
    // the accumulators start from the compensation (the first tile's from zero: its constants are not in LDS yet,
    // its epilogue adds the compensation)
    v16i acc[TM];
#pragma unroll
    for (int mt = 0; mt < TM; ++mt)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        float4 c = make_float4(0.f, 0.f, 0.f, 0.f);
        if (!FIRST) c = cl_read(2, mt, q);
        acc[mt][4 * q] = __float_as_int(c.x); acc[mt][4 * q + 1] = __float_as_int(c.y);
        acc[mt][4 * q + 2] = __float_as_int(c.z); acc[mt][4 * q + 3] = __float_as_int(c.w);
      }
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
      if (FIRST && ks == NKS - 2) {
        // every load the compiler knows of (weights, constants) has been consumed or is pinned here, before the
        // next load it does not know of is issued behind them: its own waits stay exact.  The constants go to LDS.
#pragma unroll
        for (int mt = 0; mt < TM; ++mt) asm volatile("" : : "v"(areg[NKS - 1][mt]), "v"(areg[NKS - 2][mt]));
        if (lane < OCW) {
          cl_f[lane] = c_sc;
          cl_f[OCW + lane] = c_sh;
          reinterpret_cast<int *>(cl_f)[2 * OCW + lane] = c_comp;
        }
        for (int tt = 2; tt <= npre && tt < ntiles; ++tt) issue_tile(tt, tt);   // (their stages have never been used)
      }
      // (the first tile does this behind its epilogue: its second tile was asked for a moment ago and is a trip to
      // memory away, time in which the epilogue's stores can already leave)
      if (!FIRST && ks == NKS - 2 && t + 1 < ntiles) {
        // this wave's share of tile t + 1 has landed: tiles issued behind it are t + 2 .. min(t + nbuf - 2, ntiles - 1)
        const int last = t + nbuf - 2 < ntiles - 1 ? t + nbuf - 2 : ntiles - 1;
        wait_vm(LPT * (last - (t + 1) > 0 ? last - (t + 1) : 0));
        __syncthreads();
        // everybody's share has; and nobody reads tile t - 1's stage any more
      }
      // (all of a tile's loads go out before the k-step of the barrier, whose wait counts them: PER per k-step)
      constexpr int PER = (LPT + NKS - 3) / (NKS - 2);
      if (!FIRST && issue) {
#pragma unroll
        for (int d = ks * PER; d < (ks + 1) * PER; ++d)
          if (d < LPT) issue_load(d);
      }
#pragma unroll
      for (int mt = 0; mt < TM; ++mt) {
        acc[mt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(areg[ks][mt], bq[ks & 3], acc[mt], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        if (mt == 0 && (ks + 2 < NKS || !FIRST)) bq[(ks + 2) & 3] = ks + 2 < NKS ? tb[(ks + 2) * 64] : tbn[(ks + 2 - NKS) * 64];
        if (mt == TM - 1) bq[(ks + 1) & 3] ^= (int)0x80808080;
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    // ---- the tile's epilogue: arithmetic and rounding are those of lean_store_typed ---------------------------
    const PixInfo pi = pix_info(t);
#pragma unroll
    for (int mt = 0; mt < TM; ++mt) {
      v4i old;
      if (SUM) old = lds[(size_t)st * stage_cells + 64 * (NKS + TM * wave + mt) + lane];
      v4i out;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const float4 s4 = cl_read(0, mt, q), h4 = cl_read(1, mt, q);
        const float sc[4] = {s4.x, s4.y, s4.z, s4.w};
        const float sh[4] = {h4.x, h4.y, h4.z, h4.w};
        int cv[4] = {0, 0, 0, 0};
        if (FIRST) {
          const float4 c4 = cl_read(2, mt, q);
          cv[0] = __float_as_int(c4.x); cv[1] = __float_as_int(c4.y); cv[2] = __float_as_int(c4.z); cv[3] = __float_as_int(c4.w);
        }
        unsigned pk = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          float f = __builtin_fmaf((float)(FIRST ? acc[mt][4 * q + j] + cv[j] : acc[mt][4 * q + j]), sc[j], sh[j]);
          if (SUM) {
            const unsigned b = ((unsigned)old[q] >> (8 * j)) & 0xffu;
            const int o = SUM == 2 ? (int)(signed char)b : (int)b;
            f = __builtin_fmaf((float)o, sum_scale, f);
          }
          f = __builtin_amdgcn_fmed3f(f, lo, hi);
          pk = __builtin_amdgcn_cvt_pk_u8_f32(f, j, pk);
        }
        out[q] = (int)pk;
      }
      if (pi.valid && oc_lane + 32 * mt < oc_real) {
        // blocked output: non-temporal, the written line is not kept in L2 (10-15 % on the ResNet layers at 28 x 28 and
        // 56 x 56, 12.3 -> 11.95 us on the 512 -> 1024 stride-2 layer); nhwc output: plain -- a line's 16-byte pieces
        // come from several waves and must meet in L2 (256 -> 1024 at 14 x 14: 8.3 us plain, 13.6 non-temporal)
        uint8_t *dst = static_cast<uint8_t *>(a.out) + (pi.out_off + lane_cell + mt * tile_stride);
        // (the empty statements keep the compiler from merging the two stores: merged, they lose the non-temporal bit)
        if (a.out_nhwc) {
          asm volatile("" ::: "memory");
          store_out16<false>(dst, out);
        } else {
          store_out16<true>(dst, out);
          asm volatile("" ::: "memory");
        }
      }
    }
    if (FIRST && ntiles > 1) {
      // the second tile: this wave's share has landed (the epilogue's stores are younger than every load issued so
      // far and only make the wait stricter), then everybody's; its first two operands
      const int last = npre < ntiles - 1 ? npre : ntiles - 1;
      wait_vm(LPT * (last - 1 > 0 ? last - 1 : 0));
      __syncthreads();
      bq[0] = tbn[0];
      bq[1] = tbn[64];
      bq[0] ^= (int)0x80808080;
    }
  };
  tile_step(std::true_type{}, 0, 0);
  TRACE_POINT(3);
  for (int t = 1, st = 1 == nbuf ? 0 : 1; t < ntiles; ++t) {
    tile_step(std::false_type{}, t, st);
    st = st + 1 == nbuf ? 0 : st + 1;
  }
  TRACE_POINT(15);
}

namespace {
typedef void (*wres_kernel_t)(EHIP_WRES_HEAD, GemmArgs);
constexpr size_t kWresLds = 80 * 1024;   // two workgroups per CU

hipError_t wres_enqueue(const LaunchPlan<GemmArgs> &plan, hipStream_t s)
{
  const GemmArgs &a = plan.args;
  const bool dense = a.stride_h == 1 && a.stride_w == 1 && a.iw == a.ow;
  const unsigned geom = (unsigned)a.stride_h | (unsigned)a.stride_w << 8 | (dense ? 1u << 16 : 0u) | (unsigned)a.ny << 20;
  hipLaunchKernelGGL(reinterpret_cast<wres_kernel_t>(plan.kernel), plan.grid, plan.block, plan.lds, s, a.in, a.w, a.ep.scale, a.p_total,
                     a.ohw, a.ohw_magic, a.ihw, a.ocpp, geom, a.nx, (unsigned)a.ow | (unsigned)a.iw << 16, a.ow_magic, a);
  return hipGetLastError();
}

// TM: 32-channel tiles per wave.  Two with up to 512 input channels (the weights of 64 channels are 128 registers),
// one with 1024.
int wres_tm(int nks) { return nks <= 16 ? 2 : 1; }

wres_kernel_t wres_kernel(int nks, int sum, int nw)
{
  (void)nw;   // (eight waves in one workgroup per CU with up to 512 input channels: measured, 14.1 against 13.1 us on the
              // 512 -> 1024 stride-2 layer; two workgroups of four waves stay)
  switch (nks * 4 + sum) {
  case 4 * 4 + 0: return k_gemm1x1_wres<4, 2, 0, 4>;
  case 4 * 4 + 1: return k_gemm1x1_wres<4, 2, 1, 4>;
  case 4 * 4 + 2: return k_gemm1x1_wres<4, 2, 2, 4>;
  case 8 * 4 + 0: return k_gemm1x1_wres<8, 2, 0, 4>;
  case 8 * 4 + 1: return k_gemm1x1_wres<8, 2, 1, 4>;
  case 8 * 4 + 2: return k_gemm1x1_wres<8, 2, 2, 4>;
  case 16 * 4 + 0: return k_gemm1x1_wres<16, 2, 0, 4>;
  case 16 * 4 + 1: return k_gemm1x1_wres<16, 2, 1, 4>;
  case 16 * 4 + 2: return k_gemm1x1_wres<16, 2, 2, 4>;
  case 32 * 4 + 0: return k_gemm1x1_wres<32, 1, 0, 8>;
  case 32 * 4 + 1: return k_gemm1x1_wres<32, 1, 1, 8>;
  case 32 * 4 + 2: return k_gemm1x1_wres<32, 1, 2, 8>;
  }
  return nullptr;
}
int wres_nw(int nks) { return nks <= 16 ? 4 : 8; }

// The launch geometry, or false when the layer is not one for this kernel: two workgroups per CU (80 KB of LDS
// each) where the ring of stages then still holds three tiles or a whole run, else one per CU with all 160 KB.
struct WresGeom {
  int nks, tm, nw, sum, nb, nreg, tiles, stage, nbuf;
  size_t lds_bytes;
};
bool wres_geom(const GemmArgs &a, WresGeom &g)
{
  g.nks = a.ic2 / 2;   // (the packed weights may be padded to more units: never read)
  g.tm = wres_tm(g.nks);
  g.nw = wres_nw(g.nks);
  const int lean = lean_mode(a.ep, false);
  g.sum = (lean & 4) ? (a.ep.out_type == EHIP_S8 ? 2 : 1) : 0;
  g.nb = (a.oc2 * 16 + 32 * g.nw * g.tm - 1) / (32 * g.nw * g.tm);
  g.tiles = (a.p_total + 31) / 32;
  g.stage = g.nks * 1024 + (g.sum ? g.nw * g.tm * 1024 : 0);
  const size_t cl_bytes = g.nw * 3 * 32 * g.tm * 4;   // per-channel constants of the waves
  int forced_slots = 0, forced_nbuf = 0;
  if (const char *env = getenv("EHIP_WRES_SLOTS")) forced_slots = atoi(env);
  if (const char *env = getenv("EHIP_WRES_NBUF")) forced_nbuf = atoi(env);
  for (int per_cu = g.nw == 8 ? 1 : 2; per_cu >= 1; --per_cu) {
    const int slots = forced_slots > 0 ? forced_slots : 256 * per_cu;
    g.nreg = slots / g.nb > 0 ? slots / g.nb : 1;
    if (g.nreg > g.tiles) g.nreg = g.tiles;
    const int run = (g.tiles + g.nreg - 1) / g.nreg;   // tiles of the longest run
    int nbuf = (int)((160 * 1024 / per_cu - cl_bytes) / (size_t)g.stage);
    if (nbuf > 8) nbuf = 8;
    if (forced_nbuf >= 2 && forced_nbuf <= nbuf) nbuf = forced_nbuf;
    if (nbuf > run) nbuf = run < 2 ? 2 : run;
    if (nbuf >= 3 || (nbuf >= 2 && run <= nbuf)) {
      g.nbuf = nbuf;
      g.lds_bytes = (size_t)nbuf * g.stage + cl_bytes;
      return true;
    }
  }
  return false;
}
}  // namespace

// Does the layer run on the weights-resident kernel?  Blocked input, 1x1, 256 / 512 / 1024 input channels in whole
// k-steps, the lean epilogue, at least three quarters of the last channel block real.
bool gemm1x1_wres_applies(const GemmArgs &a, int nbatch)
{
  const char *env = getenv("EHIP_GEMM1X1_WRES");
  if (env && env[0] == '0') return false;
  if (nbatch != 1 || a.kh * a.kw > 1 || a.ep.shift_tab || a.in_nhwc) return false;
  if (!lean_mode(a.ep, false)) return false;
  // the kernel takes the per-channel constants as ONE leading pointer: scale, shift and compensation in one allocation
  if (a.ep.shift != a.ep.scale + a.ocpp || reinterpret_cast<const float *>(a.ep.comp) != a.ep.scale + 2 * (size_t)a.ocpp) return false;
  if (a.ic2 != 8 && a.ic2 != 16 && a.ic2 != 32 && a.ic2 != 64) return false;
  if (a.stride_h > 255 || a.stride_w > 255 || a.ow >= 65536 || a.iw >= 65536) return false;
  const int oc = a.oc2 * 16;
  const int oc_wg = 32 * wres_nw(a.ic2 / 2) * wres_tm(a.ic2 / 2);
  const int nb = (oc + oc_wg - 1) / oc_wg;
  if (nb >= 4096) return false;
  // fewer than three quarters of the channel blocks' rows real, or too few pixels to give every CU a run: the
  // other kernels' smaller tiles do better (EHIP_GEMM1X1_WRES=1 runs such layers here all the same: tests)
  const bool forced = env && env[0] == '1';
  if (!forced && (oc * 4 < nb * oc_wg * 3 || a.p_total < 32 * 64)) return false;
  // Measured against the resident-tile kernel at N = 64: ahead where a workgroup's run is three tiles or more with
  // up to 512 input channels (512 -> 1024 stride 2 at 14 x 14: 13.4 vs 16.5 us, 256 -> 1024 at 14 x 14: 8.3 vs 10.5,
  // 512 -> 256 at 28 x 28: 11.7 vs 13.4, 256 -> 256 at 28 x 28: 8.3 vs 9.8), level or behind with shorter runs
  // (512 -> 512 at 14 x 14: 8.0 vs 7.7, 512 -> 2048 at 7 x 7: 8.2 vs 8.0) and with 1024 input channels, whose waves own
  // one tile of 32 channels (1024 -> 256 at 14 x 14: 8.6 vs 8.4, 1024 -> 1024 at 7 x 7: 8.6 vs 7.2)
  if (!forced && (a.ic2 > 32 || (long long)((a.p_total + 31) / 32) * nb < 3 * 512)) return false;
  // a lane's offsets into the input and the output are 32 bits wide
  const long long n_img = a.p_total / (a.ohw > 0 ? a.ohw : 1);
  if (n_img * a.ic2 * a.ihw * 16 >= (1ll << 32) || (long long)a.p_total * a.oc2 * 16 >= (1ll << 32)) return false;
  WresGeom g;
  return wres_geom(a, g);
}

hipError_t launch_gemm1x1_wres(const GemmArgs &a0, hipStream_t s, LaunchPlan<GemmArgs> *plan)
{
  GemmArgs a = a0;
  a.lean = lean_mode(a.ep, false);
  WresGeom g;
  if (!wres_geom(a, g)) return hipErrorInvalidValue;
  wres_kernel_t kernel = wres_kernel(g.nks, g.sum, g.nw);
  if (!kernel) return hipErrorInvalidValue;
  a.ny = g.nb;
  a.nx = g.nreg;
  a.wr_region = g.tiles;
  a.wr_stage = g.stage;
  a.wr_nbuf = g.nbuf;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)g.lds_bytes);
  if (e != hipSuccess) return e;
  LaunchPlan<GemmArgs> local;
  LaunchPlan<GemmArgs> *p = plan ? plan : &local;
  p->kernel = reinterpret_cast<void (*)(GemmArgs)>(kernel);
  p->grid = dim3(8 * g.nb * ((g.nreg + 7) / 8));
  p->block = dim3(g.nw * 64);
  p->lds = (unsigned)g.lds_bytes;
  p->args = a;
  p->enqueue = wres_enqueue;
  p->name = "k_gemm1x1_wres";
  return plan_first_launch(p, s);
}

}  // namespace ehip
