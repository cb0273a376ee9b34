// Winograd GEMMs + output transform, the form whose lanes own a tile x four channels at every position, so that nothing
// is exchanged through LDS between the GEMMs and the transform: with the weights of 16 channels resident in LDS (up to
// 256 input channels in one pass, 512 in two) or with both operands streamed (up to 256).
//
// Replaces, for those layers, elx_int8_conv_wino_gemm_t::execute + trans_output as the reference's fused schedule
// runs them per thread (a161, src/elx_int8_conv_wino_xopt.hpp:21-179; src/elx_int8_conv_wino_gemm.cpp:23-205,
// src/elx_conv_wino_trans_output.cpp:212-423).
//
// A file of its own because it is compiled with the accumulators of the matrix instructions in the ordinary vector
// registers (-amdgpu-mfma-vgpr-form): the requantized values then take the accumulators' place and two workgroups
// fit on a CU, where the general kernel of ehip_wino.hip needs the accumulation registers for its 288 accumulators.
#include "ehip_internal.hpp"
#include "ehip_wino_tiles.hpp"
#include <type_traits>

namespace ehip {

namespace {

__device__ __forceinline__ float comp_of(const float4 &v, int k) { return k == 0 ? v.x : (k == 1 ? v.y : (k == 2 ? v.z : v.w)); }

// The pieces of output_tile (ehip_wino.hip) for u8 / s8 output with few registers: one channel at a time, its bytes
// packed into the pixels' dwords as they come (16 dwords live instead of 4 x 16 floats; the old output of the in-place
// sum stays packed as well).  Same operations in the same order per value as output_tile.
// pack_channel: channel k of the lane's four -- bias, output scale, old output, ReLU, rounding, byte k of the dwords.
template <int OUT, int A>
__device__ __forceinline__ void pack_channel(const float *o, float b, int k, bool with_relu, float repS, float z, bool with_sum,
                                             const unsigned *old, unsigned *pk)
{
  static_assert(OUT == EHIP_U8 || OUT == EHIP_S8, "quantized output");
  constexpr int M = A - 2;
#pragma unroll
  for (int e = 0; e < M * M; ++e) {
    float r = o[e] + b;
    r = __builtin_fmaf(r, repS, z);
    if (with_sum) {
      const unsigned ob = (old[e] >> (8 * k)) & 0xffu;
      r = r + (OUT == EHIP_U8 ? (float)ob : (float)(int)(signed char)ob);
    }
    if (with_relu) {
      r = __builtin_amdgcn_fmed3f(r, 0.0f, OUT == EHIP_S8 ? 127.0f : 255.0f);
      if (A == 4) r = __builtin_floorf(r);
      pk[e] = __builtin_amdgcn_cvt_pk_u8_f32(r, k, pk[e]);
    } else if (A == 4) {
      const float fl = __builtin_floorf(r);
      if (OUT == EHIP_U8) pk[e] = __builtin_amdgcn_cvt_pk_u8_f32(r >= 0.0f ? fl : 300.0f, k, pk[e]);
      else pk[e] |= ((unsigned)ssat8(cvt_s32_rne(fl)) & 0xffu) << (8 * k);
    } else {
      if (OUT == EHIP_U8) pk[e] = __builtin_amdgcn_cvt_pk_u8_f32(r >= -0.5f ? r : 300.0f, k, pk[e]);
      else pk[e] |= ((unsigned)ssat8(cvt_s32_rne(r)) & 0xffu) << (8 * k);
    }
  }
}

// 4 x 4 transpose of dwords between four registers and the four 16-lane rows of a wave: register j of row g becomes
// register g of row j (v_permlane32_swap exchanges the upper rows of one register with the lower rows of another,
// v_permlane16_swap the odd rows with the even ones).  All lanes take part.
__device__ __forceinline__ void rows_transpose(unsigned &x0, unsigned &x1, unsigned &x2, unsigned &x3)
{
  auto a = __builtin_amdgcn_permlane32_swap(x0, x2, false, false);
  auto b = __builtin_amdgcn_permlane32_swap(x1, x3, false, false);
  auto c = __builtin_amdgcn_permlane16_swap(a[0], b[0], false, false);
  auto d = __builtin_amdgcn_permlane16_swap(a[1], b[1], false, false);
  x0 = c[0];
  x1 = c[1];
  x2 = d[0];
  x3 = d[1];
}

// Output by whole cells of 16 channels: the four lanes of a tile (rows g = 0 .. 3 of the wave, four channels each) hold
// the 16 bytes of every pixel between them; after the transpose the lane of row g holds the whole cell of the pixel in
// column g of the tile's row i and writes it with one 16-byte store (a wave then covers 16 tiles x 4 pixels of an
// image row = up to 1 KB in one piece, where dword stores leave 16 pieces of 16 bytes per instruction).
// block: the tile's image and channel block; ok: the tile exists.  Called by all lanes.
template <int A>
__device__ __forceinline__ void store_cells(const unsigned *pk, uint8_t *block, int g, bool ok, int th, int tw, int oh_n, int ow_n,
                                            int px)
{
  constexpr int M = A - 2;
#pragma unroll
  for (int i = 0; i < M; ++i) {
    unsigned c0 = pk[M * i], c1 = pk[M * i + 1], c2 = M > 2 ? pk[M * i + (M > 2 ? 2 : 0)] : 0u, c3 = M > 3 ? pk[M * i + (M > 3 ? 3 : 0)] : 0u;
    rows_transpose(c0, c1, c2, c3);
    const int oh = M * th + i, ow = M * tw + g;
    if (ok && g < M && oh < oh_n && ow < ow_n) {
      // (non-temporal: the output would only push the transformed input, which the other channel blocks' workgroups
      // still read, out of the L2 -- 128 -> 128 at 112 x 112: 130 -> 100 us)
      typedef unsigned v4u __attribute__((ext_vector_type(4)));
      const v4u vv = {c0, c1, c2, c3};
      __builtin_nontemporal_store(vv, reinterpret_cast<v4u *>(block + ((size_t)oh * ow_n + ow) * px));
    }
  }
}

// the old output of the in-place sum the same way round: cells in, the lane's four channels of every pixel out
template <int A>
__device__ __forceinline__ void load_old_cells(unsigned *old, const uint8_t *block, int g, int th, int tw, int oh_n, int ow_n, int px)
{
  constexpr int M = A - 2;
#pragma unroll
  for (int i = 0; i < M; ++i) {
    const int oh = M * th + i, ow = M * tw + g;
    const bool in = g < M && oh < oh_n && ow < ow_n;
    const uint4 c = *reinterpret_cast<const uint4 *>(block + (in ? ((size_t)oh * ow_n + ow) * px : 0));
    unsigned c0 = c.x, c1 = c.y, c2 = c.z, c3 = c.w;
    rows_transpose(c0, c1, c2, c3);
    old[M * i] = c0;
    old[M * i + 1] = c1;
    if (M > 2) old[M * i + (M > 2 ? 2 : 0)] = c2;
    if (M > 3) old[M * i + (M > 3 ? 3 : 0)] = c3;
  }
}

// All positions of the lane's tile x four channels -> the output: Y = At M A channel by channel, packed, and written by
// whole cells.  Called by all lanes of the wave (ok: the lane's tile and channels exist).
template <int OUT, int A>
__device__ __forceinline__ void output_tile_packed(const float4 *m, const float4 &bias, bool with_relu, float repS, float z,
                                                   uint8_t *block, int g, bool ok, int th, int tw, int oh_n, int ow_n,
                                                   bool with_sum, int px)
{
  constexpr int AA = A * A, M = A - 2;
  unsigned pk[M * M], old[M * M];
#pragma unroll
  for (int e = 0; e < M * M; ++e) pk[e] = 0u;
  if (with_sum) load_old_cells<A>(old, block, g, th, tw, oh_n, ow_n, px);
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    float f[AA], o[M * M];
#pragma unroll
    for (int e = 0; e < AA; ++e) f[e] = comp_of(m[e], k);
    wino::tile_output<A>(f, o);
    pack_channel<OUT, A>(o, comp_of(bias, k), k, with_relu, repS, z, with_sum, old, pk);
    // (one channel after the other: interleaved, the four transforms' intermediates do not fit the registers)
    __builtin_amdgcn_sched_barrier(0);
  }
  store_cells<A>(pk, block, g, ok, th, tw, oh_n, ow_n, px);
}

// f32 output (no output scale, no in-place sum here): bias and ReLU as output_tile applies them, and the lane's four
// channels of every pixel leave as one 16-byte store (the four lanes of a tile write the 64 bytes of a pixel's block).
// y: [channel][pixel]; block: the tile's image and channel block, in floats.
template <int A>
__device__ __forceinline__ void finish_channel_f32(float *y, float b, bool with_bias, bool with_relu)
{
  constexpr int M = A - 2;
#pragma unroll
  for (int e = 0; e < M * M; ++e) {
    float r = y[e];
    if (with_bias) r = r + b;
    if (with_relu) r = r > 0.0f ? r : 0.0f;
    y[e] = r;
  }
}
template <int A>
__device__ __forceinline__ void store_f32(const float (*y)[(A - 2) * (A - 2)], float *block, int g, bool ok, int th, int tw, int oh_n,
                                          int ow_n, int px)
{
  constexpr int M = A - 2;
  typedef float v4f __attribute__((ext_vector_type(4)));
  if (!ok) return;
#pragma unroll
  for (int i = 0; i < M; ++i) {
    const int oh = M * th + i;
    if (oh >= oh_n) break;
#pragma unroll
    for (int j = 0; j < M; ++j) {
      const int ow = M * tw + j;
      if (ow >= ow_n) break;
      const int e = M * i + j;
      const v4f vv = {y[0][e], y[1][e], y[2][e], y[3][e]};
      // (non-temporal: output that nothing reads back soon)
      __builtin_nontemporal_store(vv, reinterpret_cast<v4f *>(block + ((size_t)oh * ow_n + ow) * px + 4 * g));
    }
  }
}

// the one-dimensional output transform of tile sizes 6 and 5
template <int A>
__device__ __forceinline__ void out_1d(const float *f, float *o)
{
  if (A == 6) wino::out6_1d(f, o);
  else wino::out5_1d(f, o);
}

}  // namespace

// The general kernel (k_wino_gemm_output, ehip_wino.hip) keeps 64 channels x 32 tiles x all positions in its four waves'
// registers, one wave per SIMD, and passes the results through 144 KB of LDS to the transform; with few input channels
// it is all output phase (64 -> 64: 37 K of a workgroup's 47 K clocks).
// Here v_mfma_i32_16x16x64_i8 makes the GEMM's own result layout the transform's: a lane of the 16 x 16 result holds
// four consecutive rows = four consecutive output channels of ONE tile, so with all A x A positions of its 16
// channels x 16 tiles in one wave (4 accumulator registers per position) every lane already owns the A x A values
// of one tile x four channels -- requantization and Y = At M A happen in the lane, with no exchange through LDS, no
// barrier, and two workgroups per CU to hide each other's latencies; only the finished bytes are transposed between the
// wave's rows, for stores of whole cells.  The price is the operand stream: 2 KB per 16 x 16 x 64 MFMA, which only so
// short a K loop can afford.
// Workgroup = 32 channels x 32 tiles (one block of the blocked tinput); wave = (half of the channels, half of the
// tiles); NKS = k-steps of 64 channels per position (1, 2 or 4).
template <int A, bool SUM, int NKS>
__global__ __launch_bounds__(kBlock, 2) void k_wino_gemm_output_lanes(WinoFusedArgs a)
{
  constexpr int AA = A * A, D = 8, STEPS = AA * NKS;
  extern __shared__ float4 cl[];   // [AA][3][8 quads of the workgroup's 32 channels]: scale, shift, compensation
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l16 = lane & 15, g = lane >> 4;
  const int xcd = blockIdx.x & 7, seq = blockIdx.x >> 3;
  const int by = seq % a.ny;
  const int bx = (seq / a.ny) * 8 + xcd;
  if (bx >= a.nx) return;          // whole workgroup
  const int oc0 = by * 32;
  // the wave's 16 channels are one block of the output: of the group of 32 packed rows (row 8 gq + 4 h + j holds
  // channel 16 h + 4 gq + j) it takes the rows of half h, gathered so that MFMA row 4 gq + j is channel 16 h + 4 gq + j
  const int h = wave & 1;
  const int th16 = (wave >> 1) * 16;       // its tiles inside the block of 32
  const int oc_real = a.oc2 * 16;

  // operands: lane = packed row / tile l16 of unit 4 ks + g, one 16-byte cell each; a wave-uniform base per step plus
  // one 32-bit offset per lane (as 64-bit pointers per lane the unrolled loop's 72 addresses fill the register file)
  const unsigned a_off = (unsigned)(g * a.ocpp + oc0 + 8 * (l16 >> 2) + 4 * h + (l16 & 3)) * 16u;
  const long long w_pos = (long long)a.units_pad * a.ocpp * 16, w_ks = (long long)4 * a.ocpp * 16;
  const uint8_t *tbase = a.tin + (long long)bx * AA * a.ic2 * 512;
  const long long t_pos = (long long)a.ic2 * 512;
  unsigned b_off[NKS];
#pragma unroll
  for (int ks = 0; ks < NKS; ++ks) {
    // units past the last real one multiply zero weights: any valid cell will do
    int u = 4 * ks + g;
    u = u < a.ic2 ? u : a.ic2 - 1;
    b_off[ks] = (unsigned)(u * 512 + (th16 + l16) * 16);
  }
  v4i ra[D], rb[D];
  auto issue = [&](int slot, int sn) {
    const int p = sn / NKS, ks = sn - NKS * p;
    const int8_t *wp = a.w + p * w_pos + ks * w_ks;      // wave-uniform
    const uint8_t *tp = tbase + p * t_pos;               // wave-uniform
    ra[slot] = *reinterpret_cast<const v4i *>(wp + a_off);
    rb[slot] = *reinterpret_cast<const v4i *>(tp + b_off[ks]);
  };
  // the first operands are requested before anything else; the constants of the workgroup's channels (24 cells of
  // four channels per position) travel behind them, all of a thread's loads before its first store
#pragma unroll
  for (int k = 0; k < D; ++k)
    if (k < STEPS) issue(k, k);
  {
    constexpr int NC = (AA * 24 + kBlock - 1) / kBlock;
    float4 cst[NC];
#pragma unroll
    for (int j = 0; j < NC; ++j) {
      int idx = tid + j * kBlock;
      idx = idx < AA * 24 ? idx : AA * 24 - 1;
      const int p = idx / 24, rem = idx - 24 * p, arr = rem >> 3, cell = rem & 7;
      const float *src = arr == 0 ? a.scale : (arr == 1 ? a.shift : reinterpret_cast<const float *>(a.comp));
      cst[j] = *reinterpret_cast<const float4 *>(src + (long long)p * a.ocpp + oc0 + 4 * cell);
    }
#pragma unroll
    for (int j = 0; j < NC; ++j) {
      const int idx = tid + j * kBlock;
      if (idx < AA * 24) cl[idx] = cst[j];
    }
  }
  __syncthreads();   // the constants are in LDS
  const int quad = 4 * h + g;   // the lane's four channels: cell inside the group of 32
  // the accumulators start from the compensation 128 * sum(weights) of their (position, channel)
  v4i acc[AA];
#pragma unroll
  for (int e = 0; e < AA; ++e) {
    const float4 cf = cl[e * 24 + 16 + quad];
    acc[e] = v4i{__float_as_int(cf.x), __float_as_int(cf.y), __float_as_int(cf.z), __float_as_int(cf.w)};
  }
#pragma unroll
  for (int sn = 0; sn < STEPS; ++sn) {
    const v4i b = rb[sn % D] ^ (int)0x80808080;
    acc[sn / NKS] = __builtin_amdgcn_mfma_i32_16x16x64_i8(ra[sn % D], b, acc[sn / NKS], 0, 0, 0);
    if (sn + D < STEPS) issue(sn % D, sn + D);
    __builtin_amdgcn_sched_barrier(0);   // (the loads stay where the ring puts them: hoisted, they spill)
  }
  const int oc = oc0 + 4 * quad;
  const int t = bx * 32 + th16 + l16;
  // (lanes without a tile or channel of their own take part with tile 0 / channel 0 and store nothing)
  const bool valid = t < a.t && oc < oc_real;
  float4 m[AA];
  int cq = quad;   // (the constants' cell, re-derived group by group: see below)
#pragma unroll
  for (int e = 0; e < AA; ++e) {
    const float4 sc = cl[e * 24 + cq], sh = cl[e * 24 + 8 + cq];
    m[e].x = __builtin_fmaf((float)acc[e][0], sc.x, sh.x);
    m[e].y = __builtin_fmaf((float)acc[e][1], sc.y, sh.y);
    m[e].z = __builtin_fmaf((float)acc[e][2], sc.z, sh.z);
    m[e].w = __builtin_fmaf((float)acc[e][3], sc.w, sh.w);
    // (four positions' constants in flight at a time: the compiler would read all 108 cells first and spill the
    // accumulators to make room, so the next group's address is made to depend on this group's last result)
    // (and every value is pinned where it is computed: sunk towards their use, the values leave their constants live)
    asm volatile("" : "+v"(m[e].x), "+v"(m[e].y), "+v"(m[e].z), "+v"(m[e].w));
    if ((e & 3) == 3) asm volatile("" : "+v"(cq) : "v"(m[e].w));
  }
  const int tc = valid ? t : 0, occ = valid ? oc : 0;
  const int n = tc / a.nt;
  const int rem = tc - n * a.nt;
  const int th = rem / a.wt;
  const int tw = rem - th * a.wt;
  float4 bias = make_float4(0.f, 0.f, 0.f, 0.f);
  if (a.with_bias) bias = *reinterpret_cast<const float4 *>(a.bias + occ);
  const size_t block = a.out_nhwc ? (size_t)n * a.oh * a.ow * a.oc2 * 16 + (occ >> 4) * 16
                                  : ((size_t)n * a.oc2 + (occ >> 4)) * a.oh * a.ow * 16;
  const int px = a.out_nhwc ? a.oc2 * 16 : 16;
  if (!SUM && a.out_type == EHIP_F32) {
    // channel by channel: a channel's requantized positions die as its 16 outputs are born
    constexpr int M = A - 2;
    float y[4][M * M];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      float f[AA];
#pragma unroll
      for (int e = 0; e < AA; ++e) f[e] = comp_of(m[e], k);
      wino::tile_output<A>(f, y[k]);
      finish_channel_f32<A>(y[k], comp_of(bias, k), a.with_bias != 0, a.with_relu != 0);
#pragma unroll
      for (int e = 0; e < M * M; ++e) asm volatile("" : "+v"(y[k][e]));
      __builtin_amdgcn_sched_barrier(0);
    }
    store_f32<A>(y, static_cast<float *>(a.out) + block, g, valid, th, tw, a.oh, a.ow, px);
    return;
  }
  if (a.out_type == EHIP_U8)
    output_tile_packed<EHIP_U8, A>(m, bias, a.with_relu != 0, a.out_repS, a.out_z, static_cast<uint8_t *>(a.out) + block, g,
                                   valid, th, tw, a.oh, a.ow, SUM, px);
  else
    output_tile_packed<EHIP_S8, A>(m, bias, a.with_relu != 0, a.out_repS, a.out_z, static_cast<uint8_t *>(a.out) + block, g,
                                   valid, th, tw, a.oh, a.ow, SUM, px);
}

// The same lanes, weights resident: with at most 128 input channels the packed weights of 16 channels at every position
// fit the LDS twice over (36 or 72 KB a workgroup; with 192 / 256 channels once: NW = 4 or 8 waves, one workgroup per
// CU), so a workgroup = 16 channels x 16 NW tiles stages them once and then walks over blocks of that many tiles: the operand stream from L2 is the transformed input alone (half of what the form
// above requests per MFMA), every wave has tiles of its own (nothing is requested twice inside a workgroup), and the
// ring of input operands runs on from one block of tiles to the next, so the first operands of the next block travel
// while this one's output transform keeps the vector units busy.  No barrier after the staging.
// a.nx = blocks of 16 NW tiles, a.ny = groups of 16 packed rows; grid = 8 XCDs x a.ny x slots, a slot walks over the
// blocks slot * 8 + xcd, + 8 * slots, ...
template <int A, bool SUM, int NKS, int NW = 4>
__global__ __launch_bounds__(64 * NW, 2) void k_wino_gemm_output_lanes_wres(WinoFusedArgs a)
{
  constexpr int TB = 64 * NW;   // threads; a block of tiles of the workgroup = 16 NW tiles = NW / 2 blocks of 32
  constexpr int AA = A * A, STEPS = AA * NKS;
  constexpr int D = A == 6 ? (SUM ? 6 : 12) : (A == 5 ? 5 : 8);   // divides STEPS: a ring slot holds the same steps in every block
  static_assert(STEPS % D == 0, "ring");
  extern __shared__ float4 lds[];
  v4i *wl = reinterpret_cast<v4i *>(lds);   // [STEPS][4 units][16 packed rows] cells of 16 bytes
  float4 *cl = lds + STEPS * 64;            // [AA][3][4 quads of the workgroup's 16 rows]: scale, shift, compensation
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l16 = lane & 15, g = lane >> 4;
  const int xcd = blockIdx.x & 7, seq = blockIdx.x >> 3;
  const int by = seq % a.ny;
  const int slot = seq / a.ny;
  const int item_step = 8 * (int)(gridDim.x / (8u * a.ny));
  int item = slot * 8 + xcd;
  if (item >= a.nx) return;          // whole workgroup
  // the workgroup's 16 channels are one block of the output: of the group of 32 packed rows (row 8 gq + 4 h + j holds
  // channel 16 h + 4 gq + j) it takes the rows of half h, gathered so that MFMA row 4 gq + j is channel 16 h + 4 gq + j
  // and the four lanes of a tile write the 16 bytes of a pixel's channel block together
  const int oc0 = (by >> 1) * 32, h = by & 1;
  const int oc_real = a.oc2 * 16;
  const int nblk = (a.t + 31) >> 5;

  const long long t_pos = (long long)a.ic2 * 512;
  const long long t_blk = t_pos * AA;
  unsigned b_off[NKS];
#pragma unroll
  for (int ks = 0; ks < NKS; ++ks) {
    // units past the last real one multiply zero weights: any valid cell will do
    int u = 4 * ks + g;
    u = u < a.ic2 ? u : a.ic2 - 1;
    b_off[ks] = (unsigned)(u * 512 + ((wave & 1) * 16 + l16) * 16);
  }
  // the wave's block of 32 tiles inside the item (the last item of an odd count has one block only: its upper waves
  // read the lower block again and store nothing)
  auto base_of = [&](int it) {
    int blk = (NW / 2) * it + (wave >> 1);
    blk = blk < nblk ? blk : nblk - 1;
    return a.tin + blk * t_blk;      // wave-uniform
  };
  v4i rb[D];
  // step sn = (column i, row r, k-step ks) in that order; its position is A r + i (tile size 4: one group, in order)
  auto issue = [&](int rs, int sn, const uint8_t *tb) {
    const int ks = sn % NKS, pr = sn / NKS;
    const int p = A == 4 ? pr : A * (pr % A) + pr / A;
    rb[rs] = *reinterpret_cast<const v4i *>(tb + p * t_pos + b_off[ks]);
  };
  const uint8_t *tb = base_of(item);
#pragma unroll
  for (int k = 0; k < D; ++k) issue(k, k, tb);
  {
    // the weights: per (step, unit) 16 rows x 16 bytes = 256 contiguous bytes of [pos][unit][OCpp][16]
    constexpr int NP = (STEPS * 64 + TB - 1) / TB;
    const long long w_pos = (long long)a.units_pad * a.ocpp * 16;
    v4i tmp[NP];
#pragma unroll
    for (int j = 0; j < NP; ++j) {
      int idx = tid + j * TB;
      idx = idx < STEPS * 64 ? idx : STEPS * 64 - 1;
      const int chunk = idx >> 4, cell = idx & 15;
      const int sn = chunk >> 2, u = chunk & 3;
      const int p = sn / NKS, ks = sn - NKS * p;
      tmp[j] = *reinterpret_cast<const v4i *>(a.w + p * w_pos +
                                              ((long long)(4 * ks + u) * a.ocpp + oc0 + 8 * (cell >> 2) + 4 * h + (cell & 3)) * 16);
    }
    constexpr int NC = (AA * 12 + TB - 1) / TB;
    float4 cst[NC];
#pragma unroll
    for (int j = 0; j < NC; ++j) {
      int idx = tid + j * TB;
      idx = idx < AA * 12 ? idx : AA * 12 - 1;
      const int p = idx / 12, rem = idx - 12 * p, arr = rem >> 2, gq = rem & 3;
      const float *src = arr == 0 ? a.scale : (arr == 1 ? a.shift : reinterpret_cast<const float *>(a.comp));
      cst[j] = *reinterpret_cast<const float4 *>(src + (long long)p * a.ocpp + oc0 + 16 * h + 4 * gq);
    }
#pragma unroll
    for (int j = 0; j < NP; ++j) {
      const int idx = tid + j * TB;
      if (idx < STEPS * 64) wl[idx] = tmp[j];
    }
#pragma unroll
    for (int j = 0; j < NC; ++j) {
      const int idx = tid + j * TB;
      if (idx < AA * 12) cl[idx] = cst[j];
    }
  }
  const int oc = oc0 + 16 * h + 4 * g;   // the lane's four channels
  const bool oc_ok = oc < oc_real;
  float4 bias = make_float4(0.f, 0.f, 0.f, 0.f);
  if (a.with_bias && oc_ok) bias = *reinterpret_cast<const float4 *>(a.bias + oc);
  const int px = a.out_nhwc ? a.oc2 * 16 : 16;
  __syncthreads();   // weights and constants are in LDS; the waves run on their own from here
  // the lane's cells as opaque bases: every read below is base + immediate offset (left to itself the compiler folds
  // the constants' place behind the weights into each address, beyond the offset field, one register per cell)
  int wla = g * 16 + l16, clg = STEPS * 64 + g;   // cells of 16 bytes from the start of the LDS
  asm volatile("" : "+v"(wla), "+v"(clg));
  // Tile sizes 6 and 5: Y = At M A one dimension at a time.  The steps run column by column of M (positions A r + i,
  // r = 0 .. A - 1): a column's A positions are multiplied, requantized and taken through the first one-dimensional
  // transform at once, which leaves (A - 2) values per column and channel -- so a lane keeps 4 x (A - 2) x A floats and
  // one column of accumulators instead of all A x A positions, and the vector work of one column runs while the
  // operands of the next ones travel.  Tile size 4 (a two-dimensional formula in the reference) keeps its 16 positions.
  constexpr int M = A - 2;
  constexpr int NCOL = A == 4 ? 1 : A;      // groups of positions that are finished together
  constexpr int PER = AA / NCOL;            // positions per group
  // the weights of step sn: cell offset of its (position, k-step)
  auto wcell = [](int sn) {
    const int ks = sn % NKS, pr = sn / NKS;
    const int p = A == 4 ? pr : A * (pr % A) + pr / A;
    return (p * NKS + ks) * 64;
  };
  for (;;) {
    const int next = item + item_step;
    const bool more = next < a.nx;                      // wave-uniform
    const uint8_t *tbn = base_of(more ? next : item);   // (the last block's tail requests its own head again: unused)
    const int t = item * (16 * NW) + wave * 16 + l16;
    const bool valid = t < a.t && oc_ok;
    // (lanes without a tile or channel of their own take part with tile 0 / channel 0 and store nothing)
    const int tc = valid ? t : 0, occ = valid ? oc : 0;
    const int n = tc / a.nt;
    const int rem = tc - n * a.nt;
    const int th = rem / a.wt;
    const int tw = rem - th * a.wt;
    uint8_t *plane = static_cast<uint8_t *>(a.out) +
        (a.out_nhwc ? (size_t)n * a.oh * a.ow * a.oc2 * 16 + (occ >> 4) * 16 : ((size_t)n * a.oc2 + (occ >> 4)) * a.oh * a.ow * 16);
    float T[4][M][A == 4 ? 1 : A];   // first-stage results [channel][row][column]
    float4 m4[A == 4 ? AA : 1];      // tile size 4: the requantized positions
    unsigned old[M * M];
    v4i ra[3];
    ra[0] = wl[wla + wcell(0)];
    ra[1] = wl[wla + wcell(1)];
#pragma unroll
    for (int i = 0; i < NCOL; ++i) {
      if (SUM && i == NCOL - 1) load_old_cells<A>(old, plane, g, th, tw, a.oh, a.ow, px);
      // the accumulators start from the compensation 128 * sum(weights) of their (position, channel)
      v4i acc[PER];
#pragma unroll
      for (int r = 0; r < PER; ++r) {
        const int p = NCOL == 1 ? r : A * r + i;
        const float4 cf = lds[clg + p * 12 + 8];
        acc[r] = v4i{__float_as_int(cf.x), __float_as_int(cf.y), __float_as_int(cf.z), __float_as_int(cf.w)};
      }
#pragma unroll
      for (int r = 0; r < PER; ++r)
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) {
          const int sn = (i * PER + r) * NKS + ks;
          if (sn + 2 < STEPS) ra[(sn + 2) % 3] = wl[wla + wcell(sn + 2)];   // the weights of the step after next
          const v4i b = rb[sn % D] ^ (int)0x80808080;
          acc[r] = __builtin_amdgcn_mfma_i32_16x16x64_i8(ra[sn % 3], b, acc[r], 0, 0, 0);
          if (sn + D < STEPS) issue(sn % D, sn + D, tb);
          else issue(sn % D, sn + D - STEPS, tbn);
          __builtin_amdgcn_sched_barrier(0);   // (the loads stay where the ring puts them: hoisted, they spill)
        }
      float4 mc[PER];
#pragma unroll
      for (int r = 0; r < PER; ++r) {
        const int p = NCOL == 1 ? r : A * r + i;
        const float4 sc = lds[clg + p * 12], sh = lds[clg + p * 12 + 4];
        mc[r].x = __builtin_fmaf((float)acc[r][0], sc.x, sh.x);
        mc[r].y = __builtin_fmaf((float)acc[r][1], sc.y, sh.y);
        mc[r].z = __builtin_fmaf((float)acc[r][2], sc.z, sh.z);
        mc[r].w = __builtin_fmaf((float)acc[r][3], sc.w, sh.w);
        // (pinned where it is computed: the compiler would read every constant first)
        asm volatile("" : "+v"(mc[r].x), "+v"(mc[r].y), "+v"(mc[r].z), "+v"(mc[r].w));
      }
      __builtin_amdgcn_sched_barrier(0);
      if (NCOL == 1) {
#pragma unroll
        for (int r = 0; r < PER; ++r) m4[NCOL == 1 ? r : 0] = mc[r];
      } else {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          float f[PER], o[M];
#pragma unroll
          for (int r = 0; r < PER; ++r) f[r] = comp_of(mc[r], k);
          out_1d<A>(f, o);
#pragma unroll
          for (int r = 0; r < M; ++r) {
            // (pinned: left to the compiler the transform moves to the end and the requantized column stays live)
            asm volatile("" : "+v"(o[r]));
            T[k][r][NCOL == 1 ? 0 : i] = o[r];
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
    unsigned pk[M * M];
#pragma unroll
    for (int e = 0; e < M * M; ++e) pk[e] = 0u;
    // second dimension, output scale, rounding and packing, one channel after the other (interleaved, the four
    // transforms' intermediates do not fit the registers); output type and ReLU are chosen once per block of tiles
    auto finish = [&](auto out_c, auto relu_c) {
      constexpr int OUT = decltype(out_c)::value;
      constexpr bool RELU = decltype(relu_c)::value;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        float y[M * M];
        if (NCOL == 1) {
          float f[AA];
#pragma unroll
          for (int e = 0; e < AA; ++e) f[e] = comp_of(m4[NCOL == 1 ? e : 0], k);
          wino::tile_output<A>(f, y);
        } else {
#pragma unroll
          for (int r = 0; r < M; ++r) out_1d<A>(T[k][r], &y[M * r]);
        }
        pack_channel<OUT, A>(y, comp_of(bias, k), k, RELU, a.out_repS, a.out_z, SUM, old, pk);
#pragma unroll
        for (int e = 0; e < M * M; ++e) asm volatile("" : "+v"(pk[e]));
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    using U8C = std::integral_constant<int, EHIP_U8>;
    using S8C = std::integral_constant<int, EHIP_S8>;
    if (!SUM && a.out_type == EHIP_F32) {
      float y[4][M * M];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        if (NCOL == 1) {
          float f[AA];
#pragma unroll
          for (int e = 0; e < AA; ++e) f[e] = comp_of(m4[NCOL == 1 ? e : 0], k);
          wino::tile_output<A>(f, y[k]);
        } else {
#pragma unroll
          for (int r = 0; r < M; ++r) out_1d<A>(T[k][r], &y[k][M * r]);
        }
        finish_channel_f32<A>(y[k], comp_of(bias, k), a.with_bias != 0, a.with_relu != 0);
#pragma unroll
        for (int e = 0; e < M * M; ++e) asm volatile("" : "+v"(y[k][e]));
        __builtin_amdgcn_sched_barrier(0);
      }
      // (plane: the block's offset in elements, worked out on the byte pointer)
      store_f32<A>(y, static_cast<float *>(a.out) + (plane - static_cast<uint8_t *>(a.out)), g, valid, th, tw, a.oh, a.ow, px);
    } else {
      if (a.out_type == EHIP_U8) {
        if (a.with_relu) finish(U8C{}, std::true_type{});
        else finish(U8C{}, std::false_type{});
      } else {
        if (a.with_relu) finish(S8C{}, std::true_type{});
        else finish(S8C{}, std::false_type{});
      }
      store_cells<A>(pk, plane, g, valid, th, tw, a.oh, a.ow, px);
    }
    if (!more) break;
    item = next;
    tb = tbn;
  }
}

namespace {
// second dimension of Y = At M A from the first-stage results T[channel][row][column], then output scale, rounding,
// packing and the store by cells (u8 / s8), or bias / ReLU and the 16-byte stores of f32 output: what the kernel above
// does at the end of a block of tiles, for the kernel below
template <int A, bool SUM>
__device__ __forceinline__ void finish_columns(const WinoFusedArgs &a, float (&T)[4][A - 2][A], const unsigned *old, const float4 &bias,
                                               uint8_t *plane, int g, bool valid, int th, int tw, int px)
{
  constexpr int M = A - 2;
  if (!SUM && a.out_type == EHIP_F32) {
    float y[4][M * M];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
#pragma unroll
      for (int r = 0; r < M; ++r) out_1d<A>(T[k][r], &y[k][M * r]);
      finish_channel_f32<A>(y[k], comp_of(bias, k), a.with_bias != 0, a.with_relu != 0);
#pragma unroll
      for (int e = 0; e < M * M; ++e) asm volatile("" : "+v"(y[k][e]));
      __builtin_amdgcn_sched_barrier(0);
    }
    store_f32<A>(y, static_cast<float *>(a.out) + (plane - static_cast<uint8_t *>(a.out)), g, valid, th, tw, a.oh, a.ow, px);
    return;
  }
  unsigned pk[M * M];
#pragma unroll
  for (int e = 0; e < M * M; ++e) pk[e] = 0u;
  auto finish = [&](auto out_c, auto relu_c) {
    constexpr int OUT = decltype(out_c)::value;
    constexpr bool RELU = decltype(relu_c)::value;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      float y[M * M];
#pragma unroll
      for (int r = 0; r < M; ++r) out_1d<A>(T[k][r], &y[M * r]);
      pack_channel<OUT, A>(y, comp_of(bias, k), k, RELU, a.out_repS, a.out_z, SUM, old, pk);
#pragma unroll
      for (int e = 0; e < M * M; ++e) asm volatile("" : "+v"(pk[e]));
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  using U8C = std::integral_constant<int, EHIP_U8>;
  using S8C = std::integral_constant<int, EHIP_S8>;
  if (a.out_type == EHIP_U8) {
    if (a.with_relu) finish(U8C{}, std::true_type{});
    else finish(U8C{}, std::false_type{});
  } else {
    if (a.with_relu) finish(S8C{}, std::true_type{});
    else finish(S8C{}, std::false_type{});
  }
  store_cells<A>(pk, plane, g, valid, th, tw, a.oh, a.ow, px);
}
}  // namespace

// 512 input channels (tile sizes 6 and 5): the weights of 16 channels at every position are 295 / 205 KB, twice the LDS,
// but those of HALF the columns of M fit.  The workgroup (one per CU) therefore walks over its blocks of tiles twice:
// with the weights of the first columns it leaves the first-stage results of those columns -- (A - 2) floats per
// column and channel, a third of what the positions themselves would be -- in a.tpart, then stages the other columns'
// weights, walks again and finishes every block with both halves in hand.  What a lane parks it reads back itself,
// 16 bytes per lane and value in lane order.
// a.tpart: [a.ny][a.nx][NW][(A - 2) x C0][64 lanes] float4, C0 = columns of the first pass (wino_lanes_tpart_bytes).
template <int A, bool SUM, int NKS, int NW>
__global__ __launch_bounds__(64 * NW, 2) void k_wino_gemm_output_lanes_wres2(WinoFusedArgs a)
{
  static_assert(A == 6 || A == 5, "tile sizes with a column-wise transform");
  constexpr int TB = 64 * NW;
  constexpr int AA = A * A, M = A - 2;
  constexpr int C0 = (A + 1) / 2, C1 = A - C0;               // columns of the two passes
  constexpr int STEPS0 = C0 * A * NKS;
  constexpr int D = A == 6 ? (SUM ? 6 : 12) : 5;             // divides the steps of both passes
  static_assert(STEPS0 % D == 0 && (C1 * A * NKS) % D == 0, "ring");
  extern __shared__ float4 lds[];
  v4i *wl = reinterpret_cast<v4i *>(lds);   // [steps of the pass][4 units][16 packed rows] cells of 16 bytes
  float4 *cl = lds + STEPS0 * 64;           // [AA][3][4 quads of the workgroup's 16 rows]: scale, shift, compensation
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l16 = lane & 15, g = lane >> 4;
  const int xcd = blockIdx.x & 7, seq = blockIdx.x >> 3;
  const int by = seq % a.ny;
  const int slot = seq / a.ny;
  const int item_step = 8 * (int)(gridDim.x / (8u * a.ny));
  const int item0 = slot * 8 + xcd;
  if (item0 >= a.nx) return;          // whole workgroup
  const int oc0 = (by >> 1) * 32, h = by & 1;   // (the workgroup's 16 channels: see the kernel above)
  const int oc_real = a.oc2 * 16;
  const int nblk = (a.t + 31) >> 5;
  const long long t_pos = (long long)a.ic2 * 512;
  const long long t_blk = t_pos * AA;
  unsigned b_off[NKS];
#pragma unroll
  for (int ks = 0; ks < NKS; ++ks) {
    int u = 4 * ks + g;
    u = u < a.ic2 ? u : a.ic2 - 1;
    b_off[ks] = (unsigned)(u * 512 + ((wave & 1) * 16 + l16) * 16);
  }
  auto base_of = [&](int it) {
    int blk = (NW / 2) * it + (wave >> 1);
    blk = blk < nblk ? blk : nblk - 1;
    return a.tin + blk * t_blk;      // wave-uniform
  };
  const int oc = oc0 + 16 * h + 4 * g;   // the lane's four channels
  const bool oc_ok = oc < oc_real;
  float4 bias = make_float4(0.f, 0.f, 0.f, 0.f);
  if (a.with_bias && oc_ok) bias = *reinterpret_cast<const float4 *>(a.bias + oc);
  const int px = a.out_nhwc ? a.oc2 * 16 : 16;
  int wla = g * 16 + l16, clg = STEPS0 * 64 + g;   // the lane's cells of 16 bytes from the start of the LDS, opaque
  asm volatile("" : "+v"(wla), "+v"(clg));
  v4i rb[D];

  auto run_pass = [&](auto qc) {
    constexpr int Q = decltype(qc)::value;
    constexpr int CB = Q == 0 ? 0 : C0, CN = Q == 0 ? C0 : C1, STEPS = CN * A * NKS;
    // step sn of the pass = (column CB + i, row r, k-step ks) in that order; its position is A r + CB + i
    auto pos_of = [](int sn) { const int pr = sn / NKS; return A * (pr % A) + CB + pr / A; };
    auto issue = [&](int rs, int sn, const uint8_t *tb) {
      rb[rs] = *reinterpret_cast<const v4i *>(tb + pos_of(sn) * t_pos + b_off[sn % NKS]);
    };
    int item = item0;
    const uint8_t *tb = base_of(item);
#pragma unroll
    for (int k = 0; k < D; ++k) issue(k, k, tb);
    if (Q > 0) __syncthreads();   // every wave has left the first pass's weights
    {
      constexpr int NP = (STEPS * 64 + TB - 1) / TB;
      const long long w_pos = (long long)a.units_pad * a.ocpp * 16;
      v4i tmp[NP];
#pragma unroll
      for (int j = 0; j < NP; ++j) {
        int idx = tid + j * TB;
        idx = idx < STEPS * 64 ? idx : STEPS * 64 - 1;
        const int chunk = idx >> 4, cell = idx & 15;
        const int sn = chunk >> 2, u = chunk & 3;
        // (runtime step -> position: the same map as pos_of)
        const int pr = sn / NKS, ks = sn - NKS * pr;
        const int pp = A * (pr % A) + CB + pr / A;
        tmp[j] = *reinterpret_cast<const v4i *>(a.w + pp * w_pos +
                                                ((long long)(4 * ks + u) * a.ocpp + oc0 + 8 * (cell >> 2) + 4 * h + (cell & 3)) * 16);
      }
      constexpr int NC = Q == 0 ? (AA * 12 + TB - 1) / TB : 1;
      float4 cst[NC];
      if (Q == 0) {
#pragma unroll
        for (int j = 0; j < NC; ++j) {
          int idx = tid + j * TB;
          idx = idx < AA * 12 ? idx : AA * 12 - 1;
          const int p = idx / 12, rem = idx - 12 * p, arr = rem >> 2, gq = rem & 3;
          const float *src = arr == 0 ? a.scale : (arr == 1 ? a.shift : reinterpret_cast<const float *>(a.comp));
          cst[j] = *reinterpret_cast<const float4 *>(src + (long long)p * a.ocpp + oc0 + 16 * h + 4 * gq);
        }
      }
#pragma unroll
      for (int j = 0; j < NP; ++j) {
        const int idx = tid + j * TB;
        if (idx < STEPS * 64) wl[idx] = tmp[j];
      }
      if (Q == 0) {
#pragma unroll
        for (int j = 0; j < NC; ++j) {
          const int idx = tid + j * TB;
          if (idx < AA * 12) cl[idx] = cst[j];
        }
      }
    }
    __syncthreads();   // the pass's weights (and the constants) are in LDS; the waves run on their own from here
    for (;;) {
      const int next = item + item_step;
      const bool more = next < a.nx;                      // wave-uniform
      const uint8_t *tbn = base_of(more ? next : item);   // (the last block's tail requests its own head again: unused)
      const int t = item * (16 * NW) + wave * 16 + l16;
      const bool valid = t < a.t && oc_ok;
      const int tc = valid ? t : 0, occ = valid ? oc : 0;
      const int n = tc / a.nt;
      const int rem = tc - n * a.nt;
      const int th = rem / a.wt;
      const int tw = rem - th * a.wt;
      uint8_t *plane = static_cast<uint8_t *>(a.out) +
          (a.out_nhwc ? (size_t)n * a.oh * a.ow * a.oc2 * 16 + (occ >> 4) * 16 : ((size_t)n * a.oc2 + (occ >> 4)) * a.oh * a.ow * 16);
      // the lane's parked values of this block: [row][column of the first pass], one float4 (four channels) each
      float4 *park = a.tpart + ((((size_t)by * a.nx + item) * NW + wave) * (M * C0)) * 64 + lane;
      float T[4][M][A];
      unsigned old[M * M];
      if (Q == 1) {
#pragma unroll
        for (int r = 0; r < M; ++r)
#pragma unroll
          for (int i = 0; i < C0; ++i) {
            const float4 v = park[(size_t)(r * C0 + i) * 64];
            T[0][r][i] = v.x; T[1][r][i] = v.y; T[2][r][i] = v.z; T[3][r][i] = v.w;
          }
      }
      v4i ra[3];
      ra[0] = wl[wla + 0];
      ra[1] = wl[wla + 64];
#pragma unroll
      for (int i = 0; i < CN; ++i) {
        if (SUM && Q == 1 && i == CN - 1) load_old_cells<A>(old, plane, g, th, tw, a.oh, a.ow, px);
        v4i acc[A];
#pragma unroll
        for (int r = 0; r < A; ++r) {
          const float4 cf = lds[clg + (A * r + CB + i) * 12 + 8];
          acc[r] = v4i{__float_as_int(cf.x), __float_as_int(cf.y), __float_as_int(cf.z), __float_as_int(cf.w)};
        }
#pragma unroll
        for (int r = 0; r < A; ++r)
#pragma unroll
          for (int ks = 0; ks < NKS; ++ks) {
            const int sn = (i * A + r) * NKS + ks;
            if (sn + 2 < STEPS) ra[(sn + 2) % 3] = wl[wla + (sn + 2) * 64];   // the weights of the step after next
            const v4i b = rb[sn % D] ^ (int)0x80808080;
            acc[r] = __builtin_amdgcn_mfma_i32_16x16x64_i8(ra[sn % 3], b, acc[r], 0, 0, 0);
            if (sn + D < STEPS) issue(sn % D, sn + D, tb);
            else issue(sn % D, sn + D - STEPS, tbn);
            __builtin_amdgcn_sched_barrier(0);
          }
        float4 mc[A];
#pragma unroll
        for (int r = 0; r < A; ++r) {
          const int p = A * r + CB + i;
          const float4 sc = lds[clg + p * 12], sh = lds[clg + p * 12 + 4];
          mc[r].x = __builtin_fmaf((float)acc[r][0], sc.x, sh.x);
          mc[r].y = __builtin_fmaf((float)acc[r][1], sc.y, sh.y);
          mc[r].z = __builtin_fmaf((float)acc[r][2], sc.z, sh.z);
          mc[r].w = __builtin_fmaf((float)acc[r][3], sc.w, sh.w);
          asm volatile("" : "+v"(mc[r].x), "+v"(mc[r].y), "+v"(mc[r].z), "+v"(mc[r].w));
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          float f[A], o[M];
#pragma unroll
          for (int r = 0; r < A; ++r) f[r] = comp_of(mc[r], k);
          out_1d<A>(f, o);
#pragma unroll
          for (int r = 0; r < M; ++r) {
            asm volatile("" : "+v"(o[r]));
            T[k][r][CB + i] = o[r];
          }
          __builtin_amdgcn_sched_barrier(0);
        }
        if (Q == 0) {
          // the column's results are parked as they come
#pragma unroll
          for (int r = 0; r < M; ++r)
            park[(size_t)(r * C0 + i) * 64] = make_float4(T[0][r][i], T[1][r][i], T[2][r][i], T[3][r][i]);
        }
      }
      if (Q == 1) finish_columns<A, SUM>(a, T, old, bias, plane, g, valid, th, tw, px);
      if (!more) break;
      item = next;
      tb = tbn;
    }
  };
  run_pass(std::integral_constant<int, 0>{});
  run_pass(std::integral_constant<int, 1>{});
}

namespace {
template <int A, bool SUM>
auto pick_wres_nks(int nks64, int nw) -> void (*)(WinoFusedArgs)
{
  switch (nks64) {
    case 1: return k_wino_gemm_output_lanes_wres<A, SUM, 1>;
    case 2: return k_wino_gemm_output_lanes_wres<A, SUM, 2>;
    case 3: return nw == 8 ? k_wino_gemm_output_lanes_wres<A, SUM, 3, 8> : k_wino_gemm_output_lanes_wres<A, SUM, 3>;
    case 4: return nw == 8 ? k_wino_gemm_output_lanes_wres<A, SUM, 4, 8> : k_wino_gemm_output_lanes_wres<A, SUM, 4>;
    case 8:
      if (A == 4) return nw == 8 ? k_wino_gemm_output_lanes_wres<4, SUM, 8, 8> : k_wino_gemm_output_lanes_wres<4, SUM, 8>;
      // (two passes over half of the columns each)
      return nw == 8 ? k_wino_gemm_output_lanes_wres2<A == 4 ? 6 : A, SUM, 8, 8> : k_wino_gemm_output_lanes_wres2<A == 4 ? 6 : A, SUM, 8, 4>;
    default: return nullptr;
  }
}
auto pick_wres(int A, bool sum, int nks64, int nw) -> void (*)(WinoFusedArgs)
{
  if (A == 4) return sum ? pick_wres_nks<4, true>(nks64, nw) : pick_wres_nks<4, false>(nks64, nw);
  if (A == 5) return sum ? pick_wres_nks<5, true>(nks64, nw) : pick_wres_nks<5, false>(nks64, nw);
  return sum ? pick_wres_nks<6, true>(nks64, nw) : pick_wres_nks<6, false>(nks64, nw);
}
}  // namespace

namespace {
// 512 input channels with tile size 6 or 5, two passes with resident weights: pays when a workgroup has at least two
// blocks of 128 tiles to walk over (N = 64, fused stage: 512 -> 512 at 28 x 28 134 -> 113 us, at 14 x 14 36.6 -> 42.8 us,
// at 7 x 7 26.5 -> 31.2 us), else the general kernel stays
bool two_pass_pays(int tile, int ic2, int oc2, int t)
{
  const int A = tile ? tile : 6, nks64 = (ic2 + 3) / 4;
  if (A == 4 || nks64 != 8) return false;
  if (const char *env = getenv("EHIP_WINO_LANES_TWO_PASS")) return env[0] != '0';   // (1: also for the small layers)
  const long long ny = 2 * ((oc2 * 16 + 31) / 32);
  // (and the parking space stays below 1 GB: beyond, the general kernel)
  if (ny * ((t + 127) / 128 * 128) * (long long)(A - 2) * ((A + 1) / 2) * 64 > (1ll << 30)) return false;
  return (long long)((t + 127) / 128) * ny >= 512;
}
}  // namespace

size_t wino_lanes_tpart_bytes(int tile, int ic2, int oc2, int t)
{
  const int A = tile ? tile : 6;
  if (!two_pass_pays(tile, ic2, oc2, t)) return 0;
  const char *env = getenv("EHIP_WINO_LANES");
  if (env && env[0] == '0') return 0;
  // per tile and group of 16 channels: (A - 2) rows x the first pass's columns x 16 channels x 4 bytes (four lanes with
  // a float4 each); tiles in whole blocks of 128, channel groups of whole 32s
  const size_t per_tile = (size_t)(A - 2) * ((A + 1) / 2) * 64;
  return (size_t)2 * ((oc2 * 16 + 31) / 32) * ((t + 127) / 128 * 128) * per_tile;
}

bool wino_lanes_applies(const WinoFusedArgs &a)
{
  const char *env = getenv("EHIP_WINO_LANES");
  const int nks64 = (a.ic2 + 3) / 4;
  // Measured at N = 64, u8 in / s8 out, against the general kernel (fused stage, us): 64 -> 64 at 56 x 56 28.5 vs 34.1, at
  // 224 x 224 370 vs 459; 128 -> 128 at 112 x 112 238 vs 300; 128 -> 256 at 56 x 56 107 vs 133; 256 -> 256 at 56 x 56 164 vs 171;
  // 512 -> 512 at 28 x 28 (eight k-steps per position, 288 unrolled steps) 648 vs 134: up to 256 input channels.
  const int A = a.tile ? a.tile : 6;
  // the weights of 16 channels at every position must fit the LDS (the streamed form: 1, 2 or 4 k-steps)
  // (tile sizes 6 and 5 with 512 channels: half the columns at a time, results parked in a.tpart)
  const bool fits = nks64 <= 4 || (A == 4 && nks64 == 8) || (two_pass_pays(a.tile, a.ic2, a.oc2, a.t) && a.tpart != nullptr);
  return a.tin_blocked && fits && a.units_pad % 4 == 0 && a.units_pad >= 4 * nks64 && !(a.out_type == EHIP_F32 && a.with_sum) &&
      !(env && env[0] == '0');
}

hipError_t launch_wino_gemm_output_lanes(const WinoFusedArgs &a0, hipStream_t s, LaunchPlan<WinoFusedArgs> *plan)
{
  WinoFusedArgs a = a0;
  const int A = a.tile ? a.tile : 6, AA = A * A;
  const int nks64 = (a.ic2 + 3) / 4;
  void (*kernel)(WinoFusedArgs) = nullptr;
  const char *env = getenv("EHIP_WINO_LANES_WRES");
  if (!(env && env[0] == '0') || nks64 == 3 || nks64 > 4) {   // (the streamed form below has 1, 2 and 4 k-steps only)
    // weights resident: the weights of 16 channels in LDS, workgroups walking over blocks of tiles.  Up to 128 input
    // channels: four waves, 64 tiles a block, two workgroups per CU; 256: the weights fill the LDS (tile size 6: 147 KB),
    // one workgroup per CU, of eight waves (128 tiles a block) so that every SIMD still has two
    const bool two_pass = A != 4 && nks64 == 8;   // the weights of half the columns at a time
    const size_t lds = (two_pass ? (size_t)((A + 1) / 2) * A : (size_t)AA) * nks64 * 1024 + (size_t)AA * 12 * sizeof(float4);
    const int per_cu = 2 * lds <= 160 * 1024 ? 2 : 1;
    const char *wv = getenv("EHIP_WINO_LANES_WAVES");
    a.ny = 2 * ((a.oc2 * 16 + 31) / 32);
    // (eight waves where that still gives every CU a workgroup: 256 -> 256 at 56 x 56 104 -> 89 us, at 14 x 14 14.5 -> 15.8 us)
    int nw = per_cu == 1 && (long long)((a.t + 127) / 128) * a.ny >= 256 ? 8 : 4;
    if (wv) nw = wv[0] == '8' && nks64 >= 3 ? 8 : 4;
    a.nx = (a.t + 16 * nw - 1) / (16 * nw);
    int slots = 32 * per_cu / a.ny;   // 8 XCDs x ny x slots ~ 256 workgroups per workgroup a CU holds
    if (const char *sl = getenv("EHIP_WINO_LANES_SLOTS")) slots = atoi(sl);   // (fewer: more blocks of tiles per workgroup)
    slots = slots < 1 ? 1 : slots;
    const int need = (a.nx + 7) / 8;
    slots = slots < need ? slots : need;
    kernel = pick_wres(A, a.with_sum != 0, nks64, nw);
    if (!kernel) return hipErrorInvalidValue;
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    const hipError_t rc = plan_launch(plan, kernel, dim3(8 * a.ny * slots), dim3(64 * nw), lds, a, s);
    if (plan && rc == hipSuccess) plan->name = "k_wino_gemm_output_lanes_wres";
    return rc;
  }
  a.nx = (a.t + 31) / 32;
  a.ny = (a.oc2 * 16 + 31) / 32;
#define EHIP_WL(AV)                                                                                                    \
  kernel = a.with_sum ? (nks64 == 1 ? k_wino_gemm_output_lanes<AV, true, 1>                                             \
                                    : (nks64 == 2 ? k_wino_gemm_output_lanes<AV, true, 2> : k_wino_gemm_output_lanes<AV, true, 4>)) \
                      : (nks64 == 1 ? k_wino_gemm_output_lanes<AV, false, 1>                                            \
                                    : (nks64 == 2 ? k_wino_gemm_output_lanes<AV, false, 2> : k_wino_gemm_output_lanes<AV, false, 4>))
  if (A == 4) EHIP_WL(4);
  else if (A == 5) EHIP_WL(5);
  else EHIP_WL(6);
#undef EHIP_WL
  const size_t lds = (size_t)AA * 24 * sizeof(float4);
  const hipError_t rc = plan_launch(plan, kernel, dim3(8 * a.ny * ((a.nx + 7) / 8)), dim3(kBlock), lds, a, s);
  if (plan && rc == hipSuccess) plan->name = "k_wino_gemm_output_lanes";
  return rc;
}

}  // namespace ehip
