// Depthwise 3x3 u8 x s8 convolution (stride 1 and 2) with fused requantization: a bandwidth kernel.
//
// Replaces elx_int8_conv_direct_depthwise_t::__execute_c160 + conv_c160
// (src/elx_int8_conv_direct_depthwise_xopt.hpp:19-66, src/elx_int8_conv_direct_depthwise.cpp:294-319)
// and the depthwise micro-kernel (src/kernel/elk_u8s8_depthwise_conv.hxx:219-474).
//
// There is no contraction over channels, so the matrix cores have nothing to do; the work is
// 1 byte in + 1 byte out per 9 multiply-adds and the kernel has to keep the VALU cost per byte
// below what HBM can deliver.  A lane owns 4 channels (one dword of a 16-channel cell) x 2 output
// columns x RB output rows.  Per input row it loads the 4 pixels its two columns touch (4 dwords;
// the 4 lanes of a cell read 16 contiguous bytes), flips the top bits (u8 -> s8, undone by the
// 128 * sum(w) the accumulators start from; out-of-image pixels count as u8 0), and byte-transposes
// the 4 pixels x 4 channels block with 8 v_perm_b32 so that one dword holds the four horizontally
// adjacent pixels of ONE channel.  The three taps of a kernel row are then a single v_dot4_i32_i8
// against weights packed [kh][channel][kw0 kw1 kw2 0] -- and the same dword serves the second
// column against the weights shifted by one byte.  The packed layout is the reference's own
// ([g/16][kh][16][KW=4], src/elx_int8_conv_direct_depthwise.cpp:224-236).
//
// Stride 2 (the micro-kernel's S template parameter, src/kernel/elk_u8s8_depthwise_conv.hxx:371-403):
// the lane's two output columns sit two input pixels apart, so a fifth pixel is loaded and one more
// v_perm_b32 per channel splices it behind pixels 2 and 3 of the transposed dword; an output row
// reads input rows 2r .. 2r + 2.
//
// The u8 store reproduces the reference's width-block rule: inside every block of T output columns
// (Tr for the last block) the columns before 4*floor(Tz/4) are rounded toward -infinity and
// byte-merged without saturation, the remaining ones are rounded to nearest even and saturated.
#include "ehip_internal.hpp"

namespace ehip {

namespace {
// v_perm_b32: result byte i = byte sel[i] of the 8-byte pool {hi: 4..7, lo: 0..3}
__device__ __forceinline__ unsigned perm(unsigned hi, unsigned lo, unsigned sel)
{
  return __builtin_amdgcn_perm(hi, lo, sel);
}
// Raw buffer access: a 32-bit byte offset into [base, base + bytes); an offset outside that range is not an
// error -- a load returns zeros and a store is dropped.
#if defined(__HIP_DEVICE_COMPILE__)
typedef __amdgpu_buffer_rsrc_t BufferRsrc;
__device__ __forceinline__ BufferRsrc make_rsrc(const void *base, unsigned bytes)
{
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), (short)0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ uint4 buffer_load_16(BufferRsrc r, unsigned off)
{
  typedef unsigned v4u __attribute__((ext_vector_type(4)));
  const v4u v = __builtin_amdgcn_raw_buffer_load_b128(r, (int)off, 0, 0);
  return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void buffer_store_8(BufferRsrc r, unsigned off, uint2 v)
{
  typedef unsigned v2u __attribute__((ext_vector_type(2)));
  const v2u d = {v.x, v.y};
  // non-temporal (the line is not kept in L2): C5a 13.6 -> 12.3 us
  __builtin_amdgcn_raw_buffer_store_b64(d, r, (int)off, 0, 2);
}
__device__ __forceinline__ void wait_vmem() { __builtin_amdgcn_s_waitcnt(0x0f70); }   // vmcnt(0)
#else   // the host pass only needs the names
typedef int BufferRsrc;
__device__ inline void wait_vmem() {}
__device__ inline BufferRsrc make_rsrc(const void *, unsigned) { return 0; }
__device__ inline uint4 buffer_load_16(BufferRsrc, unsigned) { return uint4(); }
__device__ inline void buffer_store_8(BufferRsrc, unsigned, uint2) {}
#endif

// lanes 0-31 get {their x, x of lane + 32}; lanes 32-63 get {y of lane - 32, their y}
__device__ __forceinline__ uint2 swap_halves(unsigned x, unsigned y)
{
#if defined(__HIP_DEVICE_COMPILE__)
  const auto r = __builtin_amdgcn_permlane32_swap(x, y, false, false);
  return make_uint2(r[0], r[1]);
#else
  return make_uint2(x, y);
#endif
}
}  // namespace

// MODE 0: any output type / bounds.  MODE 1: u8 output, ReLU with 0 <= lo <= hi <= 255 (floor and
// round-to-nearest both land in the code range, so the pack-with-saturation instruction, which
// rounds to nearest even itself, finishes either).  MODE 2: as 1 with lo == 0 and hi == 255, where
// the clamp is the instruction's own saturation.
// Both kernels take what a wave's first loads need -- three pointers and the geometry the addresses are made of,
// packed into 16 dwords -- as leading scalar arguments, which the dispatcher preloads into scalar registers with
// the wave (the file is compiled with -amdgpu-kernarg-preload-count=16); the rest of the argument block is loaded
// as usual meanwhile.  ihw = ih | iw << 16, ohw = oh | ow << 16, geom = pad_t | pad_l << 8 | stride << 16,
// ppb_lp = planes_per_block | lanes_padded << 16.
#define EHIP_DW_HEAD                                                                                                   \
  const uint8_t *in_, const int8_t *w_, const int *wsum_, int n_, int g2_, unsigned ihw_, unsigned ohw_, unsigned geom_, \
      int blocks_per_plane_, int lanes_per_plane_, unsigned ppb_lp_, unsigned wp_magic_, int strips_per_wg_
#define EHIP_DW_UNPACK                                                                                                 \
  DepthwiseArgs a = rest;                                                                                              \
  a.in = in_; a.w = w_; a.wsum = wsum_; a.n = n_; a.g2 = g2_; a.ih = (int)(ihw_ & 0xffffu); a.iw = (int)(ihw_ >> 16);  \
  a.oh = (int)(ohw_ & 0xffffu); a.ow = (int)(ohw_ >> 16); a.pad_t = (int)(geom_ & 0xffu);                              \
  a.pad_l = (int)((geom_ >> 8) & 0xffu); a.stride = (int)(geom_ >> 16); a.blocks_per_plane = blocks_per_plane_;        \
  a.lanes_per_plane = lanes_per_plane_; a.planes_per_block = (int)(ppb_lp_ & 0xffffu);                                 \
  a.lanes_padded = (int)(ppb_lp_ >> 16); a.wp_magic = wp_magic_; a.strips_per_wg = strips_per_wg_
template <int RB, int MODE, int S>
__global__ __launch_bounds__(kBlock) void k_depthwise3x3_u8s8(EHIP_DW_HEAD, DepthwiseArgs rest)
{
  EHIP_DW_UNPACK;
  constexpr int NPX = S == 1 ? 4 : 5;          // input pixels per row a lane touches
  constexpr int NROWS = S * (RB - 1) + 3;      // input rows
  // A plane (one image x one 16-channel block) is split into blocks over its lanes (q fastest, then
  // column pair, then row block).  Workgroups go round the eight XCDs (block b runs on XCD b % 8), each
  // with an L2 of its own, and neighbouring row blocks share two input rows: so all blocks of a plane
  // are given to ONE XCD, one after the other -- plane = 8 * (seq / blocks_per_plane) + xcd.
  // Small planes (7 x 7: 64 lanes) share a workgroup, planes_per_block of them, each on whole waves of its
  // own: one-wave workgroups by the ten thousand are bound by the rate at which workgroups are dispatched.
  const int xcd = blockIdx.x & 7, seq = blockIdx.x >> 3;
  const int pgrp = seq / a.blocks_per_plane;
  const int sub = a.planes_per_block > 1 ? (int)threadIdx.x / a.lanes_padded : 0;   // wave-uniform
  const int plane_id = (pgrp * 8 + xcd) * a.planes_per_block + sub;
  if (plane_id >= a.n * a.g2) return;   // whole waves
  const int wp = (a.ow + 1) >> 1;
  const int local = a.planes_per_block > 1 ? (int)threadIdx.x - sub * a.lanes_padded
                                           : (seq - pgrp * a.blocks_per_plane) * (int)blockDim.x + (int)threadIdx.x;
  if (local >= a.lanes_per_plane) return;
  const int q = local & 3;
  const int hb = fastdiv(local >> 2, wp, a.wp_magic);
  const int p = (local >> 2) - hb * wp;
  const int g2 = plane_id % a.g2;
  const unsigned ng = plane_id;   // image * g2 + channel block
  const int oh0 = hb * RB;
  const int c0 = 2 * p;
  const int ch0 = g2 * 16 + 4 * q;  // first of the lane's 4 channels

  // weights: [g2][kh][16][4] -> per kh one dword per channel (kw0 kw1 kw2 0); second column: << 8
  unsigned wa[3][4], wb[3][4];
#pragma unroll
  for (int kh = 0; kh < 3; ++kh) {
    const uint4 w4 = *reinterpret_cast<const uint4 *>(a.w + (((size_t)g2 * 3 + kh) * 16 + 4 * q) * 4);
    wa[kh][0] = w4.x; wa[kh][1] = w4.y; wa[kh][2] = w4.z; wa[kh][3] = w4.w;
#pragma unroll
    for (int j = 0; j < 4; ++j) wb[kh][j] = wa[kh][j] << 8;
  }
  const v4i ws = *reinterpret_cast<const v4i *>(a.wsum + ch0);

  int acc[RB][2][4];
#pragma unroll
  for (int r = 0; r < RB; ++r)
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      acc[r][c][0] = 128 * ws.x; acc[r][c][1] = 128 * ws.y; acc[r][c][2] = 128 * ws.z; acc[r][c][3] = 128 * ws.w;
    }

  // the 4 input columns of this lane (clamped; invalid ones are replaced after the load); all
  // addresses are 32-bit byte offsets from the tensor base (the launcher checks the size)
  unsigned coloff[NPX];
  bool colok[NPX];
#pragma unroll
  for (int k = 0; k < NPX; ++k) {
    const int iw = S * c0 - a.pad_l + k;
    colok[k] = iw >= 0 && iw < a.iw;
    coloff[k] = (unsigned)(iw < 0 ? 0 : (iw >= a.iw ? a.iw - 1 : iw)) * 16u;
  }
  const unsigned plane_off = ng * (unsigned)(a.ih * a.iw) * 16u + 4u * q;
  const char *in_base = reinterpret_cast<const char *>(a.in);

#pragma unroll
  for (int hr = 0; hr < NROWS; ++hr) {
    const int ih = S * oh0 - a.pad_t + hr;
    const bool rowok = ih >= 0 && ih < a.ih;
    const int ihc = ih < 0 ? 0 : (ih >= a.ih ? a.ih - 1 : ih);
    const unsigned row_off = plane_off + (unsigned)(ihc * a.iw) * 16u;
    unsigned x[NPX];
#pragma unroll
    for (int k = 0; k < NPX; ++k) {
      const unsigned v = *reinterpret_cast<const unsigned *>(in_base + (size_t)(row_off + coloff[k]));
      x[k] = (rowok && colok[k]) ? v ^ 0x80808080u : 0x80808080u;
    }
    // 4 pixels x 4 channels -> 4 channels x 4 pixels
    const unsigned a0 = perm(x[1], x[0], 0x05010400u), a1 = perm(x[1], x[0], 0x07030602u);
    const unsigned b0 = perm(x[3], x[2], 0x05010400u), b1 = perm(x[3], x[2], 0x07030602u);
    unsigned t[4];
    t[0] = perm(b0, a0, 0x05040100u);
    t[1] = perm(b0, a0, 0x07060302u);
    t[2] = perm(b1, a1, 0x05040100u);
    t[3] = perm(b1, a1, 0x07060302u);
    // second column, stride 2: pixels 2, 3, 4 of channel j = bytes 2, 3 of t[j] and byte j of x[4]
    unsigned t2[4];
    if (S == 2) {
#pragma unroll
      for (int j = 0; j < 4; ++j) t2[j] = perm(x[NPX - 1], t[j], 0x00040302u + ((unsigned)j << 16));
    }
#pragma unroll
    for (int r = 0; r < RB; ++r) {
      const int kh = hr - S * r;  // input row ih feeds output row oh0 + r through kernel row kh
      if (kh < 0 || kh > 2) continue;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        acc[r][0][j] = __builtin_amdgcn_sdot4((int)t[j], (int)wa[kh][j], acc[r][0][j], false);
        if (S == 1) acc[r][1][j] = __builtin_amdgcn_sdot4((int)t[j], (int)wb[kh][j], acc[r][1][j], false);
        else acc[r][1][j] = __builtin_amdgcn_sdot4((int)t2[j], (int)wa[kh][j], acc[r][1][j], false);
      }
    }
  }

  const float4 sc = *reinterpret_cast<const float4 *>(a.scale + ch0);
  const float4 sh = *reinterpret_cast<const float4 *>(a.shift + ch0);
  const float scv[4] = {sc.x, sc.y, sc.z, sc.w}, shv[4] = {sh.x, sh.y, sh.z, sh.w};
  const bool relu = a.with_relu != 0;

#pragma unroll
  for (int c = 0; c < 2; ++c) {
    const int ow = c0 + c;
    if (ow >= a.ow) break;
    // width-block rule for this column
    const int blk = fastdiv(ow, a.T, a.T_magic);
    const int tpos = ow - blk * a.T;
    const int Tz = blk == a.wt - 1 ? a.Tr : a.T;
    const bool floor_col = a.out_type == EHIP_U8 && tpos < 4 * (Tz / 4);
#pragma unroll
    for (int r = 0; r < RB; ++r) {
      const int oh = oh0 + r;
      if (oh >= a.oh) break;
      const unsigned cell = (ng * (unsigned)a.oh + oh) * (unsigned)a.ow + ow;   // < 2^28, checked by the launcher
      if (MODE == 0 && a.out_type == EHIP_S32) {
        reinterpret_cast<v4i *>(a.out)[(size_t)cell * 4 + q] = v4i{acc[r][c][0], acc[r][c][1], acc[r][c][2], acc[r][c][3]};
        continue;
      }
      unsigned o = 0u;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        float f = __builtin_fmaf((float)acc[r][c][j], scv[j], shv[j]);
        if (MODE == 0) {
          if (relu) f = __builtin_fminf(__builtin_fmaxf(f, a.lo), a.hi);
          unsigned qv;
          if (floor_col) {
            const int fl = (!(f >= -2147483648.0f && f < 2147483648.0f)) ? (int)0x80000000 : (int)__builtin_floorf(f);
            qv = (unsigned)fl & 0xffu;
          } else if (a.out_type == EHIP_U8) {
            qv = usat8((unsigned)cvt_s32_rne(f));
          } else {
            qv = (unsigned)ssat8(cvt_s32_rne(f)) & 0xffu;
          }
          o |= qv << (8 * j);
        } else {
          if (MODE == 1) f = __builtin_fminf(__builtin_fmaxf(f, a.lo), a.hi);
          const float fl = __builtin_floorf(f);
          f = floor_col ? fl : f;
          o = __builtin_amdgcn_cvt_pk_u8_f32(f, j, o);
        }
      }
      *reinterpret_cast<unsigned *>(static_cast<char *>(a.out) + (size_t)(cell * 16u + 4u * q)) = o;
    }
  }
}

// ---- stride 1 on the matrix cores ---------------------------------------------------------------
// The dot4 kernel above is bound by vector-instruction issue (transposes, one dot per kernel row and
// output, the epilogue): about 17 lane-instructions per output byte.  v_mfma_i32_32x32x32_i8 takes the
// nChw16c cell as it lies in memory: with K = (two pixels) x (16 channels) and A = the weights of one
// kernel column spread on a diagonal (row c, byte c = w[c][kh][kw], everything else zero), one
// instruction multiplies 32 pixels x 16 channels x 2 taps for two output rows at once -- rows 0-15 of
// the result are the channels of one output row, rows 16-31 those of the row above.  97 % of the
// multiplies hit zeros; the instruction still does in 32 clocks what takes the vector unit 24 dot
// instructions plus 16 byte permutes, and there is nothing left to transpose.  The arithmetic is the
// same exact s32 sum (u8 as s8 via ^0x80, accumulators start from 128 * sum(w)); the epilogue and the
// width-block rule of the u8 store are those of the kernel above.
//
// The unit of work is a strip of R = 8 output rows of one plane: R + 2 input rows (zero frame included,
// flipped to s8) staged in LDS, the six diagonal weight matrices (2 row pairings x 3 kernel columns, built
// at weight preparation) as A operands, one pair of output rows per wave: per chunk of 32 columns
//   pairing 1: B = input rows (a, a + 1):   out[a+1] += kh0, kh1;   out[a] += kh1, kh2
//   pairing 2: B = input rows (a - 1, a + 2): out[a] += kh0 (first half);  out[a+1] += kh2 (second half)
// (a = the input row under output row a's centre tap), three kernel columns each = 6 MFMAs for
// 2 x 32 x 16 outputs.  An accumulator lane holds 8 channels of one pixel for both rows; the two
// half-waves swap a dword (v_permlane32_swap) so that every lane stores 8 contiguous bytes.
// A workgroup walks a run of consecutive strips and keeps the memory pipe busy while it computes: the
// next strip's rows are loaded into registers before the current strip's MFMAs start, and go to the
// other half of a double LDS buffer once the arithmetic is done (one barrier per strip).  A layer this short (57.8 MB,
// 9 us for a plain copy) has no time for workgroups that load, compute and store one after the other.
template <int MODE, int NC>
__global__ __launch_bounds__(kBlock) void k_depthwise3x3_mfma(EHIP_DW_HEAD, DepthwiseArgs rest)
{
  EHIP_DW_UNPACK;
  constexpr int R = 8, WL = 32 * NC + 2, CELLS = (R + 2) * WL, PER = (CELLS + kBlock - 1) / kBlock;
  constexpr unsigned kNowhere = 0xffffff00u;   // an offset past the end of every tensor: loads give 0, stores vanish
  __shared__ uint4 tile[2][CELLS];
  const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, lh = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // strips [first, last) of this workgroup: XCD x (workgroups x, x + 8, ...) walks the x-th eighth of all
  // strips, a workgroup a contiguous run of it -- neighbouring strips share two input rows in that XCD's L2
  const int per_xcd = gridDim.x >> 3;
  const int w_lin = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  const int first = w_lin * a.strips_per_wg;
  const int total = a.n * a.g2 * a.blocks_per_plane;    // blocks_per_plane = strips per plane
  const int last = first + a.strips_per_wg < total ? first + a.strips_per_wg : total;
  if (first >= last) return;
  const BufferRsrc rin = make_rsrc(a.in, (unsigned)(a.n * a.g2) * (unsigned)(a.ih * a.iw) * 16u);
  const BufferRsrc rout = make_rsrc(a.out, (unsigned)(a.n * a.g2) * (unsigned)(a.oh * a.ow) * 16u);

  // what a thread stages never changes: cells tid, tid + 256, ... of the (R + 2) x WL tile
  int cell_lr[PER], cell_off[PER];
  bool cell_colok[PER];
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    const int idx = tid + k * kBlock;
    const int lr = idx / WL, lc = idx - lr * WL;
    const int iw = lc - a.pad_l;
    cell_lr[k] = lr - a.pad_t;
    cell_colok[k] = idx < CELLS && iw >= 0 && iw < a.iw;
    cell_off[k] = (cell_lr[k] * a.iw + iw) * 16;
  }
  // Every load and store of the loop is issued unconditionally -- what must not happen is sent to an
  // offset outside the buffer, where a load returns the zero frame and a store is dropped.
  uint4 stage[PER];
  auto fetch = [&](int item) {   // input rows oh0 - pad_t .. + R + 1 of the strip's plane, into registers
    const int plane = item / a.blocks_per_plane;
    const int oh0 = (item - plane * a.blocks_per_plane) * R;
    const unsigned base = ((unsigned)plane * (unsigned)(a.ih * a.iw) + (unsigned)(oh0 * a.iw)) * 16u;
#pragma unroll
    for (int k = 0; k < PER; ++k) {
      const int ih = oh0 + cell_lr[k];
      const bool ok = cell_colok[k] && ih >= 0 && ih < a.ih;
      stage[k] = buffer_load_16(rin, ok ? base + (unsigned)cell_off[k] : kNowhere);
    }
  };
  auto hand_over = [&](int buf) {   // flip to s8 and put the strip where the waves read it
#pragma unroll
    for (int k = 0; k < PER; ++k) {
      uint4 v = stage[k];
      v.x ^= 0x80808080u; v.y ^= 0x80808080u; v.z ^= 0x80808080u; v.w ^= 0x80808080u;
      if (tid + k * kBlock < CELLS) tile[buf][tid + k * kBlock] = v;
    }
  };

  // width-block rule of the u8 store for the lane's column of every chunk
  bool floor_col[NC];
#pragma unroll
  for (int ck = 0; ck < NC; ++ck) {
    const int col = 32 * ck + l32;
    const int blk = fastdiv(col, a.T, a.T_magic);
    const int tpos = col - blk * a.T;
    const int Tz = blk == a.wt - 1 ? a.Tr : a.T;
    floor_col[ck] = tpos < 4 * (Tz / 4);
  }

  v4i wa[6];
  v16i comp;   // what the accumulators start from: 128 * sum(w) of the row's channel, the C operand of the first MFMA
  float scv[8], shv[8];
  int g2_now = -1;
  fetch(first);
  hand_over(0);
  // Loads and stores of a wave complete out of order with each other, so a wait for loads is a wait for
  // every store issued before it as well.  The order below gives each strip's stores a whole strip of
  // arithmetic to drain before the next such wait: barrier, next strip's loads, this strip's MFMAs and
  // epilogue arithmetic, wait + hand-over of the next strip, then this strip's stores.
  for (int item = first; item < last; ++item) {
    const int buf = (item - first) & 1;
    const int plane = item / a.blocks_per_plane;
    const int oh0 = (item - plane * a.blocks_per_plane) * R;
    const int g2 = plane % a.g2;
    __syncthreads();   // the only barrier of a strip: tile[buf] is complete, tile[buf ^ 1] was last read a strip ago
    if (g2 != g2_now) {   // uniform and rare (a new plane): the unit's diagonal weight matrices and constants
      g2_now = g2;
#pragma unroll
      for (int m = 0; m < 6; ++m) wa[m] = *reinterpret_cast<const v4i *>(a.wdiag + ((size_t)g2 * 6 + m) * 64 + lane);
      const int ch0 = g2 * 16 + 4 * lh;   // the lane's 8 channels: 4 lh .. + 3 and 8 + 4 lh .. + 3
      const v4i ws0 = *reinterpret_cast<const v4i *>(a.wsum + ch0), ws1 = *reinterpret_cast<const v4i *>(a.wsum + ch0 + 8);
      const float4 sc0 = *reinterpret_cast<const float4 *>(a.scale + ch0), sc1 = *reinterpret_cast<const float4 *>(a.scale + ch0 + 8);
      const float4 sh0 = *reinterpret_cast<const float4 *>(a.shift + ch0), sh1 = *reinterpret_cast<const float4 *>(a.shift + ch0 + 8);
      wait_vmem();   // here, not at the first use: past this branch nothing of it is in flight
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        comp[v] = comp[8 + v] = 128 * ws0[v];
        comp[4 + v] = comp[12 + v] = 128 * ws1[v];
      }
      scv[0] = sc0.x; scv[1] = sc0.y; scv[2] = sc0.z; scv[3] = sc0.w; scv[4] = sc1.x; scv[5] = sc1.y; scv[6] = sc1.z; scv[7] = sc1.w;
      shv[0] = sh0.x; shv[1] = sh0.y; shv[2] = sh0.z; shv[3] = sh0.w; shv[4] = sh1.x; shv[5] = sh1.y; shv[6] = sh1.z; shv[7] = sh1.w;
    }
    fetch(item + 1 < last ? item + 1 : item);   // (the last strip fetches itself again: no branch around memory instructions)

    const int oa = oh0 + 2 * wave;      // the wave's output rows: oa (rows 16-31 of the result) and oa + 1 (rows 0-15)
    const unsigned out_plane = (unsigned)plane * (unsigned)(a.oh * a.ow) * 16u + 8u * lh;
    const v4i *t1 = reinterpret_cast<const v4i *>(tile[buf]) + (2 * wave + 1 + lh) * WL + l32;   // pairing 1: rows 2w+1, 2w+2
    const v4i *t2 = reinterpret_cast<const v4i *>(tile[buf]) + (2 * wave + 3 * lh) * WL + l32;   // pairing 2: rows 2w, 2w+3
    uint2 res[NC][2];
#pragma unroll
    for (int ck = 0; ck < NC; ++ck) {
      v16i acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(wa[0], t1[32 * ck], comp, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(wa[3], t2[32 * ck], acc, 0, 0, 0);
#pragma unroll
      for (int kw = 1; kw < 3; ++kw) {
        acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(wa[kw], t1[32 * ck + kw], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(wa[3 + kw], t2[32 * ck + kw], acc, 0, 0, 0);
      }
      float f[16];
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        f[v] = __builtin_fmaf((float)acc[v], scv[v & 7], shv[v & 7]);
        if (MODE == 1) f[v] = __builtin_fminf(__builtin_fmaxf(f[v], a.lo), a.hi);
      }
      if (floor_col[ck]) {
#pragma unroll
        for (int v = 0; v < 16; ++v) f[v] = __builtin_floorf(f[v]);
        asm volatile("" ::: "memory");   // keep this a branch: sixteen selects cost more than the skipped floors
      }
#pragma unroll
      for (int hi = 0; hi < 2; ++hi) {
        unsigned g0 = 0u, g1 = 0u;   // channels 4 lh .. + 3 and 8 + 4 lh .. + 3 of output row oa + 1 - hi
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          g0 = __builtin_amdgcn_cvt_pk_u8_f32(f[8 * hi + j], j, g0);
          g1 = __builtin_amdgcn_cvt_pk_u8_f32(f[8 * hi + 4 + j], j, g1);
        }
        // lanes 0-31 end with channels 0-7 of their pixel, lanes 32-63 with channels 8-15 of theirs
        res[ck][hi] = swap_halves(g0, g1);
      }
    }
    hand_over(buf ^ 1);   // waits for the next strip's rows (and, with them, for the previous strip's stores)
#pragma unroll
    for (int ck = 0; ck < NC; ++ck)
#pragma unroll
      for (int hi = 0; hi < 2; ++hi) {
        const int col = 32 * ck + l32, oh = oa + 1 - hi;
        const bool ok = col < a.ow && oh < a.oh;
        buffer_store_8(rout, ok ? out_plane + (unsigned)(oh * a.ow + col) * 16u : kNowhere, res[ck][hi]);
      }
  }
}

// The A operands of k_depthwise3x3_mfma: [g2][6 matrices][64 lanes] cells of 16 bytes.  Lane l of matrix m
// (m = 3 * pairing + kw) feeds row i = l % 32 of A -- channel c = i % 16 of output row a + 1 - i / 16 -- with
// the K bytes of input-row half h = l / 32: all zero except byte c, the weight of kernel row kh and column kw.
// Pairing 1 (input rows a, a + 1): kh = h + i / 16.  Pairing 2 (input rows a - 1, a + 2): only the first half
// for output row a (kh 0) and the second half for output row a + 1 (kh 2) are non-zero.
__global__ __launch_bounds__(kBlock) void k_depthwise_diag(const int8_t *w, int g2n, uint4 *diag)
{
  const int idx = blockIdx.x * kBlock + threadIdx.x;
  if (idx >= g2n * 6 * 64) return;
  const int l = idx & 63, m = (idx >> 6) % 6, g2 = idx / (6 * 64);
  const int type = m >= 3 ? 1 : 0, kw = m - 3 * type;
  const int i = l & 31, h = l >> 5, c = i & 15, hi = i >> 4;
  const bool live = type == 0 || (h ^ hi) == 1;
  const int kh = type == 0 ? h + hi : 2 * h;
  const unsigned wv = live ? (unsigned)(uint8_t)w[(((size_t)g2 * 3 + kh) * 16 + c) * 4 + kw] : 0u;
  const unsigned dw = wv << (8 * (c & 3));
  uint4 cell;
  cell.x = (c >> 2) == 0 ? dw : 0u;
  cell.y = (c >> 2) == 1 ? dw : 0u;
  cell.z = (c >> 2) == 2 ? dw : 0u;
  cell.w = (c >> 2) == 3 ? dw : 0u;
  diag[idx] = cell;
}

hipError_t launch_depthwise_diag(const int8_t *wpacked, int g2n, void *diag, hipStream_t s)
{
  hipLaunchKernelGGL(k_depthwise_diag, dim3((g2n * 6 * 64 + kBlock - 1) / kBlock), dim3(kBlock), 0, s, wpacked, g2n,
                     static_cast<uint4 *>(diag));
  return hipGetLastError();
}

namespace {
typedef void (*dw_kernel_t)(EHIP_DW_HEAD, DepthwiseArgs);
hipError_t dw_enqueue(const LaunchPlan<DepthwiseArgs> &plan, hipStream_t s)
{
  const DepthwiseArgs &a = plan.args;
  hipLaunchKernelGGL(reinterpret_cast<dw_kernel_t>(plan.kernel), plan.grid, plan.block, plan.lds, s, a.in, a.w, a.wsum, a.n, a.g2,
                     (unsigned)a.ih | (unsigned)a.iw << 16, (unsigned)a.oh | (unsigned)a.ow << 16,
                     (unsigned)a.pad_t | (unsigned)a.pad_l << 8 | (unsigned)a.stride << 16, a.blocks_per_plane, a.lanes_per_plane,
                     (unsigned)a.planes_per_block | (unsigned)a.lanes_padded << 16, a.wp_magic, a.strips_per_wg, a);
  return hipGetLastError();
}
hipError_t dw_launch(LaunchPlan<DepthwiseArgs> *plan, dw_kernel_t kernel, dim3 grid, dim3 block, const DepthwiseArgs &a, hipStream_t s)
{
  // what the packed leading arguments can hold
  if (a.ih >= 65536 || a.iw >= 65536 || a.oh >= 65536 || a.ow >= 65536 || a.pad_t < 0 || a.pad_t > 255 || a.pad_l < 0 ||
      a.pad_l > 255 || a.planes_per_block >= 65536 || a.lanes_padded >= 65536) {
    set_error("depthwise: plane or padding too large");
    return hipErrorInvalidValue;
  }
  LaunchPlan<DepthwiseArgs> local;
  LaunchPlan<DepthwiseArgs> *p = plan ? plan : &local;
  p->kernel = reinterpret_cast<void (*)(DepthwiseArgs)>(kernel);
  p->grid = grid;
  p->block = block;
  p->lds = 0;
  p->args = a;
  p->enqueue = dw_enqueue;
  return plan_first_launch(p, s);
}
template <int RB, int S>
dw_kernel_t kernel_rbs(int mode)
{
  return mode == 2 ? k_depthwise3x3_u8s8<RB, 2, S> : (mode == 1 ? k_depthwise3x3_u8s8<RB, 1, S> : k_depthwise3x3_u8s8<RB, 0, S>);
}
template <int RB>
dw_kernel_t kernel_rb(int stride, int mode)
{
  return stride == 2 ? kernel_rbs<RB, 2>(mode) : kernel_rbs<RB, 1>(mode);
}
}  // namespace

// The matrix-core kernel: stride 1, u8 output with a ReLU inside the code range, pads 0 / 1, and a plane
// of up to four 32-column chunks whose chunks and 8-row strips are mostly real pixels (EHIP_DW_MFMA=0 / 1
// overrides the last condition).
bool depthwise_mfma_applies(int stride, int oh, int ow, int pad_t, int pad_l, int out_type, int with_relu, float lo, float hi,
                            long long planes, int ih, int iw)
{
  if (stride != 1 || out_type != EHIP_U8 || !with_relu || !(lo >= 0.0f && hi <= 255.0f && hi >= lo)) return false;
  if (pad_t < 0 || pad_t > 1 || pad_l < 0 || pad_l > 1 || ow > 128) return false;
  // the kernel addresses both tensors with 32-bit byte offsets and keeps the last 64 KB of that range as "nowhere";
  // a larger layer runs on the dot4 kernel
  if (planes * ((oh + 7) / 8) >= (1ll << 30) || planes * ih * iw * 16 >= (1ll << 32) - 65536 ||
      planes * oh * ow * 16 >= (1ll << 32) - 65536)
    return false;
  if (const char *env = getenv("EHIP_DW_MFMA")) return atoi(env) != 0;
  // measured (N = 64, with non-temporal output stores): ahead of the dot4 kernel at 28, 56 and 112 columns
  // (8.8 / 13.1 / 14.2 us against 10.2 / 16.7 / 16.4 us for 256 / 128 / 32 channels), behind it on the half-empty
  // chunks and strips of 14 x 14 and 7 x 7 planes (9.8 / 11.8 us against 7.9 / 5.0 us)
  const int nc = (ow + 31) / 32, strips = (oh + 7) / 8;
  return 32.0 * nc * 8.0 * strips <= 1.35 * ow * oh;
}

hipError_t launch_depthwise(const DepthwiseArgs &a0, hipStream_t s, LaunchPlan<DepthwiseArgs> *plan)
{
  if (plan && plan->valid) {   // everything but the tensors is as on the first launch
    return plan_relaunch(*plan, [&](DepthwiseArgs &x) { x.in = a0.in; x.out = a0.out; }, s);
  }
  DepthwiseArgs a = a0;
  if (a.stride != 1 && a.stride != 2) {
    set_error("depthwise: stride must be 1 or 2");
    return hipErrorInvalidValue;
  }
  if (depthwise_mfma_applies(a.stride, a.oh, a.ow, a.pad_t, a.pad_l, a.out_type, a.with_relu, a.lo, a.hi, (long long)a.n * a.g2, a.ih,
                             a.iw)) {
    const int nc = (a.ow + 31) / 32;
    const bool full = a.lo == 0.0f && a.hi == 255.0f;
    a.T_magic = div_magic(a.T);
    a.blocks_per_plane = (a.oh + 7) / 8;   // strips of 8 output rows per plane
    const long long total = (long long)a.n * a.g2 * a.blocks_per_plane;
    // (the kernel addresses both tensors with 32-bit byte offsets and keeps the last 64 KB of that range
    // as "nowhere")
    if (total >= (1ll << 30) || (long long)a.n * a.g2 * a.ih * a.iw * 16 >= (1ll << 32) - 65536 ||
        (long long)a.n * a.g2 * a.oh * a.ow * 16 >= (1ll << 32) - 65536) {
      set_error("depthwise: tensor too large");
      return hipErrorInvalidValue;
    }
    // a run of strips per workgroup, about four workgroups per CU (enough to hide a barrier and the
    // epilogue of one behind the MFMAs of another), the same run length for all so that none is the tail
    const int cus = 256 * 4;
    int per_wg = (int)((total + cus - 1) / cus);
    if (per_wg < 1) per_wg = 1;
    a.strips_per_wg = per_wg;
    const long long wgs = 8 * ((((total + per_wg - 1) / per_wg) + 7) / 8);
    dw_kernel_t kernel = nullptr;
#define EHIP_DWM(NC) (full ? k_depthwise3x3_mfma<2, NC> : k_depthwise3x3_mfma<1, NC>)
    kernel = nc == 1 ? EHIP_DWM(1) : (nc == 2 ? EHIP_DWM(2) : (nc == 3 ? EHIP_DWM(3) : EHIP_DWM(4)));
#undef EHIP_DWM
    return dw_launch(plan, kernel, dim3((unsigned)wgs), dim3(kBlock), a, s);
  }
  // four rows per lane on tall planes (seven where that divides the height: 28, 56, 112 -- fewer halo
  // rows re-read, 2-5 % on the MobileNet layers), fewer where that would leave lanes idle
  int rb = (a.oh >= 28 && a.oh % 7 == 0) ? 7 : (a.oh >= 16 ? 4 : (a.oh >= 7 ? 2 : 1));
  // measured at N = 64: 14 x 14 planes at stride 1 want seven rows as well (512 channels: 6.05 against 7.2 us with
  // two, 6.3 with four), 56 x 56 outputs of a stride-2 layer two (64 channels 112 -> 56: 13.4 against 15.3 us with
  // seven: 15 input rows of five pixels per lane are too many loads in flight)
  if (a.stride == 1 && a.oh == 14) rb = 7;
  if (a.stride == 2 && a.oh >= 56) rb = 2;
  const int ohb = (a.oh + rb - 1) / rb;
  const int wp = (a.ow + 1) / 2;
  a.lanes_per_plane = ohb * wp * 4;
  a.wp_magic = div_magic(wp);
  a.T_magic = div_magic(a.T);
  // 32-bit byte offsets inside the kernel
  if ((long long)a.n * a.g2 * a.ih * a.iw * 16 >= (1ll << 32) || (long long)a.n * a.g2 * a.oh * a.ow * 16 >= (1ll << 32)) {
    set_error("depthwise: tensors of 4 GiB and more are not supported");
    return hipErrorInvalidValue;
  }
  int mode = 0;
  if (a.out_type == EHIP_U8 && a.with_relu && a.lo >= 0.0f && a.hi <= 255.0f && a.hi >= a.lo)
    mode = (a.lo == 0.0f && a.hi == 255.0f) ? 2 : 1;
  int block = a.lanes_per_plane >= kBlock ? kBlock : up(a.lanes_per_plane, kWave);
  a.blocks_per_plane = (a.lanes_per_plane + block - 1) / block;
  const long long planes = (long long)a.n * a.g2;
  a.planes_per_block = 1;
  a.lanes_padded = block;
  if (block <= kBlock / 2) {   // a plane fits one or two waves: several planes per workgroup
    a.planes_per_block = kBlock / block;
    block *= a.planes_per_block;
  }
  const long long groups = (planes + a.planes_per_block - 1) / a.planes_per_block;
  dim3 grid((unsigned)(8 * ((groups + 7) / 8) * a.blocks_per_plane), 1, 1);
  const dw_kernel_t kernel = rb == 7 ? kernel_rb<7>(a.stride, mode)
      : (rb == 4 ? kernel_rb<4>(a.stride, mode) : (rb == 2 ? kernel_rb<2>(a.stride, mode) : kernel_rb<1>(a.stride, mode)));
  return dw_launch(plan, kernel, grid, dim3(block), a, s);
}

}  // namespace ehip
