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
}  // namespace

// MODE 0: any output type / bounds.  MODE 1: u8 output, ReLU with 0 <= lo <= hi <= 255 (floor and
// round-to-nearest both land in the code range, so the pack-with-saturation instruction, which
// rounds to nearest even itself, finishes either).  MODE 2: as 1 with lo == 0 and hi == 255, where
// the clamp is the instruction's own saturation.
template <int RB, int MODE, int S>
__global__ __launch_bounds__(kBlock) void k_depthwise3x3_u8s8(DepthwiseArgs a)
{
  constexpr int NPX = S == 1 ? 4 : 5;          // input pixels per row a lane touches
  constexpr int NROWS = S * (RB - 1) + 3;      // input rows
  // A plane (one image x one 16-channel block) is split into blocks over its lanes (q fastest, then
  // column pair, then row block).  Workgroups go round the eight XCDs (block b runs on XCD b % 8), each
  // with an L2 of its own, and neighbouring row blocks share two input rows: so all blocks of a plane
  // are given to ONE XCD, one after the other -- plane = 8 * (seq / blocks_per_plane) + xcd.
  const int xcd = blockIdx.x & 7, seq = blockIdx.x >> 3;
  const int pgrp = seq / a.blocks_per_plane;
  const int plane_id = pgrp * 8 + xcd;
  if (plane_id >= a.n * a.g2) return;   // whole workgroup
  const int wp = (a.ow + 1) >> 1;
  const int local = (seq - pgrp * a.blocks_per_plane) * blockDim.x + threadIdx.x;
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

namespace {
typedef void (*dw_kernel_t)(DepthwiseArgs);
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

hipError_t launch_depthwise(const DepthwiseArgs &a0, hipStream_t s, LaunchPlan<DepthwiseArgs> *plan)
{
  if (plan && plan->valid) {   // everything but the tensors is as on the first launch
    plan->args.in = a0.in;
    plan->args.out = a0.out;
    return plan_relaunch(*plan, s);
  }
  DepthwiseArgs a = a0;
  if (a.stride != 1 && a.stride != 2) {
    set_error("depthwise: stride must be 1 or 2");
    return hipErrorInvalidValue;
  }
  // four rows per lane on tall planes (seven where that divides the height: 28, 56, 112 -- fewer halo
  // rows re-read, 2-5 % on the MobileNet layers), fewer where that would leave lanes idle
  const int rb = (a.oh >= 28 && a.oh % 7 == 0) ? 7 : (a.oh >= 16 ? 4 : (a.oh >= 7 ? 2 : 1));
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
  const int block = a.lanes_per_plane >= kBlock ? kBlock : up(a.lanes_per_plane, kWave);
  a.blocks_per_plane = (a.lanes_per_plane + block - 1) / block;
  const long long planes = (long long)a.n * a.g2;
  dim3 grid((unsigned)(8 * ((planes + 7) / 8) * a.blocks_per_plane), 1, 1);
  const dw_kernel_t kernel = rb == 7 ? kernel_rb<7>(a.stride, mode)
      : (rb == 4 ? kernel_rb<4>(a.stride, mode) : (rb == 2 ? kernel_rb<2>(a.stride, mode) : kernel_rb<1>(a.stride, mode)));
  return plan_launch(plan, kernel, grid, dim3(block), 0, a, s);
}

}  // namespace ehip
