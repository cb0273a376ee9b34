// Winograd F(4x4,3x3) transforms around the int8 GEMM: bandwidth kernels.
//
//   trans_input : fp32 nChw16c -> gather 6x6 tiles (zero frame) -> V = Bt d B -> u8
//                 replaces elx_conv_wino_trans_input_t<uint8_t,...>::__execute_blocked_nhwc
//                 (src/elx_conv_wino_trans_input.cpp:599-654) + the 6x6 input kernel
//                 (src/kernel/elk_conv_wino_4x4_3x3_input.hxx:13-352)
//   trans_output: f32 GEMM result -> Y = At M A (+bias)(ReLU) -> fp32 nChw16c
//                 replaces elx_conv_wino_trans_output_t::__execute_blocked
//                 (src/elx_conv_wino_trans_output.cpp:212-277) + the output kernel
//                 (src/kernel/elk_conv_wino_4x4_3x3_output.hxx:19-201)
//   range       : min/max of the fp32 transformed input, what the reference's harness uses to
//                 calibrate wino_tinput_quant (tests/elt_conv_utils.cpp:222-262)
//
// One lane owns one tile x four channels: it loads 36 float4 (tile rows are 4 pixels apart, so the
// lanes of a wave cover 16 neighbouring tiles x 64 bytes), transforms the four channels one after
// the other in registers and writes, for each of the 36 tile positions, one dword of u8 (input
// side) -- the 64 lanes of a wave then write 256 contiguous bytes of [pos][ic2][tile][16].
//
// The float arithmetic follows the reference's compiled kernels operation for operation; which
// multiply-adds are single-rounding is spelled out with __builtin_fmaf and the file is compiled
// with -ffp-contract=off.  Tiles that touch the zero frame go through the reference's "border"
// kernel, whose compiled form rounds the products of raw inputs in the column pass (and one
// product of the last row pass) separately.
#include "ehip_internal.hpp"

namespace ehip {

namespace {

__device__ __forceinline__ void in_1d(const float f[6], float o[6], bool raw_unfused, bool t4_unfused)
{
  const float z0 = -2.25f, z1 = -0.390625f, z2 = 0.87890625f, z3 = -2.640625f, z4 = 0.625f, z5 = 1.5f;
  float t0, t1, t2, t3, t4, t5;
  if (raw_unfused) {
    t0 = f[2] * z0 + f[4];
    t1 = f[1] * z0 + f[3];
    t2 = f[2] * z1 + f[4];
    t3 = f[1] * z1 + f[3];
    t4 = f[0] * z2 + f[4];
    t5 = f[1] * z2 + f[5];
    o[0] = f[2] * z3 + t4;
    o[5] = f[3] * z3 + t5;
  } else {
    t0 = __builtin_fmaf(f[2], z0, f[4]);
    t1 = __builtin_fmaf(f[1], z0, f[3]);
    t2 = __builtin_fmaf(f[2], z1, f[4]);
    t3 = __builtin_fmaf(f[1], z1, f[3]);
    t4 = t4_unfused ? f[0] * z2 + f[4] : __builtin_fmaf(f[0], z2, f[4]);
    t5 = __builtin_fmaf(f[1], z2, f[5]);
    o[0] = __builtin_fmaf(f[2], z3, t4);
    o[5] = __builtin_fmaf(f[3], z3, t5);
  }
  o[1] = __builtin_fmaf(t1, z4, t0);
  o[2] = __builtin_fmaf(-t1, z4, t0);
  o[3] = __builtin_fmaf(t3, z5, t2);
  o[4] = __builtin_fmaf(-t3, z5, t2);
}

// d, v: [6][6] row-major
__device__ __forceinline__ void tile_input(const float d[36], float v[36], bool border)
{
  float m[36];
#pragma unroll
  for (int j = 0; j < 6; ++j) {
    float f[6], o[6];
#pragma unroll
    for (int i = 0; i < 6; ++i) f[i] = d[6 * i + j];
    in_1d(f, o, border, false);
#pragma unroll
    for (int i = 0; i < 6; ++i) m[6 * i + j] = o[i];
  }
#pragma unroll
  for (int i = 0; i < 6; ++i) in_1d(&m[6 * i], &v[6 * i], false, border && i == 5);
}

__device__ __forceinline__ void out_1d(const float f[6], float o[4])
{
  const float z0 = 1.5f, z1 = 2.25f, z2 = 3.375f, z3 = 0.625f, z4 = 0.390625f, z5 = 0.244140625f;
  const float t0 = f[1] + f[2];
  const float t1 = f[3] + f[4];
  const float t2 = f[1] - f[2];
  const float t3 = f[3] - f[4];
  o[0] = t0 + t1 + f[0];
  o[1] = __builtin_fmaf(t2, z3, t3 * z0);
  o[2] = __builtin_fmaf(t0, z4, t1 * z1);
  o[3] = __builtin_fmaf(t2, z5, t3 * z2) + f[5];
}

__device__ __forceinline__ float comp_of(const float4 &v, int k)
{
  return k == 0 ? v.x : (k == 1 ? v.y : (k == 2 ? v.z : v.w));
}

// order-preserving map float -> unsigned, for atomicMin/atomicMax
__device__ __forceinline__ unsigned f2ord(float f)
{
  unsigned u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

struct TileCoord {
  int n, th, tw, h0, w0;
  bool border;
};
__device__ __forceinline__ TileCoord tile_coord(const WinoArgs &a, int t)
{
  TileCoord c;
  c.n = t / a.nt;
  const int rem = t - c.n * a.nt;
  c.th = rem / a.wt;
  c.tw = rem - c.th * a.wt;
  c.h0 = 4 * c.th - a.pad_t;
  c.w0 = 4 * c.tw - a.pad_l;
  c.border = c.h0 < 0 || c.w0 < 0 || c.h0 + 5 >= a.ih || c.w0 + 5 >= a.iw;
  return c;
}

__device__ __forceinline__ void gather_tile(const WinoArgs &a, const TileCoord &c, int c2, int q, float4 d[36])
{
  const float4 *plane = reinterpret_cast<const float4 *>(a.in) +
      ((size_t)c.n * a.ic2 + c2) * a.ih * a.iw * 4 + q;
#pragma unroll
  for (int i = 0; i < 6; ++i)
#pragma unroll
    for (int j = 0; j < 6; ++j) {
      const int h = c.h0 + i, w = c.w0 + j;
      d[6 * i + j] = (h >= 0 && h < a.ih && w >= 0 && w < a.iw) ? plane[((size_t)h * a.iw + w) * 4]
                                                                   : make_float4(0.f, 0.f, 0.f, 0.f);
    }
}

}  // namespace

// Tiles that touch the zero frame take the "border" arithmetic, all others the plain one; a wave
// that holds both kinds would execute both.  So the grid is split: the first a.blocks_interior
// blocks enumerate only tiles away from the rim of the tile grid (never border), the remaining
// blocks enumerate the rim.  Returns false past the end of the group.
__device__ __forceinline__ bool grouped_tile(const WinoArgs &a, int block, int slot, TileCoord &c, int &t)
{
  const int wi = a.wt - 2, hi = a.ht - 2;
  const int ni = (wi > 0 && hi > 0) ? wi * hi : 0;   // interior tiles per image
  int n, th, tw;
  if (block < a.blocks_interior) {
    const int idx = block * 64 + slot;
    if (idx >= a.n * ni) return false;
    n = idx / ni;
    const int r = idx - n * ni;
    th = 1 + r / wi;
    tw = 1 + (r - (th - 1) * wi);
  } else {
    const int idx = (block - a.blocks_interior) * 64 + slot;
    const int nr = a.nt - ni;                        // rim tiles per image
    if (idx >= a.n * nr) return false;
    n = idx / nr;
    const int r = idx - n * nr;
    if (ni == 0) {                                   // fewer than 3 tile rows or columns: all rim
      th = r / a.wt;
      tw = r - th * a.wt;
    } else if (r < a.wt) {
      th = 0; tw = r;
    } else if (r < 2 * a.wt) {
      th = a.ht - 1; tw = r - a.wt;
    } else {
      const int rr = r - 2 * a.wt;
      th = 1 + (rr >> 1);
      tw = (rr & 1) ? a.wt - 1 : 0;
    }
  }
  t = n * a.nt + th * a.wt + tw;
  c.n = n; c.th = th; c.tw = tw;
  c.h0 = 4 * th - a.pad_t;
  c.w0 = 4 * tw - a.pad_l;
  c.border = c.h0 < 0 || c.w0 < 0 || c.h0 + 5 >= a.ih || c.w0 + 5 >= a.iw;
  return true;
}

// grid: (interior blocks + rim blocks, ic2); block: 64 tiles x 4 channel quads
__global__ __launch_bounds__(kBlock) void k_wino_trans_input_u8(WinoArgs a)
{
  const int q = threadIdx.x & 3;
  const int c2 = blockIdx.y;
  TileCoord c;
  int t;
  if (!grouped_tile(a, blockIdx.x, threadIdx.x >> 2, c, t)) return;
  float4 d[36];
  gather_tile(a, c, c2, q, d);
  unsigned packed[36];
#pragma unroll
  for (int k = 0; k < 36; ++k) packed[k] = 0u;
  auto channels = [&](bool border) {
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      float f[36], v[36];
#pragma unroll
      for (int e = 0; e < 36; ++e) f[e] = comp_of(d[e], k);
      tile_input(f, v, border);
#pragma unroll
      for (int e = 0; e < 36; ++e) {
        // sat_u8(rne_to_u32(V * (in_S / tin_S) + tin_z)), one rounding in the multiply-add.  The
        // reference's float -> u32 conversion turns everything below -0.5 (and NaN) into 0xffffffff,
        // which then saturates to 255; v_cvt_pk_u8_f32 rounds to nearest even and saturates the rest.
        const float y = __builtin_fmaf(v[e], a.mrepS, a.mz);
        packed[e] = __builtin_amdgcn_cvt_pk_u8_f32(y >= -0.5f ? y : 300.0f, k, packed[e]);
      }
    }
  };
  if (blockIdx.x < a.blocks_interior) {
    channels(false);
  } else {
    if (c.border) channels(true);
    else channels(false);
  }
  unsigned *dst = reinterpret_cast<unsigned *>(a.tin) + ((size_t)c2 * a.t + t) * 4 + q;
  const size_t pos_stride = (size_t)a.ic2 * a.t * 4;
#pragma unroll
  for (int e = 0; e < 36; ++e) dst[e * pos_stride] = packed[e];
}

// minmax_dev[0] = ordered-min, [1] = ordered-max (see f2ord); real channels only
__global__ __launch_bounds__(kBlock) void k_wino_tinput_range(WinoArgs a, int ic_real, unsigned *minmax_dev)
{
  const int q = threadIdx.x & 3;
  const int t = blockIdx.x * 64 + (threadIdx.x >> 2);
  const int c2 = blockIdx.y;
  float mn = 3.4e38f, mx = -3.4e38f;
  if (t < a.t) {
    const TileCoord c = tile_coord(a, t);
    float4 d[36];
    gather_tile(a, c, c2, q, d);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      if (c2 * 16 + 4 * q + k >= ic_real) continue;
      float f[36], v[36];
#pragma unroll
      for (int e = 0; e < 36; ++e) f[e] = comp_of(d[e], k);
      if (c.border) tile_input(f, v, true);
      else tile_input(f, v, false);
#pragma unroll
      for (int e = 0; e < 36; ++e) {
        mn = v[e] < mn ? v[e] : mn;
        mx = v[e] > mx ? v[e] : mx;
      }
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float omn = __shfl_xor(mn, off), omx = __shfl_xor(mx, off);
    mn = omn < mn ? omn : mn;
    mx = omx > mx ? omx : mx;
  }
  if ((threadIdx.x & 63) == 0) {
    atomicMin(&minmax_dev[0], f2ord(mn));
    atomicMax(&minmax_dev[1], f2ord(mx));
  }
}

// grid: (ceil(t / 64), oc2); block: 64 tiles x 4 channel quads
__global__ __launch_bounds__(kBlock) void k_wino_trans_output_f32(WinoArgs a)
{
  const int q = threadIdx.x & 3;
  const int t = blockIdx.x * 64 + (threadIdx.x >> 2);
  const int o2 = blockIdx.y;
  if (t >= a.t) return;
  const int n = t / a.nt;
  const int rem = t - n * a.nt;
  const int th = rem / a.wt;
  const int tw = rem - th * a.wt;

  const float4 *src = reinterpret_cast<const float4 *>(a.tout) + ((size_t)o2 * a.t + t) * 4 + q;
  const size_t pos_stride = (size_t)a.oc2 * a.t * 4;
  float4 m[36];
#pragma unroll
  for (int e = 0; e < 36; ++e) m[e] = src[e * pos_stride];

  float4 bias = make_float4(0.f, 0.f, 0.f, 0.f);
  if (a.with_bias) bias = reinterpret_cast<const float4 *>(a.bias)[o2 * 4 + q];

  float y[4][16];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    float M[4][6];
#pragma unroll
    for (int i = 0; i < 6; ++i) {
      float f[6], o[4];
#pragma unroll
      for (int r = 0; r < 6; ++r) f[r] = comp_of(m[6 * r + i], k);
      out_1d(f, o);
#pragma unroll
      for (int r = 0; r < 4; ++r) M[r][i] = o[r];
    }
    const float b = comp_of(bias, k);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float o[4];
      out_1d(M[i], o);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        float r = o[j];
        if (a.with_bias) r = r + b;
        if (a.with_relu) r = r > 0.0f ? r : 0.0f;
        y[k][4 * i + j] = r;
      }
    }
  }
  float4 *dst = reinterpret_cast<float4 *>(a.out) + ((size_t)n * a.oc2 + o2) * a.oh * a.ow * 4 + q;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int oh = 4 * th + i;
    if (oh >= a.oh) break;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int ow = 4 * tw + j;
      if (ow >= a.ow) break;
      dst[((size_t)oh * a.ow + ow) * 4] = make_float4(y[0][4 * i + j], y[1][4 * i + j], y[2][4 * i + j], y[3][4 * i + j]);
    }
  }
}

hipError_t launch_wino_trans_input(const WinoArgs &a0, hipStream_t s)
{
  WinoArgs a = a0;
  const int ni = (a.wt > 2 && a.ht > 2) ? (a.wt - 2) * (a.ht - 2) : 0;
  a.blocks_interior = (a.n * ni + 63) / 64;
  const int blocks_rim = (a.n * (a.nt - ni) + 63) / 64;
  dim3 grid(a.blocks_interior + blocks_rim, a.ic2);
  hipLaunchKernelGGL(k_wino_trans_input_u8, grid, dim3(kBlock), 0, s, a);
  return hipGetLastError();
}

hipError_t launch_wino_trans_output(const WinoArgs &a, hipStream_t s)
{
  dim3 grid((a.t + 63) / 64, a.oc2);
  hipLaunchKernelGGL(k_wino_trans_output_f32, grid, dim3(kBlock), 0, s, a);
  return hipGetLastError();
}

hipError_t launch_wino_range(const WinoArgs &a, int ic_real, unsigned *minmax_dev, hipStream_t s)
{
  dim3 grid((a.t + 63) / 64, a.ic2);
  hipLaunchKernelGGL(k_wino_tinput_range, grid, dim3(kBlock), 0, s, a, ic_real, minmax_dev);
  return hipGetLastError();
}

}  // namespace ehip
