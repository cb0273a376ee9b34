// Winograd transforms around the int8 GEMM: bandwidth kernels.  Tile size A = 6 is F(4x4,3x3) (described
// below), A = 4 F(2x2,3x3) and A = 5 F(3x3,3x3) are the same kernels with an A x A tile and an
// (A-2) x (A-2) output tile (template parameter; tile arithmetic in ehip_wino_tiles.hpp).
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
#include <mutex>

#include "ehip_internal.hpp"
#include "ehip_wino_tiles.hpp"

#ifdef EHIP_TRACE
#define TRACE_POINT(i)                                                                             \
  do {                                                                                             \
    if (a.trace && lane == 0) a.trace[((size_t)blockIdx.x * 4 + wave) * 16 + (i)] = clock64();     \
  } while (0)
#else
#define TRACE_POINT(i) do { } while (0)
#endif

namespace ehip {

namespace {

// Buffer addressing (a load whose offset lies outside the buffer returns zero and touches no memory).  The
// builtins exist in the device pass only.
#if defined(__HIP_DEVICE_COMPILE__)
typedef __amdgpu_buffer_rsrc_t BufferRsrc;
__device__ __forceinline__ BufferRsrc make_rsrc(const void *base, unsigned bytes)
{
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), (short)0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ void buffer_load_cell(BufferRsrc r, unsigned off, float4 &v)
{
  typedef float v4f __attribute__((ext_vector_type(4)));
  const v4f x = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(r, (int)off, 0, 0));
  v = make_float4(x.x, x.y, x.z, x.w);
}
__device__ __forceinline__ void buffer_load_cell(BufferRsrc r, unsigned off, unsigned &v)
{
  v = __builtin_amdgcn_raw_buffer_load_b32(r, (int)off, 0, 0);
}
__device__ __forceinline__ void buffer_load_cell(BufferRsrc r, unsigned off, uint4 &v)
{
  typedef unsigned v4u __attribute__((ext_vector_type(4)));
  const v4u x = __builtin_bit_cast(v4u, __builtin_amdgcn_raw_buffer_load_b128(r, (int)off, 0, 0));
  v = make_uint4(x.x, x.y, x.z, x.w);
}
// 4 x 4 transpose of dwords between four registers and the four lanes of a quad (lanes 4 n .. 4 n + 3): register j of
// lane q becomes register q of lane j.  Two exchanges, with the neighbour (lane ^ 1) and across (lane ^ 2); in each a lane
// sends the register its partner lacks and takes the partner's in its place.
__device__ __forceinline__ void quad_transpose(unsigned &x0, unsigned &x1, unsigned &x2, unsigned &x3, int lane)
{
  const bool odd = (lane & 1) != 0, hi = (lane & 2) != 0;
  {
    const unsigned r01 = __builtin_amdgcn_mov_dpp(odd ? x0 : x1, 0xB1, 0xf, 0xf, true);   // quad_perm [1, 0, 3, 2]
    const unsigned r23 = __builtin_amdgcn_mov_dpp(odd ? x2 : x3, 0xB1, 0xf, 0xf, true);
    if (odd) { x0 = r01; x2 = r23; } else { x1 = r01; x3 = r23; }
  }
  {
    const unsigned r02 = __builtin_amdgcn_mov_dpp(hi ? x0 : x2, 0x4E, 0xf, 0xf, true);    // quad_perm [2, 3, 0, 1]
    const unsigned r13 = __builtin_amdgcn_mov_dpp(hi ? x1 : x3, 0x4E, 0xf, 0xf, true);
    if (hi) { x0 = r02; x1 = r13; } else { x2 = r02; x3 = r13; }
  }
}
#else
typedef int BufferRsrc;
__device__ inline BufferRsrc make_rsrc(const void *, unsigned) { return 0; }
__device__ inline void buffer_load_cell(BufferRsrc, unsigned, float4 &v) { v = float4(); }
__device__ inline void buffer_load_cell(BufferRsrc, unsigned, unsigned &v) { v = 0u; }
__device__ inline void buffer_load_cell(BufferRsrc, unsigned, uint4 &v) { v = uint4(); }
__device__ inline void quad_transpose(unsigned &, unsigned &, unsigned &, unsigned &, int) {}
#endif

__device__ __forceinline__ float comp_of(const float4 &v, int k)
{
  return k == 0 ? v.x : (k == 1 ? v.y : (k == 2 ? v.z : v.w));
}

// four u8 codes in a dword: the reference turns the codes into floats as they are
// (src/kernel/elk_conv_wino_4x4_3x3_input.hxx:40-47)
__device__ __forceinline__ float comp_of(const unsigned &v, int k)
{
  return (float)((v >> (8 * k)) & 0xffu);
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
template <int A>
__device__ __forceinline__ TileCoord tile_coord(const WinoArgs &a, int t)
{
  TileCoord c;
  c.n = t / a.nt;
  const int rem = t - c.n * a.nt;
  c.th = rem / a.wt;
  c.tw = rem - c.th * a.wt;
  c.h0 = (A - 2) * c.th - a.pad_t;
  c.w0 = (A - 2) * c.tw - a.pad_l;
  c.border = c.h0 < 0 || c.w0 < 0 || c.h0 + A - 1 >= a.ih || c.w0 + A - 1 >= a.iw;
  return c;
}

// the lane's four channels of the A x A pixels of a tile: float4 (f32 input) or 4 packed codes (u8)
template <int A>
__device__ __forceinline__ void gather_tile(const WinoArgs &a, const TileCoord &c, int c2, int q, float4 *d)
{
  // blocked: the 16-channel plane of (n, c2), 4 quads per pixel; nhwc: quad c2 * 4 + q of every pixel's vector
  const size_t pq = a.in_nhwc ? (size_t)a.ic2 * 4 : 4;   // quads between neighbouring pixels
  const float4 *plane = reinterpret_cast<const float4 *>(a.in) +
      (a.in_nhwc ? (size_t)c.n * a.ih * a.iw * pq + c2 * 4 : ((size_t)c.n * a.ic2 + c2) * a.ih * a.iw * 4) + q;
#pragma unroll
  for (int i = 0; i < A; ++i)
#pragma unroll
    for (int j = 0; j < A; ++j) {
      const int h = c.h0 + i, w = c.w0 + j;
      d[A * i + j] = (h >= 0 && h < a.ih && w >= 0 && w < a.iw) ? plane[((size_t)h * a.iw + w) * pq]
                                                                   : make_float4(0.f, 0.f, 0.f, 0.f);
    }
}
template <int A>
__device__ __forceinline__ void gather_tile(const WinoArgs &a, const TileCoord &c, int c2, int q, unsigned *d)
{
  const size_t pq = a.in_nhwc ? (size_t)a.ic2 * 4 : 4;
  const unsigned *plane = reinterpret_cast<const unsigned *>(a.in) +
      (a.in_nhwc ? (size_t)c.n * a.ih * a.iw * pq + c2 * 4 : ((size_t)c.n * a.ic2 + c2) * a.ih * a.iw * 4) + q;
#pragma unroll
  for (int i = 0; i < A; ++i)
#pragma unroll
    for (int j = 0; j < A; ++j) {
      const int h = c.h0 + i, w = c.w0 + j;
      d[A * i + j] = (h >= 0 && h < a.ih && w >= 0 && w < a.iw) ? plane[((size_t)h * a.iw + w) * pq] : 0u;   // the frame is 0.0f
    }
}

// The same gather through buffer addressing, for tensors below 4 GB (WinoArgs::buf_gather).  A cell's byte
// offset is the lane's first cell's (32 bits, possibly "negative" for a tile that starts in the frame) plus
// a scalar; rows and columns are tested once each, a cell's test is the AND of two lane masks (scalar
// instructions), and a cell of the frame is sent to an offset outside the buffer, where the load returns
// the frame's zero.  Two vector instructions per cell instead of a bounds test, a 64-bit multiply-add and
// a branch.
template <int A, typename Cell>
__device__ __forceinline__ void gather_tile_buf(const WinoArgs &a, const TileCoord &c, int c2, int q, Cell *d)
{
  const unsigned pq = a.in_nhwc ? (unsigned)a.ic2 * 4u : 4u;   // cells between neighbouring pixels
  const unsigned cells = (unsigned)a.n * a.ic2 * a.ih * a.iw * 4u;
  const BufferRsrc rin = make_rsrc(a.in, cells * (unsigned)sizeof(Cell));
  const unsigned plane = a.in_nhwc ? (unsigned)c.n * a.ih * a.iw * pq + c2 * 4u
                                   : ((unsigned)c.n * a.ic2 + c2) * a.ih * a.iw * 4u;
  const unsigned voff = (plane + (unsigned)(c.h0 * a.iw + c.w0) * pq + q) * (unsigned)sizeof(Cell);
  bool rv[A], cv[A];
#pragma unroll
  for (int i = 0; i < A; ++i) {
    rv[i] = (unsigned)(c.h0 + i) < (unsigned)a.ih;
    cv[i] = (unsigned)(c.w0 + i) < (unsigned)a.iw;
  }
#pragma unroll
  for (int i = 0; i < A; ++i)
#pragma unroll
    for (int j = 0; j < A; ++j) {
      const unsigned so = (unsigned)(i * a.iw + j) * pq * (unsigned)sizeof(Cell);   // scalar
      buffer_load_cell(rin, (rv[i] && cv[j]) ? voff + so : 0xffffff00u, d[A * i + j]);
    }
}

// u8 input below 4 GB, by whole cells: the four lanes of a tile (one channel quad each) share the tile's pixels out
// between them -- lane q loads the 16 bytes (all four quads) of pixels q, 4 + q, 8 + q, ... -- and a transpose inside
// the quad hands every lane its own quad of four pixels at a time.  A wave's load then covers 16 tiles x four
// neighbouring pixels = up to 1 KB in lane order, a quarter of the load instructions and of the cache lines looked up
// per byte (one dword per lane and pixel looks up a 64-byte line for 16 bytes).  Cells of the zero frame are sent
// to an offset outside the buffer, as in gather_tile_buf.
template <int A>
__device__ __forceinline__ void gather_tile_wide(const WinoArgs &a, const TileCoord &c, int c2, int q, unsigned *d)
{
  constexpr int AA = A * A;
  const unsigned pc = a.in_nhwc ? (unsigned)a.ic2 : 1u;   // cells between neighbouring pixels
  const unsigned cells = (unsigned)a.n * a.ic2 * a.ih * a.iw;
  const BufferRsrc rin = make_rsrc(a.in, cells * 16u);
  const unsigned plane = a.in_nhwc ? (unsigned)c.n * a.ih * a.iw * pc + c2 : ((unsigned)c.n * a.ic2 + c2) * a.ih * a.iw;
  constexpr int NK = (AA + 3) / 4;
  uint4 v[NK];
  // every load first (offsets without a branch), then the exchanges
#pragma unroll
  for (int k = 0; k < NK; ++k) {
    const int e = 4 * k + q;       // the lane's pixel of this group
    const int i = e / A, j = e - A * i;
    const int h = c.h0 + i, w = c.w0 + j;
    const bool ok = e < AA && (unsigned)h < (unsigned)a.ih && (unsigned)w < (unsigned)a.iw;
    const unsigned off = (plane + (unsigned)(h * a.iw + w) * pc) * 16u;
    buffer_load_cell(rin, ok ? off : 0xffffff00u, v[k]);
  }
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int k = 0; k < NK; ++k) {
    quad_transpose(v[k].x, v[k].y, v[k].z, v[k].w, q);
    d[4 * k] = v[k].x;
    if (4 * k + 1 < AA) d[4 * k + 1 < AA ? 4 * k + 1 : 0] = v[k].y;
    if (4 * k + 2 < AA) d[4 * k + 2 < AA ? 4 * k + 2 : 0] = v[k].z;
    if (4 * k + 3 < AA) d[4 * k + 3 < AA ? 4 * k + 3 : 0] = v[k].w;
  }
}
template <int A>
__device__ __forceinline__ void gather_tile_wide(const WinoArgs &, const TileCoord &, int, int, float4 *) {}   // (u8 input only)

}  // namespace

// block: 64 consecutive tiles x 4 channel quads of one 16-channel unit.  Work items are numbered tile
// block first, then unit, and XCD x (workgroup b runs on XCD b % 8) takes the x-th eighth of them:
// neighbouring tile blocks read the same two input rows where they meet, and find them in their XCD's L2.
// Tiles that touch the zero frame take the reference's "border" arithmetic, the others the plain one; a
// wave that holds both kinds (nearly every wave: two rim tiles per row of tiles) runs the per-lane,
// branch-free form of the transform instead of both forms under complementary masks.
// Cell = float4 (f32 user input) or unsigned (u8 user input: four codes per lane and pixel).
template <typename Cell, int A = 6>
__global__ __launch_bounds__(kBlock) void k_wino_trans_input_u8(WinoArgs a)
{
  constexpr int AA = A * A;
  constexpr bool kCodes = sizeof(Cell) == sizeof(unsigned);
  const int q = threadIdx.x & 3;
  const int item = (blockIdx.x & 7) * a.items_per_xcd + (blockIdx.x >> 3);
  if (item >= a.nblocks * a.ic2) return;   // whole workgroup
  // plain layout: an XCD walks the tile blocks of one unit after the other (neighbours share input rows in
  // its L2); blocked layout: the units of one tile block after the other, whose pieces are neighbours in tin
  const int c2 = a.tin_blocked ? item % a.ic2 : item / a.nblocks;
  const int t = (a.tin_blocked ? item / a.ic2 : item - c2 * a.nblocks) * 64 + (threadIdx.x >> 2);
  if (t >= a.t) return;
  const TileCoord c = tile_coord<A>(a, t);
  Cell d[AA];
  if (kCodes && a.buf_gather == 2) gather_tile_wide<A>(a, c, c2, q, d);
  else if (a.buf_gather) gather_tile_buf<A>(a, c, c2, q, d);
  else gather_tile<A>(a, c, c2, q, d);
  unsigned packed[AA];
  // mixed: the wave holds interior and rim tiles -- the per-lane, branch-free form of the transform.
  // Quantization: sat_u8(rne_to_u32(V * (in_S / tin_S) + tin_z)), one rounding in the multiply-add.  The
  // reference's float -> u32 conversion turns everything below -0.5 (and NaN) into 0xffffffff, which then
  // saturates to 255; v_cvt_pk_u8_f32 rounds to nearest even and saturates the rest.  watch: the plain
  // conversion, with the quirk's cases only looked for -- two running integer maxima over the values' bit
  // patterns, one instruction per value instead of a compare and a select -- and the result says whether
  // one was seen (never, with a calibrated tinput_quant); the caller then runs the exact form again.
  // u8 user input: the codes are finite, so with finite quantization constants no NaN can arise and ONE running
  // float minimum (an instruction per two values) says whether anything fell below -0.5; constants that are not
  // finite send every wave to the exact form.
  const bool odd_consts = !(__builtin_fabsf(a.mrepS) <= 3.402823466e38f) || !(__builtin_fabsf(a.mz) <= 3.402823466e38f);
  auto channels = [&](bool mixed, bool watch) {
    unsigned seen_u = 0u;
    int seen_s = 0;
    float seen_min = 0.0f;
#pragma unroll
    for (int k = 0; k < AA; ++k) packed[k] = 0u;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      float f[AA], v[AA];
#pragma unroll
      for (int e = 0; e < AA; ++e) f[e] = comp_of(d[e], k);
      if (mixed) wino::tile_input_lanes<A>(f, v, c.border);
      else wino::tile_input<A>(f, v, false);
      if (watch) {
        float y[AA];
#pragma unroll
        for (int e = 0; e < AA; ++e) {
          y[e] = __builtin_fmaf(v[e], a.mrepS, a.mz);
          packed[e] = __builtin_amdgcn_cvt_pk_u8_f32(y[e], k, packed[e]);
        }
        // bit patterns above 0xbf000000 unsigned: below -0.5, or a negative NaN; above 0x7f800000 signed: a
        // positive NaN
        if (kCodes) {
#pragma unroll
          for (int e = 0; e + 1 < AA; e += 2) seen_min = __builtin_fminf(seen_min, __builtin_fminf(y[e], y[e + 1]));
          if (AA & 1) seen_min = __builtin_fminf(seen_min, y[AA - 1]);
        } else {
#pragma unroll
          for (int e = 0; e + 1 < AA; e += 2) {
            const unsigned b0 = __float_as_uint(y[e]), b1 = __float_as_uint(y[e + 1]);
            seen_u = max(seen_u, max(b0, b1));
            seen_s = max(seen_s, max((int)b0, (int)b1));
          }
          if (AA & 1) {
            const unsigned b = __float_as_uint(y[AA - 1]);
            seen_u = max(seen_u, b);
            seen_s = max(seen_s, (int)b);
          }
        }
      } else {
#pragma unroll
        for (int e = 0; e < AA; ++e) {
          const float y = __builtin_fmaf(v[e], a.mrepS, a.mz);
          packed[e] = __builtin_amdgcn_cvt_pk_u8_f32(y >= -0.5f ? y : 300.0f, k, packed[e]);
        }
      }
    }
    return kCodes ? (seen_min < -0.5f || odd_consts) : (seen_u > 0xbf000000u || seen_s > 0x7f800000);
  };
  const bool mixed = __ballot(c.border) != 0;   // wave-uniform
  bool again;
  if (mixed) again = channels(true, true);
  else again = channels(false, true);
  if (__ballot(again) != 0) {
    if (mixed) channels(true, false);
    else channels(false, false);
  }
  // A position's store = a wave-uniform base + position x stride + one 32-bit offset per lane that never changes
  // (47.3 against 48.7 us on 256 channels at 56 x 56 with the index worked out per lane in 64 bits; forcing the scalar
  // base into every store with assembly: no further gain).  Blocked layout: a wave's sixteen tiles lie in one block of 32.
  const int t32 = __builtin_amdgcn_readfirstlane(t >> 5);
  const uint8_t *base = a.tin_blocked ? a.tin + ((size_t)t32 * AA * a.ic2 + c2) * 512 : a.tin + (size_t)c2 * a.t * 16;
  const unsigned voff = a.tin_blocked ? (unsigned)((t & 31) * 4 + q) * 4u : (unsigned)(t * 4 + q) * 4u;
  const size_t pos_stride = a.tin_blocked ? (size_t)a.ic2 * 512 : (size_t)a.ic2 * a.t * 16;   // bytes
#pragma unroll
  for (int e = 0; e < AA; ++e)
    *reinterpret_cast<unsigned *>(const_cast<uint8_t *>(base) + e * pos_stride + voff) = packed[e];
}

// partials[2 * c2] = ordered-min, [2 * c2 + 1] = ordered-max (see f2ord) of 16-channel unit c2; real
// channels only.  One pair per unit keeps the atomics of different units on different addresses.
template <typename Cell, int A = 6>
__global__ __launch_bounds__(kBlock) void k_wino_tinput_range(WinoArgs a, int ic_real, unsigned *partials)
{
  constexpr int AA = A * A;
  const int q = threadIdx.x & 3;
  const int t = blockIdx.x * 64 + (threadIdx.x >> 2);
  const int c2 = blockIdx.y;
  float mn = 3.4e38f, mx = -3.4e38f;
  if (t < a.t) {
    const TileCoord c = tile_coord<A>(a, t);
    Cell d[AA];
    gather_tile<A>(a, c, c2, q, d);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      if (c2 * 16 + 4 * q + k >= ic_real) continue;
      float f[AA], v[AA];
#pragma unroll
      for (int e = 0; e < AA; ++e) f[e] = comp_of(d[e], k);
      wino::tile_input_lanes<A>(f, v, c.border);
#pragma unroll
      for (int e = 0; e < AA; ++e) {
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
    atomicMin(&partials[2 * c2], f2ord(mn));
    atomicMax(&partials[2 * c2 + 1], f2ord(mx));
  }
}

// every pair starts as (largest, smallest) ordered value
__global__ __launch_bounds__(kBlock) void k_wino_range_init(unsigned *partials, int units)
{
  const int i = blockIdx.x * kBlock + threadIdx.x;
  if (i < 2 * units) partials[i] = (i & 1) ? 0u : 0xffffffffu;
}

// one wave: min / max over the units' pairs, back to floats, to out[0] = min, out[1] = max
__global__ __launch_bounds__(kWave) void k_wino_range_finish(const unsigned *partials, int units, float *out)
{
  unsigned mn = 0xffffffffu, mx = 0u;
  for (int i = threadIdx.x; i < units; i += kWave) {
    const unsigned a = partials[2 * i], b = partials[2 * i + 1];
    mn = a < mn ? a : mn;
    mx = b > mx ? b : mx;
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const unsigned omn = __shfl_xor(mn, off), omx = __shfl_xor(mx, off);
    mn = omn < mn ? omn : mn;
    mx = omx > mx ? omx : mx;
  }
  if (threadIdx.x == 0) {
    out[0] = __uint_as_float((mn & 0x80000000u) ? (mn & 0x7fffffffu) : ~mn);
    out[1] = __uint_as_float((mx & 0x80000000u) ? (mx & 0x7fffffffu) : ~mx);
  }
}

// Y = At M A (+ bias)(output quantization)(ReLU) of one tile x four channels (the four components
// of the float4s) and its store.  `plane` is the tile's image plane ([oh][ow][16] of OUT's type), q the
// lane's channel quad.  u8 / s8 output (src/kernel/elk_conv_wino_4x4_3x3_output.hxx:94-111,165-171):
// value * (1 / out_S) + out_z in one rounding BEFORE the ReLU, then round to nearest even and
// saturate; the u8 store converts through an unsigned integer, so anything below -0.5 (and NaN)
// ends as 255.  Border tiles write their valid rows and columns only.
// The F(2x2,3x3) kernel converts toward minus infinity in its u8 / s8 store
// (src/kernel/elk_conv_wino_2x2_3x3_output.hxx:142-151), the others to nearest even.
// with_sum (in-place sum): the old output -- an f32, or the u8 / s8 code as a float, no scale -- is added
// after the output quantization and before the ReLU (src/kernel/elk_conv_wino_4x4_3x3_output.hxx:168-187).
template <int OUT, int A = 6>
__device__ __forceinline__ void output_tile(const float4 *m, const float4 &bias, bool with_bias, bool with_relu,
                                            float repS, float z, void *plane, int q, int th, int tw, int oh_n, int ow_n,
                                            bool with_sum = false, int px = 16)
{
  // px: elements between neighbouring pixels of `plane` (16 blocked; the channel count for nhwc, where
  // `plane` points at the tile's 16-channel block inside the first pixel's vector)
  constexpr int AA = A * A, M = A - 2;
  float y[4][M * M];
  float old[4][M * M];
  if (with_sum) {
#pragma unroll
    for (int i = 0; i < M; ++i)
#pragma unroll
      for (int j = 0; j < M; ++j) {
        const int oh = M * th + i, ow = M * tw + j;
        const bool in = oh < oh_n && ow < ow_n;
        const size_t cell = in ? ((size_t)oh * ow_n + ow) * px + 4 * q : 0;
        if (OUT == EHIP_F32) {
          const float4 v = *reinterpret_cast<const float4 *>(static_cast<const float *>(plane) + cell);
          old[0][M * i + j] = v.x; old[1][M * i + j] = v.y; old[2][M * i + j] = v.z; old[3][M * i + j] = v.w;
        } else {
          const unsigned v = *reinterpret_cast<const unsigned *>(static_cast<const uint8_t *>(plane) + cell);
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            const unsigned b = (v >> (8 * k)) & 0xffu;
            old[k][M * i + j] = OUT == EHIP_U8 ? (float)b : (float)(int)(signed char)b;
          }
        }
      }
  }
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    float f[AA], o[M * M];
#pragma unroll
    for (int e = 0; e < AA; ++e) f[e] = comp_of(m[e], k);
    wino::tile_output<A>(f, o);
    const float b = comp_of(bias, k);
#pragma unroll
    for (int e = 0; e < M * M; ++e) {
      float r = o[e];
      // (the caller passes a zero bias when the layer has none; adding it anyway can only turn a -0.0 into +0.0, which
      // the output quantization's multiply-add maps to the same value -- so only f32 output needs the condition,
      // which otherwise costs a select per value)
      if (OUT != EHIP_F32 || with_bias) r = r + b;
      if (OUT != EHIP_F32) r = __builtin_fmaf(r, repS, z);
      if (with_sum) r = r + old[k][e];
      // (u8 / s8 output: the ReLU is part of the clamp in front of the byte pack below)
      if (with_relu && OUT == EHIP_F32) r = r > 0.0f ? r : 0.0f;
      y[k][e] = r;
    }
  }
#pragma unroll
  for (int i = 0; i < M; ++i) {
    const int oh = M * th + i;
    if (oh >= oh_n) break;
#pragma unroll
    for (int j = 0; j < M; ++j) {
      const int ow = M * tw + j;
      if (ow >= ow_n) break;
      const int e = M * i + j;
      const size_t cell = ((size_t)oh * ow_n + ow) * px + 4 * q;   // element index inside the plane
      if (OUT == EHIP_F32) {
        {   // non-temporal: 200 MB of f32 output that nothing reads back soon (C4a 287 -> 261 us); the 4-byte
            // stores of u8 / s8 output, and the transformed input (read right after), lose with it.  The
            // 64-byte pieces (four lanes' 16 bytes) then reach memory one by one: the write counter reads 1.7 x
            // the output against 1.25 x with plain stores, and the kernel is still the faster one (C4a 251 vs
            // 277 us; without any output store 230 us: the write path is not what bounds it)
          typedef float v4f __attribute__((ext_vector_type(4)));
          const v4f vv = {y[0][e], y[1][e], y[2][e], y[3][e]};
          __builtin_nontemporal_store(vv, reinterpret_cast<v4f *>(static_cast<float *>(plane) + cell));
        }
      } else {
        unsigned o = 0u;
        if (with_relu) {
          // ReLU and the type's upper bound in one clamp (a NaN comes out of it as 0, like out of the ReLU's
          // comparison); what is left of the conversion -- rounding to nearest even, or the floor of F(2x2,3x3)
          // first -- is the byte pack's own, and floor and clamp commute
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            float r = __builtin_amdgcn_fmed3f(y[k][e], 0.0f, OUT == EHIP_S8 ? 127.0f : 255.0f);
            if (A == 4) r = __builtin_floorf(r);
            o = __builtin_amdgcn_cvt_pk_u8_f32(r, k, o);
          }
        } else
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const float r = y[k][e];
          if (A == 4) {
            // floor; u8 through an unsigned integer: negative values and NaN end as 255
            const float fl = __builtin_floorf(r);
            if (OUT == EHIP_U8) o = __builtin_amdgcn_cvt_pk_u8_f32(r >= 0.0f ? fl : 300.0f, k, o);
            else o |= ((unsigned)ssat8(cvt_s32_rne(fl)) & 0xffu) << (8 * k);
          } else {
            if (OUT == EHIP_U8) o = __builtin_amdgcn_cvt_pk_u8_f32(r >= -0.5f ? r : 300.0f, k, o);
            else o |= ((unsigned)ssat8(cvt_s32_rne(r)) & 0xffu) << (8 * k);
          }
        }
        *reinterpret_cast<unsigned *>(static_cast<uint8_t *>(plane) + cell) = o;
      }
    }
  }
}

// grid: (ceil(t / 64), oc2); block: 64 tiles x 4 channel quads
template <int OUT, int A = 6>
__global__ __launch_bounds__(kBlock) void k_wino_trans_output(WinoArgs a)
{
  constexpr int AA = A * A;
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
  float4 m[AA];
#pragma unroll
  for (int e = 0; e < AA; ++e) m[e] = src[e * pos_stride];

  float4 bias = make_float4(0.f, 0.f, 0.f, 0.f);
  if (a.with_bias) bias = reinterpret_cast<const float4 *>(a.bias)[o2 * 4 + q];
  const size_t plane = a.out_nhwc ? (size_t)n * a.oh * a.ow * a.oc2 * 16 + o2 * 16 : ((size_t)n * a.oc2 + o2) * a.oh * a.ow * 16;
  void *dst = OUT == EHIP_F32 ? static_cast<void *>(static_cast<float *>(a.out) + plane)
                              : static_cast<void *>(static_cast<uint8_t *>(a.out) + plane);
  output_tile<OUT, A>(m, bias, a.with_bias != 0, a.with_relu != 0, a.out_repS, a.out_z, dst, q, th, tw, a.oh, a.ow,
                      a.with_sum != 0, a.out_nhwc ? a.oc2 * 16 : 16);
}

// ---- the 36 GEMMs and the output transform in one kernel ----------------------------------------
// Replaces elx_int8_conv_wino_gemm_t::execute + trans_output as the reference's fused schedule does
// per thread (a161, src/elx_int8_conv_wino_xopt.hpp:21-179): the f32 GEMM result of a block of
// tiles never leaves the chip.  Written out it is 36/16 x 4 bytes per output value each way --
// more than twice the traffic of everything else in the layer together.
//
// A workgroup owns 64 output channels x 32 tiles at ALL 36 positions.  Each of its four waves
// takes nine positions and runs their GEMMs on v_mfma_i32_32x32x32_i8 with both operands loaded
// straight from memory into a register ring of KS k-steps (nothing is shared between waves, so
// there is no LDS traffic and no barrier in the main loop; a slot is refilled with the operand
// KS steps ahead as soon as its MFMAs are issued).  Then, for each half of the channels, the waves
// requantize their accumulators to f32 (the GEMM's own epilogue: fma(float(acc), scale, shift) per
// position and channel), exchange them through LDS -- 36 x 32 x 32 floats = 144 KB -- and every
// thread gathers the 36 values of one tile x four channels, applies Y = At M A + bias, ReLU, and
// stores its 4 x 4 pixels exactly like the stand-alone output transform.
//
// Workgroups are numbered so that the channel blocks of one tile block run next to each other on
// the same XCD (blockIdx.x % 8), where the second and later ones find the tiles in that XCD's L2.
// A: the tile size (6, 5, 4); its A x A positions are dealt to the four waves in runs of PW = ceil(A x A / 4): nine
// each for A = 6, four each for A = 4, and 7 + 7 + 7 + 4 for A = 5.
// SUM: the in-place sum (a compile-time copy: as a run-time flag in the common code it cost the layers without a
// sum 4 %, as copies behind a uniform branch twice their time -- the kernel sits at the edge of its registers).
// NT: blocks of 32 tiles per workgroup.  Tile size 4 has 16 positions, four per wave: its accumulators for 64
// channels x 32 tiles fill a quarter of the wave's registers, so a workgroup takes 64 tiles (a weight operand
// then feeds two MFMAs as a tile operand does: 1 KB of operands per MFMA instead of 1.5).
// NH: halves of 32 channels per workgroup, two unless the layer has so few tiles that 64-channel workgroups would
// leave CUs without one (256 -> 256 at 14 x 14, N = 64: 128 workgroups of 64 channels).
// NKSF: 0, or the k-steps of a position when they are fewer than the ring is deep (64 / 128 input channels: 2 / 4).
// The ring then runs ahead over the wave's positions as one flat sequence of steps -- with a ring of one position
// every position costs a trip to memory (64 -> 64: 36 MFMAs per wave in 16 K clocks).
template <int KS, int A = 6, bool SUM = false, int NT = 1, int NH = 2, int NKSF = 0>
__global__ __launch_bounds__(kBlock, 1) void k_wino_gemm_output(WinoFusedArgs a)
{
  constexpr int AA = A * A, PW = (AA + 3) / 4, CN = PW * 24, NJ = (CN + 63) / 64;
  extern __shared__ float4 xl[];   // [AA][32 tiles][8 cells of 4 channels], cell ^ ((tile / 2) & 7)
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  // (not through readfirstlane: with the operand addresses computed on the scalar unit the kernel measured 3 %
  // slower -- C4b 183.1 vs 177.9 us, C4a_i8 253.8 vs 247.1 us -- although a third of its vector instructions go)
  const int wave = tid >> 6;
  const int l32 = lane & 31;
  const int lh = lane >> 5;
  const int xcd = blockIdx.x & 7, seq = blockIdx.x >> 3;
  const int by = seq % a.ny;
  const int bx = (seq / a.ny) * 8 + xcd;
  if (bx >= a.nx) return;          // whole workgroup
  const int t0 = bx * 32 * NT, oc0 = by * 32 * NH;
  const int oc_real = a.oc2 * 16;
  const int p0 = PW * wave;
  // positions of this wave: all PW, except in the last wave when four runs of PW overshoot A x A (A = 5)
  constexpr bool EVEN = 4 * PW == AA;
  const int np = EVEN ? PW : (AA - p0 < PW ? AA - p0 : PW);
  const int nks = a.units_pad >> 1;   // k-steps (32 channels) per position
  const int nkc = nks / KS;

  // operand addresses = wave-uniform pointer (scalar arithmetic) + a per-lane 32-bit offset that
  // never changes: lane = packed row / tile l32 of unit 2 * ks + lh
  const unsigned a_lane = (unsigned)(lh * a.ocpp + l32) * 16u;
  // plain layout: tile `tile` of unit lh; blocked: cell l32 of unit lh inside the block's own run (cells of
  // tiles past the end hold nothing and are never stored; a block past the last one reads the last one)
  unsigned b_lane[NT];
  long long b_block[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    const int tile = t0 + 32 * j + l32 < a.t ? t0 + 32 * j + l32 : a.t - 1;
    b_lane[j] = a.tin_blocked ? (unsigned)(lh * 32 + l32) * 16u : (unsigned)(lh * a.t + tile) * 16u;
    const int nb32 = (a.t + 31) >> 5;
    b_block[j] = bx * NT + j < nb32 ? bx * NT + j : nb32 - 1;
  }
  const int ks_last = ((a.ic2 + 1) >> 1) - 1;   // last k-step that holds real channels

  TRACE_POINT(0);
  v4i ra[KS][NH], rb[KS][NT];
  auto issue = [&](int slot, int p, int ks) {
    const int8_t *pa = a.w + (((long long)p * a.units_pad + 2 * ks) * a.ocpp + oc0) * 16;
#pragma unroll
    for (int h = 0; h < NH; ++h) ra[slot][h] = *reinterpret_cast<const v4i *>(pa + 512 * h + a_lane);
    // padded k-steps multiply zero weights: any valid cell will do (an odd unit count reads one
    // unit past the position, which is the next position or the pad unit behind the buffer)
    const int ksc = ks < ks_last ? ks : ks_last;
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      const uint8_t *pb = a.tin_blocked ? a.tin + ((b_block[j] * AA + p) * a.ic2 + 2 * ksc) * 512
                                        : a.tin + ((long long)p * a.ic2 + 2 * ksc) * a.t * 16;
      rb[slot][j] = *reinterpret_cast<const v4i *>(pb + b_lane[j]);
    }
  };

  // Per-(position, channel) scale / shift / compensation of the wave's nine positions, one half of
  // the channels at a time: 27 rows of 32 dwords, staged in the 16 KB of LDS the exchange buffer
  // leaves free.  Read from there every lane pays one LDS broadcast per constant instead of a
  // global load instruction (which costs the address path as much as a full 1 KB load).
  float4 *cl = xl + AA * 32 * 8 + wave * CN;
  float4 cst[NJ];
  auto load_consts_half = [&](int h) {
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      int idx = lane + 64 * j;
      idx = idx < CN ? idx : CN - 1;
      const int row = idx >> 3, cell = idx & 7;
      const int i = row / 3, arr = row - 3 * i;
      const int p = p0 + i < AA ? p0 + i : AA - 1;   // (a wave with fewer positions: rows nobody reads)
      const float *src = arr == 0 ? a.scale : (arr == 1 ? a.shift : reinterpret_cast<const float *>(a.comp));
      cst[j] = *reinterpret_cast<const float4 *>(src + (long long)p * a.ocpp + oc0 + 32 * h + 4 * cell);
    }
  };
  auto store_consts_half = [&]() {
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const int idx = lane + 64 * j;
      cl[idx < CN ? idx : CN - 1] = cst[j];
    }
  };
  load_consts_half(0);
  store_consts_half();

  v16i acc[PW][NH][NT];
#pragma unroll
  for (int i = 0; i < PW; ++i)
#pragma unroll
    for (int h = 0; h < NH; ++h)
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][h][j][v] = 0;

  if constexpr (NKSF > 0) {
    // flat: step s = k-step s % NKSF of position s / NKSF, slot s % KS, refilled with step s + KS (positions past the
    // wave's last one -- tile size 5, last wave -- repeat it: their accumulators are never read)
    auto issue_step = [&](int slot, int sn) {
      int pi = sn / NKSF;
      pi = pi < np ? pi : np - 1;
      issue(slot, p0 + pi, sn % NKSF);
    };
#pragma unroll
    for (int k = 0; k < KS; ++k) issue_step(k, k);
#pragma unroll
    for (int s = 0; s < PW * NKSF; ++s) {
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        const v4i b = rb[s % KS][j] ^ (int)0x80808080;
#pragma unroll
        for (int h = 0; h < NH; ++h)
          acc[s / NKSF][h][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ra[s % KS][h], b, acc[s / NKSF][h][j], 0, 0, 0);
      }
      if (s + KS < PW * NKSF) issue_step(s % KS, s + KS);
    }
  } else {
#pragma unroll
  for (int k = 0; k < KS; ++k) issue(k, p0, k);
#pragma unroll
  for (int i = 0; i < PW; ++i) {
    for (int c = 0; c < (EVEN || i < np ? nkc : 0); ++c) {
#pragma unroll
      for (int k = 0; k < KS; ++k) {
#pragma unroll
        for (int j = 0; j < NT; ++j) {
          const v4i b = rb[k][j] ^ (int)0x80808080;
#pragma unroll
          for (int h = 0; h < NH; ++h)
            acc[i][h][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ra[k][h], b, acc[i][h][j], 0, 0, 0);
        }
        // refill the slot with the operands KS steps ahead (the very last block re-reads itself)
        int pn = p0 + i, ksn = (c + 1) * KS + k;
        if (ksn >= nks) { ksn -= nks; pn += 1; }
        if (pn > p0 + np - 1) { pn = p0 + np - 1; ksn = nks - KS + k; }
        issue(k, pn, ksn);
      }
    }
  }
  }

  if (NH > 1) load_consts_half(1);   // second half's constants travel while the first half is processed
  TRACE_POINT(1);
  // ---- requantize, exchange, output transform ----------------------------------------------------
  const int tile_l = tid >> 3, q8 = tid & 7;
#pragma unroll
  for (int h = 0; h < NH; ++h) {
#pragma unroll
   for (int j = 0; j < NT; ++j) {   // a round: 32 channels x 32 tiles through the exchange buffer
    const int t = t0 + 32 * j + tile_l;
    const int tc = t < a.t ? t : a.t - 1;
    const int n = tc / a.nt;
    const int rem = tc - n * a.nt;
    const int th = rem / a.wt;
    const int tw = rem - th * a.wt;
    if (h || j) __syncthreads();   // everyone has gathered the round before
    __builtin_amdgcn_wave_barrier();
    // constants of position i + 1 are read from LDS while position i is requantized
    float4 kq[2][12];
    auto read_consts = [&](int i, int slot) {
#pragma unroll
      for (int r = 0; r < 3; ++r)
#pragma unroll
        for (int q = 0; q < 4; ++q) kq[slot][4 * r + q] = cl[(3 * i + r) * 8 + 4 * lh + q];
    };
    read_consts(0, 0);
#pragma unroll
    for (int i = 0; i < PW; ++i) {
      const int p = p0 + i;
      if (i + 1 < PW) read_consts(i + 1, (i + 1) & 1);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        if (!EVEN && i >= np) continue;   // a position the last wave does not have
        const float4 sc = kq[i & 1][q], sh = kq[i & 1][4 + q], cf = kq[i & 1][8 + q];
        float4 r;
        r.x = __builtin_fmaf((float)(acc[i][h][j][4 * q + 0] + __float_as_int(cf.x)), sc.x, sh.x);
        r.y = __builtin_fmaf((float)(acc[i][h][j][4 * q + 1] + __float_as_int(cf.y)), sc.y, sh.y);
        r.z = __builtin_fmaf((float)(acc[i][h][j][4 * q + 2] + __float_as_int(cf.z)), sc.z, sh.z);
        r.w = __builtin_fmaf((float)(acc[i][h][j][4 * q + 3] + __float_as_int(cf.w)), sc.w, sh.w);
        xl[(p * 32 + l32) * 8 + ((4 * lh + q) ^ ((l32 >> 1) & 7))] = r;
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    __builtin_amdgcn_wave_barrier();
    if (NH > 1 && h == 0 && j == NT - 1) store_consts_half();   // the wave is done with the first half's constants
    TRACE_POINT(2 + 4 * h);
    __syncthreads();
    TRACE_POINT(3 + 4 * h);
    const int oc = oc0 + 32 * h + 4 * q8;
    if (t < a.t && oc < oc_real) {
      float4 m[AA];
#pragma unroll
      for (int e = 0; e < AA; ++e) m[e] = xl[(e * 32 + tile_l) * 8 + (q8 ^ ((tile_l >> 1) & 7))];
      float4 bias = make_float4(0.f, 0.f, 0.f, 0.f);
      if (a.with_bias) bias = *reinterpret_cast<const float4 *>(a.bias + oc);
      const size_t plane = a.out_nhwc ? (size_t)n * a.oh * a.ow * a.oc2 * 16 + (oc >> 4) * 16
                                      : ((size_t)n * a.oc2 + (oc >> 4)) * a.oh * a.ow * 16;
      const int px = a.out_nhwc ? a.oc2 * 16 : 16;
      const int q = (oc >> 2) & 3;
      TRACE_POINT(4 + 4 * h);
      if (a.out_type == EHIP_U8)
        output_tile<EHIP_U8, A>(m, bias, a.with_bias != 0, a.with_relu != 0, a.out_repS, a.out_z,
                                static_cast<uint8_t *>(a.out) + plane, q, th, tw, a.oh, a.ow, SUM, px);
      else if (a.out_type == EHIP_S8)
        output_tile<EHIP_S8, A>(m, bias, a.with_bias != 0, a.with_relu != 0, a.out_repS, a.out_z,
                                static_cast<uint8_t *>(a.out) + plane, q, th, tw, a.oh, a.ow, SUM, px);
      else
        output_tile<EHIP_F32, A>(m, bias, a.with_bias != 0, a.with_relu != 0, 0.f, 0.f, static_cast<float *>(a.out) + plane, q,
                                 th, tw, a.oh, a.ow, SUM, px);
    }
    TRACE_POINT(5 + 4 * h);
   }
  }
}

hipError_t launch_wino_trans_input(const WinoArgs &a0, hipStream_t s, LaunchPlan<WinoArgs> *plan)
{
  if (plan && plan->valid) {   // everything but the tensors is as on the first launch
    return plan_relaunch(*plan, [&](WinoArgs &x) { x.in = a0.in; }, s);
  }
  WinoArgs a = a0;
  {
    const unsigned long long bytes = (unsigned long long)a.n * a.ic2 * a.ih * a.iw * 16 * (a.in_u8 ? 1 : 4);
    const char *env = getenv("EHIP_WINO_BUF_GATHER");
    a.buf_gather = bytes <= 0xffffff00ull && !(env && env[0] == '0');
    const char *wide = getenv("EHIP_WINO_WIDE_GATHER");
    if (a.buf_gather && a.in_u8 && !(wide && wide[0] == '0')) a.buf_gather = 2;   // whole cells and a transpose inside the quad
  }
  a.nblocks = (a.t + 63) / 64;
  a.items_per_xcd = (int)(((long long)a.nblocks * a.ic2 + 7) / 8);
  dim3 grid(8 * a.items_per_xcd, 1);
  void (*kern)(WinoArgs) = nullptr;
  if (a.tile == 4) kern = a.in_u8 ? k_wino_trans_input_u8<unsigned, 4> : k_wino_trans_input_u8<float4, 4>;
  else if (a.tile == 5) kern = a.in_u8 ? k_wino_trans_input_u8<unsigned, 5> : k_wino_trans_input_u8<float4, 5>;
  else kern = a.in_u8 ? k_wino_trans_input_u8<unsigned, 6> : k_wino_trans_input_u8<float4, 6>;
  return plan_launch(plan, kern, grid, dim3(kBlock), 0, a, s);
}

hipError_t launch_wino_trans_output(const WinoArgs &a, hipStream_t s, LaunchPlan<WinoArgs> *plan)
{
  if (plan && plan->valid) {   // everything but the tensors is as on the first launch
    return plan_relaunch(*plan, [&](WinoArgs &x) { x.out = a.out; x.bias = a.bias; }, s);
  }
  dim3 grid((a.t + 63) / 64, a.oc2);
  void (*kern)(WinoArgs) = nullptr;
#define EHIP_WO(A)                                                                                         \
  kern = a.out_type == EHIP_U8 ? k_wino_trans_output<EHIP_U8, A>                                           \
      : (a.out_type == EHIP_S8 ? k_wino_trans_output<EHIP_S8, A> : k_wino_trans_output<EHIP_F32, A>)
  if (a.tile == 4) EHIP_WO(4);
  else if (a.tile == 5) EHIP_WO(5);
  else EHIP_WO(6);
#undef EHIP_WO
  return plan_launch(plan, kern, grid, dim3(kBlock), 0, a, s);
}

// k-steps per ring block: the largest of 8, 4, 2 that divides the k-steps of a position
hipError_t launch_wino_gemm_output(const WinoFusedArgs &a0, hipStream_t s, LaunchPlan<WinoFusedArgs> *plan)
{
  if (plan && plan->valid) {   // everything but the tensors is as on the first launch
    return plan_relaunch(*plan, [&](WinoFusedArgs &x) { x.out = a0.out; x.bias = a0.bias; }, s);
  }
  WinoFusedArgs a = a0;
  const int A = a.tile ? a.tile : 6, AA = A * A;
  if (wino_lanes_applies(a)) return launch_wino_gemm_output_lanes(a, s, plan);
  const int ntb = A == 4 ? 2 : 1;   // blocks of 32 tiles per workgroup
  a.nx = (a.t + 32 * ntb - 1) / (32 * ntb);
  // 64 channels per workgroup; 32 where that would leave a quarter of the CUs or more without a workgroup
  int nh = 2;
  if (ntb == 1 && (long long)a.nx * ((a.oc2 * 16 + 63) / 64) <= 192 && a.oc2 * 16 > 32) nh = 1;
  if (const char *env = getenv("EHIP_WINO_HALVES")) if (ntb == 1 && (env[0] == '1' || env[0] == '2')) nh = env[0] - '0';
  a.ny = (a.oc2 * 16 + 32 * nh - 1) / (32 * nh);
  const int nks = a.units_pad / 2;
  const size_t lds = (size_t)AA * 32 * 32 * sizeof(float) + 4 * (size_t)((AA + 3) / 4 * 24) * sizeof(float4);   // exchange + constants
  dim3 grid(8 * a.ny * ((a.nx + 7) / 8));
  // operand ring depth in k-steps.  Measured (C4a / C4b / C4a_i8 / C4b_i8, us): 8 deep 261.7 / 177.3 / 247.6 /
  // 178.6, 4 deep 250.4 / 172.8 / 241.2 / 176.5, 2 deep 286.8 / 215.6 (f32 layers)
  int ks_max = 4;
  if (const char *env = getenv("EHIP_WINO_KS")) ks_max = atoi(env);
  bool flat = true;   // 64 / 128 input channels: the ring runs ahead over positions
  if (const char *env = getenv("EHIP_WINO_FLAT")) flat = env[0] != '0';
  void (*kernel)(WinoFusedArgs) = nullptr;
#define EHIP_WF1(AV, SV, NHV)                                                                          \
  kernel = (nks == 2 && flat) ? k_wino_gemm_output<8, AV, SV, AV == 4 ? 2 : 1, NHV, 2>                  \
      : (nks == 4 && flat) ? k_wino_gemm_output<8, AV, SV, AV == 4 ? 2 : 1, NHV, 4>                     \
      : (nks % 8 == 0 && ks_max >= 8) ? k_wino_gemm_output<8, AV, SV, AV == 4 ? 2 : 1, NHV>          \
      : ((nks % 4 == 0 && ks_max >= 4) ? k_wino_gemm_output<4, AV, SV, AV == 4 ? 2 : 1, NHV>            \
                                       : k_wino_gemm_output<2, AV, SV, AV == 4 ? 2 : 1, NHV>)
#define EHIP_WF(AV, SV)                                                                                 \
  do {                                                                                                  \
    if (AV != 4 && nh == 1) EHIP_WF1(AV, SV, (AV != 4 ? 1 : 2));                                        \
    else EHIP_WF1(AV, SV, 2);                                                                           \
  } while (0)
  if (a.with_sum) {
    if (A == 4) EHIP_WF(4, true);
    else if (A == 5) EHIP_WF(5, true);
    else EHIP_WF(6, true);
  } else {
    if (A == 4) EHIP_WF(4, false);
    else if (A == 5) EHIP_WF(5, false);
    else EHIP_WF(6, false);
  }
#undef EHIP_WF
#undef EHIP_WF1
  if (nks % 2 != 0) return hipErrorInvalidValue;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) return e;
  return plan_launch(plan, kernel, grid, dim3(kBlock), lds, a, s);
}

// partials: 2 * a.ic2 dwords of device memory; minmax_out_dev: two floats of device memory
hipError_t launch_wino_range(const WinoArgs &a, int ic_real, unsigned *partials, float *minmax_out_dev, hipStream_t s)
{
  hipLaunchKernelGGL(k_wino_range_init, dim3((2 * a.ic2 + kBlock - 1) / kBlock), dim3(kBlock), 0, s, partials, a.ic2);
  dim3 grid((a.t + 63) / 64, a.ic2);
  void (*kern)(WinoArgs, int, unsigned *) = nullptr;
  if (a.tile == 4) kern = a.in_u8 ? k_wino_tinput_range<unsigned, 4> : k_wino_tinput_range<float4, 4>;
  else if (a.tile == 5) kern = a.in_u8 ? k_wino_tinput_range<unsigned, 5> : k_wino_tinput_range<float4, 5>;
  else kern = a.in_u8 ? k_wino_tinput_range<unsigned, 6> : k_wino_tinput_range<float4, 6>;
  hipLaunchKernelGGL(kern, grid, dim3(kBlock), 0, s, a, ic_real, partials);
  hipLaunchKernelGGL(k_wino_range_finish, dim3(1), dim3(kWave), 0, s, partials, a.ic2, minmax_out_dev);
  return hipGetLastError();
}

// ---- the range without an allocation ------------------------------------------------------------
// The per-unit partial results of the range live in this array instead of in memory from hipMalloc.
// Every GPU of the process holds its own copy at its own address; host code never uses the array's
// name as a pointer, only the address hipGetSymbolAddress returned for the device in question.
static __device__ __align__(256) unsigned scratch[2 * kRangeScratchUnits];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
unsigned *g_scratch_ptr[kMaxDevices];   // by device ordinal; null until resolved
}  // namespace

hipError_t wino_range_scratch(unsigned **ptr)
{
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void *p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return e;
    if (!p) return hipErrorInvalidSymbol;
    g_scratch_ptr[dev] = static_cast<unsigned *>(p);
  }
  *ptr = g_scratch_ptr[dev];
  return hipSuccess;
}

}  // namespace ehip
