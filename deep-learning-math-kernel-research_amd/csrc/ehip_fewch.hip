// k x k direct convolution of an input with at most four channels: the first layer of an image
// network (7x7 s2 3->64, 3x3 s2 3->32, ... -- the reference runs them as direct convolutions over a
// 3-channel nhwc input, scripts/best_configs/resnetv1_5-n64-clx-1s-int8.sh:12,
// scripts/best_configs/mobilenetv1-n64-clx-1s-int8.sh:8, executor src/elx_int8_conv_direct.cpp:227-423).
//
// With so few channels a 16-byte MFMA operand cell holds ppc = 16 / ic horizontally adjacent pixels
// (ic bytes each), so a kernel row is nu = ceil(kw / ppc) cells instead of kw and the whole kernel
// kh * nu cells (14 for 7x7x3, 3 for 3x3x3): the weights of 32 output channels fit in registers.
// A workgroup takes a strip of output rows of one image:
//   1. the input rows under the strip go to LDS once, as compact rows of ic bytes per pixel with
//      the left / right padding filled in (u8 0, which contributes nothing), already remapped to s8;
//      nhwc input is compact in memory as well, so LDS dword d of a row is one aligned global dword
//      (the row keeps its byte phase), masked at the row's ends;
//   2. a wave walks over 32-pixel tiles of the strip: a lane's cell is 16 consecutive LDS bytes at
//      a byte address of any alignment, read as five dwords and shifted into place;
//   3. kh * nu / 2 MFMAs per tile against the weights in registers, then the shared epilogue.
// The four waves split into a.wo channel tiles x 4 / a.wo pixel tiles.
#include "ehip_internal.hpp"

namespace ehip {

namespace {
__device__ __forceinline__ unsigned low_bytes(long long k)   // mask of the k lowest bytes, k clamped to 0..4
{
  return k <= 0 ? 0u : k >= 4 ? 0xffffffffu : (1u << (8 * (int)k)) - 1u;
}
}  // namespace

template <int KS>
__global__ __launch_bounds__(kBlock, 2) void k_conv_fewch_u8s8(FewChArgs a)
{
  extern __shared__ unsigned rows_lds[];   // [nrows_in][lrow / 4]
  __shared__ v4i xpatch[4 * 256];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int l32 = lane & 31;
  const int lh = lane >> 5;
  const int img = blockIdx.x / a.strips, strip = blockIdx.x - img * a.strips;
  const int oh0 = strip * a.rows;
  const int rows_valid = a.oh - oh0 < a.rows ? a.oh - oh0 : a.rows;
  const int npix = rows_valid * a.ow;
  const int ihb = oh0 * a.stride_h - a.pad_t;   // input row of staged row 0
  const int lrow4 = a.lrow >> 2;
  const int rowbytes = a.iw * a.ic;

  // ---- 1. stage the input rows --------------------------------------------------------------
  // byte 0 of a staged row = pixel -pad_l of the input row (+ the row's phase for nhwc input)
  const long long g00 = ((long long)(img * a.ih + ihb) * a.iw - a.pad_l) * a.ic;   // nhwc: global byte of staged (0, 0)
  if (a.in_nhwc) {
    for (int idx = tid; idx < a.nrows_in * lrow4; idx += kBlock) {
      const int r = fastdiv(idx, lrow4, a.lrow4_magic);
      const int d = idx - r * lrow4;
      const int h = ihb + r;
      unsigned v = 0u;
      if (h >= 0 && h < a.ih) {
        const long long g0 = g00 + (long long)r * rowbytes;
        const long long rs = g0 + a.pad_l * a.ic;           // first byte of the input row
        const long long ga = g0 - (g0 & 3) + 4 * d;         // the aligned global dword behind LDS dword d
        const long long lo = rs - ga, hi = rs + rowbytes - ga;   // its bytes lo .. hi - 1 belong to the row
        if (hi > 0 && lo < 4)
          v = *reinterpret_cast<const unsigned *>(a.in + ga) & low_bytes(hi) & ~low_bytes(lo);
      }
      rows_lds[idx] = v ^ 0x80808080u;
    }
  } else {
    for (int idx = tid; idx < a.nrows_in * lrow4; idx += kBlock) rows_lds[idx] = 0x80808080u;
    __syncthreads();
    uint8_t *lb = reinterpret_cast<uint8_t *>(rows_lds);
    for (int idx = tid; idx < a.nrows_in * a.iw; idx += kBlock) {
      const int r = fastdiv(idx, a.iw, a.iw_magic);
      const int x = idx - r * a.iw;
      const int h = ihb + r;
      if (h >= 0 && h < a.ih) {
        const unsigned v = *reinterpret_cast<const unsigned *>(a.in + ((long long)(img * a.ih + h) * a.iw + x) * 16) ^ 0x80808080u;
        for (int c = 0; c < a.ic; ++c) lb[r * a.lrow + (x + a.pad_l) * a.ic + c] = (uint8_t)(v >> (8 * c));
      }
    }
  }
  __syncthreads();

  // ---- 2. / 3. tiles --------------------------------------------------------------------------
  const int wo = wave % a.wo, wp = wave / a.wo, wpn = 4 / a.wo;
  const int oc0 = (blockIdx.y * a.wo + wo) * 32;
  const int oc_real = a.oc2 * 16;
  const int ohw = a.oh * a.ow;
  v4i wreg[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks)
    wreg[ks] = *reinterpret_cast<const v4i *>(a.w + ((long long)(2 * ks + lh) * a.ocpp + oc0 + l32) * 16);
  // the lane's cells: 2 ks + lh = kernel row * nu + unit, clamped to the real ones (the weights
  // behind them are zero)
  int cell_row[KS], cell_off[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    int tc = 2 * ks + lh;
    tc = tc < a.cells ? tc : a.cells - 1;
    cell_row[ks] = tc / a.nu;
    cell_off[ks] = (tc - cell_row[ks] * a.nu) * a.ppc * a.ic;
  }
  const int phase0 = a.in_nhwc ? (int)(g00 & 3) : 0;
  const int phase_step = a.in_nhwc ? rowbytes & 3 : 0;

  const long long cidx = oc0 + 16 * lh;
  OcConsts k0;
  load_consts(k0, a.ep, cidx);
  v4i *xlds = ((a.ep.out_type == EHIP_F32 || a.ep.out_type == EHIP_S32) && !a.out_nhwc) ? xpatch + wave * 256 : nullptr;
  const long long gp0 = (long long)img * ohw + (long long)oh0 * a.ow;   // the strip's first output pixel
  auto pixel_offset = [&](int p, bool &valid) -> size_t {
    valid = p < npix;
    const int pv = valid ? p : 0;
    if (a.out_nhwc) return (size_t)(gp0 + pv) * oc_real;
    return ((size_t)img * a.oc2 * ohw + (size_t)oh0 * a.ow + pv) * 16;
  };
  const int ntiles = (npix + 31) >> 5;
  for (int tile = wp; tile < ntiles; tile += wpn) {
    int p = tile * 32 + l32;
    p = p < npix ? p : npix - 1;
    const int ro = fastdiv(p, a.ow, a.ow_magic);
    const int ox = p - ro * a.ow;
    const int row0 = ro * a.stride_h;
    const int xbyte = ox * a.stride_w * a.ic;
    v16i acc[1][1];
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[0][0][v] = 0;
    v4i b[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int row = row0 + cell_row[ks];
      const int A = row * a.lrow + ((phase0 + row * phase_step) & 3) + xbyte + cell_off[ks];
      const unsigned *src = rows_lds + (A >> 2);
      const unsigned sh = A & 3;
      const unsigned d0 = src[0], d1 = src[1], d2 = src[2], d3 = src[3], d4 = src[4];
      b[ks] = v4i{(int)__builtin_amdgcn_alignbyte(d1, d0, sh), (int)__builtin_amdgcn_alignbyte(d2, d1, sh),
                  (int)__builtin_amdgcn_alignbyte(d3, d2, sh), (int)__builtin_amdgcn_alignbyte(d4, d3, sh)};
    }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) acc[0][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wreg[ks], b[ks], acc[0][0], 0, 0, 0);
    size_t pix[1], pixT[1][2];
    bool pvalid[1], validT[1][2];
    int cls[1] = {0};
    pix[0] = pixel_offset(tile * 32 + l32, pvalid[0]);
    pixT[0][0] = pixel_offset(tile * 32 + (lane >> 2), validT[0][0]);
    pixT[0][1] = pixel_offset(tile * 32 + (lane >> 2) + 16, validT[0][1]);
    if (a.ep.shift_tab) cls[0] = a.cls_h[oh0 + ro] * a.ncls_w + a.cls_w[ox];
    epilogue_wave<1, 1, true>(a.ep, acc, k0, cidx, oc0 + 16 * lh, pix, pvalid, oc_real,
                              a.out_nhwc ? (size_t)16 : (size_t)ohw * 16, a.out, xlds, pixT, validT, cls);
  }
}

bool conv_fewch_applies(int ic, int kh, int kw)
{
  if (ic < 1 || ic > 4 || kh * kw <= 1 || kw < 2) return false;
  const int ppc = 16 / ic, nu = (kw + ppc - 1) / ppc;
  return kh * nu <= 14;
}

// pitch in bytes of a staged input row: pad_l + iw pixels or the last output pixel's last cell
// (16 bytes), whichever ends later, + 3 bytes of phase + 4 for the fifth dword of a shifted cell
int conv_fewch_row_pitch(int ic, int kw, int iw, int ow, int stride_w, int pad_l)
{
  const int ppc = 16 / ic, nu = (kw + ppc - 1) / ppc;
  int need = (pad_l + iw) * ic;
  const int last = ((ow - 1) * stride_w + (nu - 1) * ppc) * ic + 16;
  if (last > need) need = last;
  return up(need + 3 + 4, 4) + 4;
}

// Fills the derived fields (cells, strip height, LDS row pitch, wave split) and launches.
// Expects in a: tensors, epilogue, n, ih, iw, oh, ow, ic, kh, kw, strides, pads, oc2, ocpp, formats, classes.
hipError_t launch_conv_fewch(FewChArgs &a, hipStream_t s)
{
  a.ppc = 16 / a.ic;
  a.nu = (a.kw + a.ppc - 1) / a.ppc;
  a.cells = a.kh * a.nu;
  if (!conv_fewch_applies(a.ic, a.kh, a.kw)) return hipErrorInvalidValue;
  if (a.in_nhwc && (reinterpret_cast<uintptr_t>(a.in) & 3)) return hipErrorInvalidValue;   // aligned dword loads
  a.lrow = conv_fewch_row_pitch(a.ic, a.kw, a.iw, a.ow, a.stride_w, a.pad_l);
  const int octiles = up(a.oc2 * 16, 32) / 32;   // <= ocpp / 32
  a.wo = octiles % 4 == 0 ? 4 : octiles % 2 == 0 ? 2 : 1;
  const int gy = octiles / a.wo, wpn = 4 / a.wo;
  // strip height: as many rows as keep about three workgroups per CU in the grid, every wave busy,
  // and the staged rows inside 48 KB
  int rows = 1;
  const char *env = getenv("EHIP_FEWCH_ROWS");
  if (env && env[0]) {
    rows = atoi(env);
  } else {
    for (int r = 1; r <= a.oh && r <= 16; ++r) {
      if ((size_t)((r - 1) * a.stride_h + a.kh) * a.lrow > 48 * 1024) break;
      const long long wgs = (long long)a.n * ((a.oh + r - 1) / r) * gy;
      if (r > 1 && wgs < 768) break;
      rows = r;
      if ((r * a.ow + 31) / 32 >= 8 * wpn && (r * a.ow) % 32 == 0) break;
    }
  }
  if (rows < 1) rows = 1;
  if (rows > a.oh) rows = a.oh;
  a.rows = rows;
  a.strips = (a.oh + rows - 1) / rows;
  a.nrows_in = (rows - 1) * a.stride_h + a.kh;
  const size_t lds = (size_t)a.nrows_in * a.lrow + 32;
  if (lds > 48 * 1024 + 64 || (long long)a.nrows_in * a.lrow >= (1ll << 30) || (long long)rows * a.ow * a.ow >= (1ll << 32))
    return hipErrorInvalidValue;
  a.ow_magic = div_magic(a.ow);
  a.iw_magic = div_magic(a.iw);
  a.lrow4_magic = div_magic(a.lrow / 4);
  if ((long long)a.nrows_in * (a.lrow / 4) * (a.lrow / 4) >= (1ll << 32) || (long long)a.nrows_in * a.iw * a.iw >= (1ll << 32))
    return hipErrorInvalidValue;
  const int ks = (a.cells + 1) / 2;
  void (*kern)(FewChArgs) = ks <= 2 ? k_conv_fewch_u8s8<2> : ks == 3 ? k_conv_fewch_u8s8<3> : ks == 4 ? k_conv_fewch_u8s8<4>
      : ks == 5 ? k_conv_fewch_u8s8<5> : k_conv_fewch_u8s8<7>;
  hipLaunchKernelGGL(kern, dim3(a.n * a.strips, gy), dim3(kBlock), lds, s, a);
  return hipGetLastError();
}

}  // namespace ehip
