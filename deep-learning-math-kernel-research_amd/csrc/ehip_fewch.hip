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
//      nhwc input is compact in memory as well: a staged dword is two aligned global dwords shifted
//      together (rows start at any byte), masked at the row's ends;
//   2. a wave walks over 32-pixel tiles of the strip: a lane's cell is 16 consecutive LDS bytes at
//      a byte address of any alignment, read as five dwords and shifted into place;
//   3. kh * nu / 2 MFMAs per tile against the weights in registers, then the shared epilogue.
// The four waves split into a.wo channel tiles x 4 / a.wo pixel tiles.
#include "ehip_internal.hpp"

namespace ehip {

namespace {
__device__ __forceinline__ unsigned low_bytes(int k)   // mask of the k lowest bytes, k clamped to 0..4 (no branches)
{
  k = k < 0 ? 0 : k > 4 ? 4 : k;
  return (unsigned)((1ull << (8 * k)) - 1ull);
}
}  // namespace

// Section 1 of both kernels: the input rows under the strip (and, with a.tab_lds, the border-class tables and
// the shift rows of the workgroup's channels) go to LDS.  The caller synchronises.
struct FewChTables {
  float *shift;      // [class][wo * 32]
  int *cls_h, *cls_w;   // class of each of the strip's output rows (times ncls_w) / of each output column
};
__device__ __forceinline__ FewChTables fewch_stage(const FewChArgs &a, unsigned *rows_lds, int tid, int img, int ihb,
                                                   int oh0, int rows_valid)
{
  const int lrow4 = a.lrow >> 2;
  const int rowbytes = a.iw * a.ic;

  // ---- 1. stage the input rows --------------------------------------------------------------
  // byte 0 of a staged row = pixel -pad_l of the input row.
  // nhwc: byte offsets inside the image fit an int; the image starts at in + img_off, of which the
  // 4-byte aligned part goes into the pointer and the rest (e0) into the offsets.  A staged dword is
  // four consecutive bytes of the row at whatever alignment they have in memory: two aligned dwords
  // shifted together.
  const long long img_off = (long long)img * a.ih * a.iw * a.ic;
  const int e0 = (int)(img_off & 3);
  const uint8_t *const in_al = a.in + (img_off - e0);
  const int g00 = (ihb * a.iw - a.pad_l) * a.ic + e0;   // byte of staged (0, 0) relative to in_al
  const int last_dw = (e0 + a.ih * rowbytes - 1) & ~3;   // the last aligned dword with a byte of this image
  // Loads are issued kStageDepth at a time, unconditionally (outside the row: a clamped address and
  // an empty mask), before the first of them is stored: a workgroup waits for memory once per
  // batch, not once per dword.
  constexpr int kStageDepth = 8;
  float *const lds_shift = reinterpret_cast<float *>(rows_lds) + a.tab_lds;   // 16-byte aligned
  int *const lds_cls_h = reinterpret_cast<int *>(lds_shift + a.nclass * a.wo * 32);
  int *const lds_cls_w = lds_cls_h + a.rows;
  // With border classes: the class of each of the strip's rows and of each column, and the shift rows of the
  // workgroup's channels (a pixel's shift row is looked up per tile: two dependent trips to memory if the tables
  // stayed there).  Their loads go out HERE, up to sixteen per thread, and are stored behind the staging of the input
  // rows: one trip to memory for both (one load at a time, the up to 49 rows of a 7 x 7 layer were twelve trips one
  // after the other at the head of every workgroup).
  constexpr int kTabHold = 16;
  const int width = a.wo * 32, wshift = a.wo == 4 ? 7 : (a.wo == 2 ? 6 : 5);   // width = 1 << wshift
  const int cells = a.tab_lds ? a.nclass * width : 0;
  auto tab_cell = [&](int idx) -> float {
    const int c = idx >> wshift;
    return a.ep.shift_tab[(size_t)c * a.ep.tab_stride + blockIdx.y * width + (idx - (c << wshift))];
  };
  float tab_held[kTabHold];
  int cls_h_held = 0, cls_w_held = 0;
  if (a.tab_lds) {
    cls_h_held = a.cls_h[oh0 + (tid < rows_valid ? tid : 0)] * a.ncls_w;
    cls_w_held = a.cls_w[tid < a.ow ? tid : 0];
#pragma unroll
    for (int u = 0; u < kTabHold; ++u) {
      const int idx = u * kBlock + tid;
      tab_held[u] = tab_cell(idx < cells ? idx : cells - 1);
      if ((u + 1) * kBlock >= cells) break;   // uniform
    }
  }
  auto store_tables = [&]() {
    if (!a.tab_lds) return;
    if (tid < rows_valid) lds_cls_h[tid] = cls_h_held;
    if (tid < a.ow) lds_cls_w[tid] = cls_w_held;
    for (int idx = tid + kBlock; idx < rows_valid; idx += kBlock) lds_cls_h[idx] = a.cls_h[oh0 + idx] * a.ncls_w;
    for (int idx = tid + kBlock; idx < a.ow; idx += kBlock) lds_cls_w[idx] = a.cls_w[idx];
#pragma unroll
    for (int u = 0; u < kTabHold; ++u) {
      const int idx = u * kBlock + tid;
      if (idx < cells) lds_shift[idx] = tab_held[u];
      if ((u + 1) * kBlock >= cells) break;   // uniform
    }
    for (int idx = kTabHold * kBlock + tid; idx < cells; idx += kBlock) lds_shift[idx] = tab_cell(idx);
  };
  if (a.in_nhwc && a.icl != a.ic) {
    // Three channels staged as four bytes.  A thread takes four pixels: their twelve bytes, wherever they lie, come
    // out of four aligned dwords shifted together, and go to LDS as the four staged dwords at once (a staged row is
    // a whole number of such groups; group q of a row = pixels 4 q - pad_l ...).  Dwords outside the image hold
    // nothing of these pixels: any address inside will do for them.
    constexpr int kGroupDepth = 2;
    const int lrow16 = a.lrow >> 4;
    const int total = a.nrows_in * lrow16;
    for (int base = 0; base < total; base += kBlock * kGroupDepth) {
      unsigned v[kGroupDepth][4];
      int x0[kGroupDepth], sft[kGroupDepth];
      bool inside[kGroupDepth];
#pragma unroll
      for (int u = 0; u < kGroupDepth; ++u) {
        int idx = base + u * kBlock + tid;
        idx = idx < total ? idx : total - 1;
        const int r = fastdiv(idx, lrow16, a.lrow16_magic);
        const int h = ihb + r;
        x0[u] = 4 * (idx - r * lrow16) - a.pad_l;
        inside[u] = (unsigned)h < (unsigned)a.ih;
        const int g = e0 + (h * a.iw + x0[u]) * 3;
        sft[u] = g & 3;
        const int ga = g & ~3;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          int at = ga + 4 * k;
          at = at < 0 ? 0 : at > last_dw ? last_dw : at;
          v[u][k] = *reinterpret_cast<const unsigned *>(in_al + (unsigned)at);
        }
      }
#pragma unroll
      for (int u = 0; u < kGroupDepth; ++u) {
        const int idx = base + u * kBlock + tid;
        const unsigned p0 = __builtin_amdgcn_alignbyte(v[u][1], v[u][0], sft[u]);
        const unsigned p1 = __builtin_amdgcn_alignbyte(v[u][2], v[u][1], sft[u]);
        const unsigned p2 = __builtin_amdgcn_alignbyte(v[u][3], v[u][2], sft[u]);
        const unsigned px[4] = {p0, __builtin_amdgcn_alignbyte(p1, p0, 3), __builtin_amdgcn_alignbyte(p2, p1, 2), p2 >> 8};
        uint4 o;
        unsigned *const ov = reinterpret_cast<unsigned *>(&o);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const bool ok = inside[u] && (unsigned)(x0[u] + j) < (unsigned)a.iw;
          ov[j] = (px[j] & (ok ? 0x00ffffffu : 0u)) ^ 0x80808080u;
        }
        if (idx < total) *reinterpret_cast<uint4 *>(rows_lds + 4 * idx) = o;
      }
    }
  } else if (a.in_nhwc) {
    const int total = a.nrows_in * lrow4;
    for (int base = 0; base < total; base += kBlock * kStageDepth) {
      unsigned v[kStageDepth], v2[kStageDepth], m[kStageDepth], sft[kStageDepth];
#pragma unroll
      for (int u = 0; u < kStageDepth; ++u) {
        int idx = base + u * kBlock + tid;
        idx = idx < total ? idx : total - 1;
        const int r = fastdiv(idx, lrow4, a.lrow4_magic);
        const int d = idx - r * lrow4;
        const int h = ihb + r;
        const bool inside = (unsigned)h < (unsigned)a.ih;
        const int g = g00 + r * rowbytes + 4 * d;   // first byte of the staged dword
        const int rs = g00 + r * rowbytes + a.pad_l * a.ic;   // first byte of the input row
        const int lo = rs - g, hi = rs + rowbytes - g;        // bytes lo .. hi - 1 of the dword belong to the row
        m[u] = inside ? low_bytes(hi) & ~low_bytes(lo) : 0u;
        // dwords outside the image hold nothing of the row: any address inside will do for them
        int ga = g & ~3, gb = ga + 4;
        ga = ga < 0 ? 0 : ga > last_dw ? last_dw : ga;
        gb = gb < 0 ? 0 : gb > last_dw ? last_dw : gb;
        v[u] = *reinterpret_cast<const unsigned *>(in_al + ga);
        v2[u] = *reinterpret_cast<const unsigned *>(in_al + gb);
        sft[u] = g & 3;
      }
#pragma unroll
      for (int u = 0; u < kStageDepth; ++u) {
        const int idx = base + u * kBlock + tid;
        if (idx < total) rows_lds[idx] = (__builtin_amdgcn_alignbyte(v2[u], v[u], sft[u]) & m[u]) ^ 0x80808080u;
      }
    }
  } else {
    for (int idx = tid; idx < a.nrows_in * lrow4; idx += kBlock) rows_lds[idx] = 0x80808080u;
    __syncthreads();
    uint8_t *lb = reinterpret_cast<uint8_t *>(rows_lds);
    const int total = a.nrows_in * a.iw;
    for (int base = 0; base < total; base += kBlock * kStageDepth) {
      unsigned v[kStageDepth];
      int at[kStageDepth];   // LDS byte of the pixel, -1: nothing to store
#pragma unroll
      for (int u = 0; u < kStageDepth; ++u) {
        int idx = base + u * kBlock + tid;
        const bool in_range = idx < total;
        idx = in_range ? idx : total - 1;
        const int r = fastdiv(idx, a.iw, a.iw_magic);
        const int x = idx - r * a.iw;
        const int h = ihb + r;
        const bool inside = in_range && h >= 0 && h < a.ih;
        at[u] = inside ? r * a.lrow + (x + a.pad_l) * a.icl : -1;
        v[u] = *reinterpret_cast<const unsigned *>(a.in + (inside ? ((long long)(img * a.ih + h) * a.iw + x) * 16 : 0));
      }
#pragma unroll
      for (int u = 0; u < kStageDepth; ++u)
        if (at[u] >= 0) {
          const unsigned q = v[u] ^ 0x80808080u;
#pragma unroll
          for (int c = 0; c < 4; ++c)
            if (c < a.ic) lb[at[u] + c] = (uint8_t)(q >> (8 * c));
        }
    }
  }
  store_tables();
  return FewChTables{lds_shift, lds_cls_h, lds_cls_w};
}

template <int KS>
__global__ __launch_bounds__(kBlock, 3) void k_conv_fewch_u8s8(FewChArgs a)
{
  // [nrows_in][lrow / 4] staged rows; with border classes kept on chip (a.tab_lds): the shift rows of
  // the workgroup's channels [class][wo * 32], then the class of each of the strip's output rows
  // (times ncls_w) and of each output column
  extern __shared__ unsigned rows_lds[];
  __shared__ v4i xpatch[4 * 256];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform: what depends on it stays scalar
  const int l32 = lane & 31;
  const int lh = lane >> 5;
  const int img = blockIdx.x / a.strips, strip = blockIdx.x - img * a.strips;
  const int oh0 = strip * a.rows;
  const int rows_valid = a.oh - oh0 < a.rows ? a.oh - oh0 : a.rows;
  const int npix = rows_valid * a.ow;
  const int ihb = oh0 * a.stride_h - a.pad_t;   // input row of staged row 0
  const FewChTables tabs = fewch_stage(a, rows_lds, tid, img, ihb, oh0, rows_valid);
  float *const lds_shift = tabs.shift;
  int *const lds_cls_h = tabs.cls_h, *const lds_cls_w = tabs.cls_w;
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
  int cell_at[KS];   // LDS byte of the cell relative to the pixel's first cell
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    int tc = 2 * ks + lh;
    tc = tc < a.cells ? tc : a.cells - 1;
    const int kr = tc / a.nu;
    cell_at[ks] = kr * a.lrow + (tc - kr * a.nu) * a.ppc * a.icl;
  }

  const long long cidx = oc0 + 16 * lh;
  OcConsts k0;
  load_consts(k0, a.ep, cidx);
  // the on-chip shift rows get an epilogue of their own: one whose table pointer can only be LDS
  Epilogue ep_lds = a.ep;
  ep_lds.shift_tab = lds_shift;
  ep_lds.tab_stride = a.wo * 32;
  v4i *xlds = ((a.ep.out_type == EHIP_F32 || a.ep.out_type == EHIP_S32) && !a.out_nhwc) ? xpatch + wave * 256 : nullptr;
  // the accumulators start from the u8 -> s8 compensation of the lane's channels
  v16i comp0;
#pragma unroll
  for (int v = 0; v < 16; ++v) comp0[v] = k0.comp[v >> 2][v & 3];
  // element offset of output pixel p of the strip (cell of 16-channel block 0; nhwc: channel vector): linear in p
  const size_t px_stride = a.out_nhwc ? (size_t)oc_real : (size_t)16;
  const size_t out0 = a.out_nhwc ? ((size_t)img * ohw + (size_t)oh0 * a.ow) * oc_real
                                 : ((size_t)img * a.oc2 * ohw + (size_t)oh0 * a.ow) * 16;
  const size_t block_stride = a.out_nhwc ? (size_t)16 : (size_t)ohw * 16;
  const int row_step = a.stride_h * a.lrow, px_step = a.stride_w * a.icl;
  const int ntiles = (npix + 31) >> 5;
  for (int tile = wp; tile < ntiles; tile += wpn) {
    int p = tile * 32 + l32;
    p = p < npix ? p : npix - 1;
    const int ro = fastdiv(p, a.ow, a.ow_magic);
    const int ox = p - ro * a.ow;
    const int at0 = ro * row_step + ox * px_step;
    v4i b[KS];
    if (a.icl == 4) {   // every cell starts on a dword: four reads, nothing to shift
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const unsigned *src = rows_lds + ((at0 + cell_at[ks]) >> 2);
        b[ks] = v4i{(int)src[0], (int)src[1], (int)src[2], (int)src[3]};
      }
    } else {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const int A = at0 + cell_at[ks];
        const unsigned *src = rows_lds + (A >> 2);
        const unsigned sh = A & 3;
        const unsigned d0 = src[0], d1 = src[1], d2 = src[2], d3 = src[3], d4 = src[4];
        b[ks] = v4i{(int)__builtin_amdgcn_alignbyte(d1, d0, sh), (int)__builtin_amdgcn_alignbyte(d2, d1, sh),
                    (int)__builtin_amdgcn_alignbyte(d3, d2, sh), (int)__builtin_amdgcn_alignbyte(d4, d3, sh)};
      }
    }
    v16i acc[1][1];
    acc[0][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wreg[0], b[0], comp0, 0, 0, 0);
#pragma unroll
    for (int ks = 1; ks < KS; ++ks) acc[0][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wreg[ks], b[ks], acc[0][0], 0, 0, 0);
    size_t pix[1], pixT[1][2];
    bool pvalid[1], validT[1][2];
    int cls[1] = {0};
    const int p0 = tile * 32;
    pvalid[0] = p0 + l32 < npix;
    pix[0] = out0 + (size_t)(p0 + l32) * px_stride;
    validT[0][0] = p0 + (lane >> 2) < npix;
    validT[0][1] = p0 + (lane >> 2) + 16 < npix;
    pixT[0][0] = out0 + (size_t)(p0 + (lane >> 2)) * px_stride;
    pixT[0][1] = pixT[0][0] + 16 * px_stride;
    if (a.lean) {
      // Lean epilogue (u8 / s8 output, ReLU: 3-4 instructions per value instead of ~10 -- with 16-112
      // multiply-adds per output value the epilogue is most of a tile's instructions).  The scale is the
      // lane's channels'; the shift row is the one of the pixel's border class where the layer has classes.
      LeanConsts lk[1];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        lk[0].sc[q] = k0.sc[q];
        lk[0].sh[q] = k0.sh[q];
      }
      if (a.tab_lds) {
        const float *row = lds_shift + (lds_cls_h[ro] + lds_cls_w[ox]) * (a.wo * 32) + wo * 32 + 16 * lh;
#pragma unroll
        for (int q = 0; q < 4; ++q) lk[0].sh[q] = *reinterpret_cast<const float4 *>(row + 4 * q);
      } else if (a.ep.shift_tab) {
        const float *row = a.ep.shift_tab + (size_t)(a.cls_h[oh0 + ro] * a.ncls_w + a.cls_w[ox]) * a.ep.tab_stride + cidx;
#pragma unroll
        for (int q = 0; q < 4; ++q) lk[0].sh[q] = *reinterpret_cast<const float4 *>(row + 4 * q);
      }
      uint8_t *cell[1] = {static_cast<uint8_t *>(a.out) + pix[0] +
                          (a.out_nhwc ? (size_t)(oc0 + 16 * lh) : (size_t)((oc0 >> 4) + lh) * block_stride)};
            // blocked output: non-temporal stores (M1 15.9 -> 14.3 us); in nhwc a line's 16-byte pieces come from
      // several waves and should meet in L2 (R1 32.9 -> 37.6 us with them)
      if (a.out_nhwc) lean_store<1, 1>(a.lean, a.ep, acc, lk, cell, pvalid, oc0 + 16 * lh, oc_real, 0);
      else lean_store<1, 1, true>(a.lean, a.ep, acc, lk, cell, pvalid, oc0 + 16 * lh, oc_real, 0);
      continue;
    }
    if (a.tab_lds) {
      cls[0] = lds_cls_h[ro] + lds_cls_w[ox];
      epilogue_wave<1, 1, true, true>(ep_lds, acc, k0, wo * 32 + 16 * lh, oc0 + 16 * lh, pix, pvalid, oc_real,
                                      block_stride, a.out, xlds, pixT, validT, cls);
    } else {
      if (a.ep.shift_tab) cls[0] = a.cls_h[oh0 + ro] * a.ncls_w + a.cls_w[ox];
      epilogue_wave<1, 1, true, true>(a.ep, acc, k0, cidx, oc0 + 16 * lh, pix, pvalid, oc_real, block_stride, a.out,
                                      xlds, pixT, validT, cls);
    }
  }
}

// The same tiles for u8 / s8 output with ReLU (FewChArgs::lean; TAB: the shift row of the pixel's border class
// comes from LDS): nothing but that epilogue, so the tile loop is straight-line code with 32-bit output offsets,
// and the cells of a wave's next tile are read while the present one is scaled and stored.
template <int KS, bool CLAMP, bool TAB>
__global__ __launch_bounds__(kBlock, 3) void k_conv_fewch_lean(FewChArgs a)
{
  extern __shared__ unsigned rows_lds[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31;
  const int lh = lane >> 5;
  const int img = blockIdx.x / a.strips, strip = blockIdx.x - img * a.strips;
  const int oh0 = strip * a.rows;
  const int rows_valid = a.oh - oh0 < a.rows ? a.oh - oh0 : a.rows;
  const int npix = rows_valid * a.ow;
  const int ihb = oh0 * a.stride_h - a.pad_t;
  const FewChTables tabs = fewch_stage(a, rows_lds, tid, img, ihb, oh0, rows_valid);
  __syncthreads();

  const int wo = wave % a.wo, wp = wave / a.wo, wpn = 4 / a.wo;
  const int oc0 = (blockIdx.y * a.wo + wo) * 32;
  const int oc_real = a.oc2 * 16;
  const int ohw = a.oh * a.ow;
  v4i wreg[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks)
    wreg[ks] = *reinterpret_cast<const v4i *>(a.w + ((long long)(2 * ks + lh) * a.ocpp + oc0 + l32) * 16);
  int cell_at[KS];   // as in k_conv_fewch_u8s8
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    int tc = 2 * ks + lh;
    tc = tc < a.cells ? tc : a.cells - 1;
    const int kr = tc / a.nu;
    cell_at[ks] = kr * a.lrow + (tc - kr * a.nu) * a.ppc * a.icl;
  }
  const long long cidx = oc0 + 16 * lh;
  LeanConsts lk[1];
  load_lean_consts(lk[0], a.ep, cidx);
  v16i comp0;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const v4i c = *reinterpret_cast<const v4i *>(a.ep.comp + cidx + 4 * q);
#pragma unroll
    for (int j = 0; j < 4; ++j) comp0[4 * q + j] = c[j];
  }
  // output: a uniform base (the strip's first pixel) and a byte offset per lane that fits 32 bits (the launcher checks)
  const unsigned px_stride = a.out_nhwc ? (unsigned)oc_real : 16u;
  uint8_t *const out_base = static_cast<uint8_t *>(a.out) +
      (a.out_nhwc ? ((size_t)img * ohw + (size_t)oh0 * a.ow) * oc_real : ((size_t)img * a.oc2 * ohw + (size_t)oh0 * a.ow) * 16);
  const unsigned lane_off = (a.out_nhwc ? (unsigned)(oc0 + 16 * lh) : (unsigned)((oc0 >> 4) + lh) * (unsigned)ohw * 16u) +
      (unsigned)l32 * px_stride;
  const float *const shift_rows = TAB ? tabs.shift + wo * 32 + 16 * lh : nullptr;
  const int tab_width = a.wo * 32;
  const int row_step = a.stride_h * a.lrow, px_step = a.stride_w * a.icl;
  const int ntiles = (npix + 31) >> 5;

  int ro, ox;   // output row (in the strip) and column of the lane's pixel of the tile whose cells were read last
  v4i b[KS];
  auto read_cells = [&](int tile) {
    int p = tile * 32 + l32;
    p = p < npix ? p : npix - 1;   // also beyond the wave's last tile: some cell of the strip
    ro = fastdiv(p, a.ow, a.ow_magic);
    ox = p - ro * a.ow;
    const int at0 = ro * row_step + ox * px_step;
    if (a.icl == 4) {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const unsigned *src = rows_lds + ((at0 + cell_at[ks]) >> 2);
        b[ks] = v4i{(int)src[0], (int)src[1], (int)src[2], (int)src[3]};
      }
    } else {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const int A = at0 + cell_at[ks];
        const unsigned *src = rows_lds + (A >> 2);
        const unsigned sh = A & 3;
        const unsigned d0 = src[0], d1 = src[1], d2 = src[2], d3 = src[3], d4 = src[4];
        b[ks] = v4i{(int)__builtin_amdgcn_alignbyte(d1, d0, sh), (int)__builtin_amdgcn_alignbyte(d2, d1, sh),
                    (int)__builtin_amdgcn_alignbyte(d3, d2, sh), (int)__builtin_amdgcn_alignbyte(d4, d3, sh)};
      }
    }
  };
  read_cells(wp);
  for (int tile = wp; tile < ntiles; tile += wpn) {
    v16i acc[1][1];
    acc[0][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wreg[0], b[0], comp0, 0, 0, 0);
#pragma unroll
    for (int ks = 1; ks < KS; ++ks) acc[0][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wreg[ks], b[ks], acc[0][0], 0, 0, 0);
    if (TAB) {
      const float *row = shift_rows + (tabs.cls_h[ro] + tabs.cls_w[ox]) * tab_width;
#pragma unroll
      for (int q = 0; q < 4; ++q) lk[0].sh[q] = *reinterpret_cast<const float4 *>(row + 4 * q);
    }
    __builtin_amdgcn_sched_barrier(0);
    read_cells(tile + wpn);   // the MFMAs above have taken their operands
    __builtin_amdgcn_sched_barrier(0);
    const int p0 = tile * 32;
    const bool pvalid[1] = {p0 + l32 < npix};
    uint8_t *const cell[1] = {out_base + ((unsigned)p0 * px_stride + lane_off)};
    // blocked output: non-temporal stores (3x3 s2 3 -> 32 at 224 x 224, N = 64: 15.9 -> 14.3 us); in nhwc a line's
    // 16-byte pieces come from several waves and should meet in L2 (7x7 s2 3 -> 64: 32.9 -> 37.6 us with them)
    if (a.out_nhwc) lean_store_typed<1, 1, false, CLAMP, false>(a.ep, acc, lk, cell, pvalid, oc0 + 16 * lh, oc_real, 0, nullptr);
    else lean_store_typed<1, 1, false, CLAMP, true>(a.ep, acc, lk, cell, pvalid, oc0 + 16 * lh, oc_real, 0, nullptr);
  }
}

int conv_fewch_icl(int ic, int kw)
{
  if (ic != 3 || (kw + 3) / 4 != (kw + 4) / 5) return ic;
  // A cell is four dword reads instead of five and four byte shifts, and nhwc input is staged four pixels per
  // thread: 7x7, stride 2 at 224 x 224, N = 64: 31.9 -> 26.4 us; 3x3, stride 2: 13.9 -> 12.6 us.
  const char *env = getenv("EHIP_FEWCH_PAD_PIXEL");
  return env && env[0] == '0' ? 3 : 4;
}

bool conv_fewch_applies(int ic, int kh, int kw)
{
  if (ic < 1 || ic > 4 || kh * kw <= 1 || kw < 2) return false;
  const int ppc = 16 / ic, nu = (kw + ppc - 1) / ppc;   // the same nu with padded pixels
  return kh * nu <= 14;
}

// pitch in bytes of a staged input row: pad_l + iw pixels or the last output pixel's last cell
// (16 bytes), whichever ends later, + 4 for the fifth dword of a shifted cell
int conv_fewch_row_pitch(int icl, int kw, int iw, int ow, int stride_w, int pad_l)
{
  const int ppc = 16 / icl, nu = (kw + ppc - 1) / ppc;
  int need = (pad_l + iw) * icl;
  const int last = ((ow - 1) * stride_w + (nu - 1) * ppc) * icl + 16;
  if (last > need) need = last;
  // four-byte pixels: whole 16-byte groups (the staging writes four pixels at a time); else the cell reads' fifth dword
  return icl == 4 ? up(need + 4, 16) : up(need + 4, 4) + 4;
}

// Fills the derived fields (cells, strip height, LDS row pitch, wave split) and launches.
// Expects in a: tensors, epilogue, n, ih, iw, oh, ow, ic, kh, kw, strides, pads, oc2, ocpp, formats, classes.
hipError_t launch_conv_fewch(FewChArgs &a, hipStream_t s, LaunchPlan<FewChArgs> *plan)
{
  if (plan && plan->valid) {   // everything but the tensors is as on the first launch
    if (a.in_nhwc && (reinterpret_cast<uintptr_t>(a.in) & 3)) return hipErrorInvalidValue;   // aligned dword loads
    return plan_relaunch(*plan, [&](FewChArgs &x) { x.in = a.in; x.out = a.out; }, s);
  }
  {
    // lean_mode() but for the per-pixel shift rows, which this kernel's lean path reads itself
    Epilogue e = a.ep;
    e.shift_tab = nullptr;
    a.lean = lean_mode(e, false);
    if (a.ep.with_sum) a.lean = 0;
  }
  if (a.icl != a.ic && !(a.ic == 3 && a.icl == 4)) return hipErrorInvalidValue;
  a.ppc = 16 / a.icl;
  a.nu = (a.kw + a.ppc - 1) / a.ppc;
  a.cells = a.kh * a.nu;
  if (!conv_fewch_applies(a.ic, a.kh, a.kw)) return hipErrorInvalidValue;
  if (a.in_nhwc && (reinterpret_cast<uintptr_t>(a.in) & 3)) return hipErrorInvalidValue;   // aligned dword loads
  a.lrow = conv_fewch_row_pitch(a.icl, a.kw, a.iw, a.ow, a.stride_w, a.pad_l);
  const int octiles = up(a.oc2 * 16, 32) / 32;   // <= ocpp / 32
  a.wo = octiles % 4 == 0 ? 4 : octiles % 2 == 0 ? 2 : 1;
  const int gy = octiles / a.wo, wpn = 4 / a.wo;
  // Strip height (output rows per workgroup).  A taller strip stages fewer overlap rows per output
  // row; what it must not do is leave waves without tiles, end in a nearly empty strip, or put a
  // few workgroups more into the grid than the chip runs at once (they would run alone in a second
  // round).  All of that goes into one relative cost, minimised over the heights whose rows fit in LDS.
  int rows = 1;
  const char *env = getenv("EHIP_FEWCH_ROWS");
  if (env && env[0]) {
    rows = atoi(env);
  } else {
    static int n_cu = 0;
    if (!n_cu) {
      int dev = 0, v = 0;
      if (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0)
        n_cu = v;
      else
        n_cu = 256;
    }
    double best = 0.0;
    for (int r = 1; r <= a.oh && r <= 32; ++r) {
      const int nrows_in = (r - 1) * a.stride_h + a.kh;
      const size_t dyn = (size_t)nrows_in * a.lrow + 32;
      if (dyn > 40 * 1024) break;
      // workgroups of 4 waves resident per CU: registers (3 waves per SIMD; 4 for the lean kernel with at most
      // five operands, which stays below 128 registers), LDS (the general kernel's 16 KB static exchange patch +
      // the rows).  3x3 s2 3 -> 32 at 224 x 224, N = 64: strips of 7 rows (4 workgroups per CU) 12.0 us, of 10 rows
      // (3 per CU) 12.6 us.
      int resident = (a.lean && (a.cells + 1) / 2 <= 5) ? 4 : 3;
      const int by_lds = (int)((160 * 1024) / ((a.lean ? 0 : 16 * 1024) + dyn));
      if (by_lds < resident) resident = by_lds < 1 ? 1 : by_lds;
      const double slots = (double)n_cu * resident;
      const double wgs = (double)a.n * ((a.oh + r - 1) / r) * gy;
      const double rounds = (double)(long long)((wgs + slots - 1) / slots);
      const int tiles = (r * a.ow + 31) / 32;
      const double cost = rounds * slots / wgs                                   // idle slots of the last round
          * ((tiles + wpn - 1) / wpn * wpn * 32.0 / (r * a.ow))                  // idle waves and lanes of the last tiles
          * ((double)((a.oh + r - 1) / r) * r / a.oh)                             // rows of the last strip below the image
          * (1.0 + 0.2 * nrows_in / (r * a.stride_h));                            // staging, relative to the tile work
      if (best == 0.0 || cost < best) { best = cost; rows = r; }
    }
  }
  if (rows < 1) rows = 1;
  if (rows > a.oh) rows = a.oh;
  a.rows = rows;
  a.strips = (a.oh + rows - 1) / rows;
  a.nrows_in = (rows - 1) * a.stride_h + a.kh;
  size_t lds = (size_t)a.nrows_in * a.lrow + 32;
  a.tab_lds = 0;
  if (a.ep.shift_tab) {
    const size_t tab = (size_t)(rows + a.ow + a.nclass * a.wo * 32) * 4;
    if (lds + tab <= 48 * 1024) {
      a.tab_lds = (int)(up((int)lds, 16) / 4);   // dword offset of the tables
      lds = (size_t)a.tab_lds * 4 + tab;
    }
  }
  if (lds > 48 * 1024 + 64 || (long long)a.nrows_in * a.lrow >= (1ll << 30) ||
      (long long)(a.ih + 2 * a.kh + 32) * (a.iw + 16) * a.ic >= (1ll << 30) || (long long)rows * a.ow * a.ow >= (1ll << 32))
    return hipErrorInvalidValue;
  a.ow_magic = div_magic(a.ow);
  a.iw_magic = div_magic(a.iw);
  a.lrow4_magic = div_magic(a.lrow / 4);
  a.lrow16_magic = div_magic(a.lrow / 16 > 0 ? a.lrow / 16 : 1);
  if ((long long)a.nrows_in * (a.lrow / 4) * (a.lrow / 4) >= (1ll << 32) || (long long)a.nrows_in * a.iw * a.iw >= (1ll << 32))
    return hipErrorInvalidValue;
  const int ks = (a.cells + 1) / 2;
  void (*kern)(FewChArgs) = ks <= 2 ? k_conv_fewch_u8s8<2> : ks == 3 ? k_conv_fewch_u8s8<3> : ks == 4 ? k_conv_fewch_u8s8<4>
      : ks == 5 ? k_conv_fewch_u8s8<5> : k_conv_fewch_u8s8<7>;
  const char *name = "k_conv_fewch_u8s8";
  // the kernel of the lean epilogue alone: shift rows per channel or on chip, an image's output below 2 GB
  const char *env_lean = getenv("EHIP_FEWCH_LEAN_KERNEL");
  if (a.lean && !(env_lean && env_lean[0] == '0') && (!a.ep.shift_tab || a.tab_lds) &&
      (long long)a.oc2 * 16 * a.oh * a.ow < (1ll << 31)) {
    const bool clamp = !(a.lean & 2), tab = a.tab_lds != 0;
#define FL(K) (clamp ? (tab ? k_conv_fewch_lean<K, true, true> : k_conv_fewch_lean<K, true, false>) \
                     : (tab ? k_conv_fewch_lean<K, false, true> : k_conv_fewch_lean<K, false, false>))
    kern = ks <= 2 ? FL(2) : ks == 3 ? FL(3) : ks == 4 ? FL(4) : ks == 5 ? FL(5) : FL(7);
#undef FL
    name = "k_conv_fewch_lean";
  }
  const hipError_t e = plan_launch(plan, kern, dim3(a.n * a.strips, gy), dim3(kBlock), lds, a, s);
  if (plan) plan->name = name;
  return e;
}

}  // namespace ehip
