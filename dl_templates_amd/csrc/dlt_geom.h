// Window geometry shared by host code, the debug exports and every attention kernel.
//
// Tokens live on a 2D grid of `TR` rows; a row holds `XL` tokens (x = c * S + s for tile
// column c and in-tile slot s), token n = r * XL + x, which is the reference's tile-major
// numbering n = (r * t_width + c) * b_size + s (src/tiled_swa.py:63,104,216).
// Dense attention is the same structure with one row and an unrestricted x interval.
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define DLT_HD __host__ __device__ inline
#else
#define DLT_HD inline
#endif

enum { DLT_GEOM_SWA = 0, DLT_GEOM_DENSE = 1, DLT_GEOM_CAUSAL = 2 };

struct DltGeom {
  int32_t mode;
  int32_t TR;        // grid rows (1 for dense / causal)
  int32_t XLq, XLk;  // tokens per row on the query side / key side
  int32_t S, TC;     // tokens per tile, tiles per row (SWA only)
  int32_t WR, WC;    // window half sizes in tiles (SWA only)
};

DLT_HD int dlt_imin(int a, int b) { return a < b ? a : b; }
DLT_HD int dlt_imax(int a, int b) { return a > b ? a : b; }

// Keys attended by query (r, x): rows [rlo, rhi] (inclusive), x in [xlo, xhi).
// SWA: |r - r'| <= WR and |c - c'| <= WC, truncated at the border
// (src/tiled_swa.py:76-79, :212-214, :701-713).
DLT_HD void dlt_key_range(const DltGeom& g, int r, int x, int& rlo, int& rhi, int& xlo, int& xhi) {
  if (g.mode == DLT_GEOM_SWA) {
    const int c = x / g.S;
    rlo = dlt_imax(r - g.WR, 0);
    rhi = dlt_imin(r + g.WR, g.TR - 1);
    xlo = dlt_imax(c - g.WC, 0) * g.S;
    xhi = dlt_imin(c + g.WC + 1, g.TC) * g.S;
  } else if (g.mode == DLT_GEOM_DENSE) {
    rlo = rhi = 0; xlo = 0; xhi = g.XLk;
  } else {
    rlo = rhi = 0; xlo = 0; xhi = dlt_imin(x + 1, g.XLk);
  }
}

// Queries that attend key (r, x): the transpose of dlt_key_range.  The SWA window is
// symmetric (the reference's backward relies on the same fact, src/tiled_swa.py:475-488).
DLT_HD void dlt_query_range(const DltGeom& g, int r, int x, int& rlo, int& rhi, int& xlo, int& xhi) {
  if (g.mode == DLT_GEOM_SWA) {
    dlt_key_range(g, r, x, rlo, rhi, xlo, xhi);
  } else if (g.mode == DLT_GEOM_DENSE) {
    rlo = rhi = 0; xlo = 0; xhi = g.XLq;
  } else {
    rlo = rhi = 0; xlo = dlt_imin(x, g.XLq); xhi = g.XLq;
  }
}

// idx decode of the rotary op: row = int16(idx >> 16), col = int16(idx & 0xFFFF)
// (src/fused_rope2d.py:41-42); an axis is rotated iff its value is >= 0 (:44-45).
DLT_HD int dlt_rope_row(int32_t idx) { return (int)(int16_t)(idx >> 16); }
DLT_HD int dlt_rope_col(int32_t idx) { return (int)(int16_t)(idx & 0xFFFF); }

// ---- image layout of the tokens --------------------------------------------------------------
// A caller that keeps q, k, v as images [B, IH, IW, heads, D] (the layout the reference's demo
// converts from and to around the operator, src/tiled_swa.py:753-755) maps pixel (y, x) of a tile
// of bh x bw pixels to token
//     n = ((y / bh * TC + x / bw) * bh + y % bh) * bw + x % bw,      S = bh * bw tokens per tile.
// The kernels go the other way: token n -> pixel (y, x) -> element offset y * stride_y + x * stride_x.
// Divisions by S, TC and bw are exact multiply-shift divisions (m = ceil(2^(31+l) / d), l = ceil(log2 d):
// floor(n m / 2^(31+l)) = floor(n / d) for every n < 2^31).
struct DltTokMap {
  int32_t img;  // 0: token n lies n * stride_n elements into its (batch, head) slab
  uint32_t S, TC, bh, bw;
  uint32_t mS, mTC, mbw;  // multipliers
  uint32_t sS, sTC, sbw;  // shifts (31 + l)
};

DLT_HD uint32_t dlt_fastdiv(uint32_t n, uint32_t m, uint32_t sh) { return (uint32_t)(((uint64_t)n * m) >> sh); }

DLT_HD void dlt_fastdiv_make(uint32_t d, uint32_t& m, uint32_t& sh) {
  uint32_t l = 0;
  while (l < 31 && ((uint32_t)1 << l) < d) l++;
  const uint64_t num = (uint64_t)1 << (31 + l);
  m = (uint32_t)((num + d - 1) / d);
  sh = 31 + l;
}

DLT_HD DltTokMap dlt_tokmap_none() {
  DltTokMap tm;
  tm.img = 0; tm.S = tm.TC = tm.bh = tm.bw = 1;
  tm.mS = tm.mTC = tm.mbw = (uint32_t)1 << 31;
  tm.sS = tm.sTC = tm.sbw = 31;
  return tm;
}

DLT_HD DltTokMap dlt_tokmap_image(uint32_t bh, uint32_t bw, uint32_t TC) {
  DltTokMap tm;
  tm.img = 1; tm.S = bh * bw; tm.TC = TC; tm.bh = bh; tm.bw = bw;
  dlt_fastdiv_make(tm.S, tm.mS, tm.sS);
  dlt_fastdiv_make(TC, tm.mTC, tm.sTC);
  dlt_fastdiv_make(bw, tm.mbw, tm.sbw);
  return tm;
}

// token n (tile-major order) -> pixel (y, x)
DLT_HD void dlt_token_pixel(const DltTokMap& tm, uint32_t n, uint32_t& y, uint32_t& x) {
  const uint32_t tile = dlt_fastdiv(n, tm.mS, tm.sS), s = n - tile * tm.S;
  const uint32_t tr = dlt_fastdiv(tile, tm.mTC, tm.sTC), tc = tile - tr * tm.TC;
  const uint32_t i = dlt_fastdiv(s, tm.mbw, tm.sbw), j = s - i * tm.bw;
  y = tr * tm.bh + i;
  x = tc * tm.bw + j;
}

// slot x' = tc * S + s inside a grid row (tile column tc, in-tile slot s) -> (pixel row inside the
// tile row, pixel x): what the kernels that walk a grid row at a time need
DLT_HD void dlt_slot_pixel(const DltTokMap& tm, uint32_t xs, uint32_t& i, uint32_t& x) {
  const uint32_t tc = dlt_fastdiv(xs, tm.mS, tm.sS), s = xs - tc * tm.S;
  i = dlt_fastdiv(s, tm.mbw, tm.sbw);
  x = tc * tm.bw + (s - i * tm.bw);
}
