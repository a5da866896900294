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
