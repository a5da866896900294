// Test shim: exposes the host/device geometry header of the product (window ranges, token -> pixel map,
// exact multiply-shift division) to the CPU tests through a C interface.  Built by tests/test_geom_cpu.py
// with the host compiler; not part of the library.
#include "../dl_templates_amd/csrc/dlt_geom.h"

extern "C" {
void shim_key_range(int mode, int TR, int TC, int S, int WR, int WC, int XLq, int XLk, int r, int x, int* out) {
  DltGeom g;
  g.mode = mode; g.TR = TR; g.TC = TC; g.S = S; g.WR = WR; g.WC = WC; g.XLq = XLq; g.XLk = XLk;
  dlt_key_range(g, r, x, out[0], out[1], out[2], out[3]);
  dlt_query_range(g, r, x, out[4], out[5], out[6], out[7]);
}
unsigned shim_fastdiv(unsigned n, unsigned d) {
  unsigned m, sh;
  dlt_fastdiv_make(d, m, sh);
  return dlt_fastdiv(n, m, sh);
}
void shim_token_pixel(unsigned bh, unsigned bw, unsigned TC, unsigned n, unsigned* y, unsigned* x) {
  const DltTokMap tm = dlt_tokmap_image(bh, bw, TC);
  dlt_token_pixel(tm, n, *y, *x);
}
void shim_slot_pixel(unsigned bh, unsigned bw, unsigned TC, unsigned xs, unsigned* i, unsigned* x) {
  const DltTokMap tm = dlt_tokmap_image(bh, bw, TC);
  dlt_slot_pixel(tm, xs, *i, *x);
}
int shim_rope_row(int idx) { return dlt_rope_row(idx); }
int shim_rope_col(int idx) { return dlt_rope_col(idx); }
}
