// Host model of the streaming token-grid kernels' address maps (dl_templates_amd/csrc/swa2_index.h, the header the
// kernels themselves compute every offset with).  For one problem and one kernel class (head dim D, NCG column groups)
// it replays, for every workgroup, chunk, wave, lane and instruction:
//   * the asynchronous copies (global byte offset, LDS destination) of both streamed tensors and of the per-token
//     scalars of the dK/dV kernel, into a model of LDS that remembers which (tensor, grid row, grid column, piece)
//     every 16-byte slot (4-byte slot for scalars) holds;
//   * the operand reads (A operand, transposing read, scalar reads) against that model;
//   * the store epilogue's tile writes and reads;
//   * the window geometry against dlt_key_range: over all column passes every key of a window is visible exactly once.
// and reports the first violated condition.  Built by tests/test_swa2_index_cpu.py with the host compiler; not part of
// the library.
#include <cstdio>
#include <cstring>
#include <vector>

#include "../dl_templates_amd/csrc/swa2_index.h"

namespace {
char g_msg[512];
int fail(const char* fmt, int a = 0, int b = 0, int c = 0, int d = 0, int e = 0, int f = 0) {
  snprintf(g_msg, sizeof g_msg, fmt, a, b, c, d, e, f);
  return 1;
}

struct Slot { int tensor, r, c, piece; };   // tensor -1: never written

template <typename C>
int model(int TR, int TCt, int WR, int WCt, int S, int npass, int band, int sn2, int ls2, long long slab_bytes, long long scal_elems, int lds_bytes, int lds_kv_bytes) {
  if (lds_bytes != C::LDS) return fail("launcher asks for %d bytes of LDS, the class needs %d", lds_bytes, C::LDS);
  if (lds_kv_bytes != C::LDS_KV) return fail("launcher asks for %d bytes of LDS (dK/dV), the class needs %d", lds_kv_bytes, C::LDS_KV);
  // token slots per grid row and the largest column extent of a window in slots (tiles of S tokens)
  const int TC = TCt * S, WC = S * WCt + S - 1;
  const int ncg_total = (4 + 2 * WC + 3) >> 2;
  if (ncg_total > C::NCG * npass) return fail("window of %d column groups on a class with %d in %d column passes", ncg_total, C::NCG, npass);
  Swa2Plan P;
  if (band != 8 && band != 16) return fail("bands of %d rows", band);
  P.band = band;   // 16: two stacked patches per wave (row groups 0 .. 3)
  P.nblk_r = (TR + band - 1) / band;
  P.nblk_c = (TC + 15) / 16;
  const int H = 1;
  P.npass = npass; P.S = S; P.WCt = WCt;
  dlt_fastdiv_make((uint32_t)S, P.m_S, P.s_S);
  dlt_fastdiv_make((uint32_t)(P.nblk_r * P.nblk_c), P.m_bh, P.s_bh);
  dlt_fastdiv_make((uint32_t)P.nblk_c, P.m_c, P.s_c);
  dlt_fastdiv_make((uint32_t)H, P.m_h, P.s_h);
  DltGeom dg;
  dg.mode = DLT_GEOM_SWA; dg.TR = TR; dg.XLq = dg.XLk = TC; dg.S = S; dg.TC = TCt; dg.WR = WR; dg.WC = WCt;
  std::vector<Slot> lds(C::LDS_KV / 4);
  const int nwg = P.nblk_r * P.nblk_c;
  for (int lin = 0; lin < nwg; lin++) {
    const Swa2Geom G0 = swa2_geom_at(TR, TC, WR, WC, H, P, lin);
    const Swa2Geom& G = G0;
    if (G.b != 0 || G.h != 0) return fail("workgroup %d decoded to batch %d head %d", lin, G.b, G.h);
    if (G.r0 >= TR || G.c0 >= TC) return fail("workgroup %d starts outside the grid (%d, %d)", lin, G.r0, G.c0);
    if (G.ch_first > G.ch_last) return fail("workgroup %d: empty chunk range", lin);
    // ---- windows against the shared geometry routine
    for (int patch = 0; patch < band / 4 * 4; patch++) {
      const int pc = patch & 3, rg = patch >> 2;
      for (int n = 0; n < 16; n++) {
        const Swa2Win W0 = swa2_window(G, rg, pc, n);
        const int r = G.r0 + 4 * rg + (n >> 2), c = G.c0 + 4 * pc + (n & 3);
        const bool own = r < TR && c < TC;
        int rlo = 0, rhi = -1, xlo = 0, xhi = 0;
        if (own) dlt_key_range(dg, r, c, rlo, rhi, xlo, xhi);
        int hits = 0;
        for (int pass = 0; pass < npass; pass++) {
          const Swa2Geom Gp = swa2_pass_geom(G0, C::NCG, pass);
          const Swa2Win W = swa2_pass_window(W0, C::NCG, pass);
          const int ncg = swa2_pass_ncg(WC, C::NCG, pass);
          for (int ch = 0; ch <= (band - 1 + 2 * WR) >> 2; ch++)
            for (int hr = 0; hr < 4; hr++) {
              const int hrow = 4 * ch + hr, kr = G.r0 - WR + hrow;
              const bool row_vis = hrow >= W.rlo && hrow <= W.rhi;
              for (int cg = 0; cg < C::NCG; cg++)
                for (int i = 0; i < 4; i++) {
                  const int kc = G.c0 - Gp.WC + 4 * (pc + cg) + i;
                  if (!own) continue;   // own positions outside the grid compute values that are never stored
                  const bool want = kr >= rlo && kr <= rhi && kc >= xlo && kc < xhi;
                  const bool got = swa2_visible(W, row_vis, cg, i, ncg);
                  if (want != got && (got || cg < ncg)) return fail("visibility of key (%d, %d) from own token (%d, %d): kernel %d, geometry %d", kr, kc, r, c, got, want);
                  hits += got;
                  if (got && (ch < G.ch_first || ch > G.ch_last || ch < W.ch_lo || ch > W.ch_hi))
                    return fail("visible key row %d (chunk %d) outside the chunk range the wave consumes [%d, %d]", kr, ch, W.ch_lo, W.ch_hi);
                }
            }
        }
        // every key of the window is seen in exactly one (pass, column group) and lies inside the band's chunks
        if (own) {
          if (hits != (rhi - rlo + 1) * (xhi - xlo)) return fail("own token (%d, %d): %d keys visible over all passes, the window holds %d", r, c, hits, (rhi - rlo + 1) * (xhi - xlo));
          if (xlo < G.c0 - WC + 4 * pc || xhi > G.c0 - WC + 4 * (pc + C::NCG * npass)) return fail("window columns [%d, %d) exceed the wave window of own token (%d, %d)", xlo, xhi, r, c);
          if (rlo < G.r0 - WR + 4 * G.ch_first || rhi > G.r0 - WR + 4 * G.ch_last + 3) return fail("window rows [%d, %d] exceed the band's chunks", rlo, rhi);
        }
      }
    }
    // ---- chunks: copies into the buffer (ch & 1), then the reads of every wave
    for (int pass = 0; pass < npass; pass++)
    for (int kv = 0; kv < 2; kv++) {   // 0: forward / dQ layout (BUF), 1: dK/dV layout (BUF_KV, with scalars)
      const Swa2Geom G = swa2_pass_geom(G0, C::NCG, pass);   // what the kernels address columns with in this pass
      const int WC = G.WC;
      const int bufsz = kv ? C::BUF_KV : C::BUF, total = kv ? C::LDS_KV : C::LDS;
      for (int ch = G.ch_first; ch <= G.ch_last; ch++) {
        for (Slot& s : lds) s.tensor = -1;
        const int buf = (ch & 1) * bufsz;
        for (int wave = 0; wave < 8; wave++) {
          const int r = swa2_issue_grid_row(G, ch, wave);
          if (r < 0 || r >= TR) return fail("copy row %d outside the grid", r);
          const int dst = buf + swa2_issue_dst_off<C>(wave);
          for (int i = 0; i < C::NI; i++)
            for (int lane = 0; lane < 64; lane++) {
              if (!swa2_stage_on<C>(lane, i)) continue;
              const long long goff = (long long)r * TC * sn2 + swa2_stage_off<C>(G, wave, lane, sn2, i);
              if (goff < 0 || goff + 16 > slab_bytes) return fail("copy reads global bytes at %d of a slab of %d (wave %d, lane %d, instruction %d)", (int)goff, (int)slab_bytes, wave, lane, i);
              const int tok = (int)((goff - (long long)r * TC * sn2) / sn2), within = (int)((goff - (long long)r * TC * sn2) % sn2);
              if (within % 16 != 0 || within + 16 > C::ROW) return fail("copy reads bytes %d..+15 of a token row of %d bytes", within, C::ROW);
              const int a = dst + 1024 * i + 16 * lane;
              if (a < buf || a + 16 > buf + C::BUF) return fail("copy writes LDS bytes at %d outside the rows of its chunk buffer [%d, %d)", a, buf, buf + C::BUF);
              if (a + 16 > total) return fail("copy writes LDS bytes at %d beyond the %d the launcher asks for", a, total);
              for (int w4 = 0; w4 < 4; w4++) {
                Slot& s = lds[a / 4 + w4];
                if (s.tensor != -1) return fail("LDS bytes at %d written twice in one chunk", a);
                s = Slot{wave >> 2, r, tok, 4 * (within / 16) + w4};
              }
            }
          if (kv) {
            const int sdst = buf + swa2_scal_dst_off<C>(wave);
            for (int lane = 0; lane < C::HCW; lane++) {
              const long long e = ((long long)r * TC + swa2_scal_col(G, lane)) * ls2;
              if (e < 0 || e >= scal_elems) return fail("scalar copy reads element %d of %d", (int)e, (int)scal_elems);
              const int a = sdst + 4 * lane;
              if (a < buf + C::BUF || a + 4 > buf + C::BUF_KV) return fail("scalar copy writes LDS bytes at %d outside the table of its chunk buffer", a);
              Slot& s = lds[a / 4];
              if (s.tensor != -1) return fail("scalar slot at %d written twice", a);
              s = Slot{2 + (wave >> 2), r, swa2_scal_col(G, lane), 0};
            }
          }
        }
        // reads
        for (int wave = 0; wave < 8; wave++) {
          const int pc = wave & 3;
          for (int lane = 0; lane < 64; lane++) {
            const int n = lane & 15, g = lane >> 4;
            Swa2Lane<C> L;
            swa2_lane_init(L, pc, n, g);
            for (int tensor = 0; tensor < 2; tensor++) {
              const int region = buf + tensor * C::REGION;
              // A operand, every column group and k-piece
              int err = 0;
              auto check_a = [&](auto cgc) {
                constexpr int CG = decltype(cgc)::value;
                for (int c = 0; c < C::KC && !err; c++) {
                  const int a = region + swa2_read_a_off<C, CG>(L, c);
                  if (a < region || a + 16 > region + C::REGION) { err = fail("A-operand read at LDS byte %d outside its region [%d, %d)", a, region, region + C::REGION); return; }
                  const int r = dlt_imax(0, dlt_imin(G.r0 - WR + 4 * ch + (n >> 2), TR - 1));
                  const int col = dlt_imax(0, dlt_imin(G.c0 - WC + 4 * (pc + CG) + (n & 3), TC - 1));
                  for (int w4 = 0; w4 < 4; w4++) {
                    const Slot& s = lds[a / 4 + w4];
                    if (s.tensor != tensor || s.r != r || s.c != col || s.piece != 4 * (4 * c + g) + w4) {
                      err = fail("A-operand read (column group %d, k-piece %d) finds tensor %d row %d column %d word %d", CG, c, s.tensor, s.r, s.c, s.piece);
                      return;
                    }
                  }
                }
              };
              auto check_tr = [&](auto kbc) {
                constexpr int KB = decltype(kbc)::value;
                for (int d = 0; d < C::VB && !err; d++)
                  for (int half = 0; half < 2; half++) {
                    const int a = region + swa2_read_tr_off<C, KB>(L, d, half);
                    if (a < region || a + 8 > region + C::REGION) { err = fail("transposing read at LDS byte %d outside its region [%d, %d)", a, region, region + C::REGION); return; }
                    const int r = dlt_imax(0, dlt_imin(G.r0 - WR + 4 * ch + g, TR - 1));
                    const int col = dlt_imax(0, dlt_imin(G.c0 - WC + 4 * (pc + 2 * KB + half) + (n >> 2), TC - 1));
                    // 8 bytes = head dims 16 d + 4 (n & 3) .. + 3 of that token
                    for (int w2 = 0; w2 < 2; w2++) {
                      const Slot& s = lds[a / 4 + w2];
                      if (s.tensor != tensor || s.r != r || s.c != col || s.piece != (16 * d + 4 * (n & 3)) / 2 + w2) {
                        err = fail("transposing read (block %d, dims 16 x %d) finds tensor %d row %d column %d word %d", KB, d, s.tensor, s.r, s.c, s.piece);
                        return;
                      }
                    }
                  }
              };
              // compile-time loops over the column groups / blocks
              auto for_cg = [&](auto self, auto ic) -> void {
                constexpr int I = decltype(ic)::value;
                if constexpr (I < C::NCG) {
                  if (!err) check_a(ic);
                  self(self, std::integral_constant<int, I + 1>{});
                }
              };
              auto for_kb = [&](auto self, auto ic) -> void {
                constexpr int I = decltype(ic)::value;
                if constexpr (I < C::NKB) {
                  if (!err) check_tr(ic);
                  self(self, std::integral_constant<int, I + 1>{});
                }
              };
              for_cg(for_cg, std::integral_constant<int, 0>{});
              for_kb(for_kb, std::integral_constant<int, 0>{});
              if (err) return err;
            }
            if (kv) {
              // scalars of the queries (halo row g, window columns 4 cg .. 4 cg + 3): 16-byte reads at + 16 cg
              const int base = buf + C::BUF + swa2_scal_lane_off<C>(g, pc);
              for (int t = 0; t < 2; t++)
                for (int cg = 0; cg < C::NCG; cg++) {
                  const int a = base + t * C::TOK * 4 + 16 * cg;
                  if (a % 16 != 0) return fail("scalar read at LDS byte %d is not 16-byte aligned", a);
                  if (a < buf + C::BUF + t * C::TOK * 4 || a + 16 > buf + C::BUF + (t + 1) * C::TOK * 4) return fail("scalar read at %d outside its table", a);
                  const int r = dlt_imax(0, dlt_imin(G.r0 - WR + 4 * ch + g, TR - 1));
                  for (int i = 0; i < 4; i++) {
                    const Slot& s = lds[a / 4 + i];
                    const int col = dlt_imax(0, dlt_imin(G.c0 - WC + 4 * (pc + cg) + i, TC - 1));
                    if (s.tensor != 2 + t || s.r != r || s.c != col) return fail("scalar read (table %d, column group %d) finds tensor %d row %d column %d", t, cg, s.tensor, s.r, s.c);
                  }
                }
            }
          }
        }
      }
    }
  }
  // ---- store epilogue: wave-private tiles
  {
    std::vector<int> tile(C::TILE / 4, -1);
    for (int lane = 0; lane < 64; lane++)
      for (int d = 0; d < C::VB; d++) {
        const int n = lane & 15, g = lane >> 4;
        const int a = swa2_tile_write_off<C>(n, g, d);
        if (a < 0 || a + 8 > C::TILE) return fail("epilogue write at %d outside the tile of %d bytes", a, C::TILE);
        for (int w2 = 0; w2 < 2; w2++) {
          if (tile[a / 4 + w2] != -1) return fail("epilogue tile bytes at %d written twice", a);
          tile[a / 4 + w2] = n * (C::D / 2) + (16 * d + 4 * g) / 2 + w2;   // token n, 32-bit word of the head dim
        }
      }
    constexpr int RPI = 64 / C::PIECES;
    for (int it = 0; it < 16 / RPI; it++)
      for (int lane = 0; lane < 64; lane++) {
        const int row = lane / C::PIECES + RPI * it, c = lane % C::PIECES;
        const int a = swa2_tile_read_off<C>(row, c);
        if (a < 0 || a + 16 > C::TILE) return fail("epilogue read at %d outside the tile", a);
        for (int w4 = 0; w4 < 4; w4++)
          if (tile[a / 4 + w4] != row * (C::D / 2) + 4 * c + w4) return fail("epilogue read of row %d piece %d finds word %d", row, c, tile[a / 4 + w4]);
      }
    if (8 * C::TILE > C::LDS) return fail("eight epilogue tiles exceed the LDS of the class");
  }
  return 0;
}
}  // namespace

extern "C" {
// 0: every condition holds; 1: see swa2_model_message().  lds_bytes / lds_kv_bytes: what the launcher passes for the
// class (checked against the class constants); slab_bytes: bytes of one (batch, head) slab of a streamed tensor;
// scal_elems: elements of one (batch, head) slab of lse2 / delta.
// TC, WC: tiles per grid row and window half-width in tiles; S: tokens per tile
int swa2_model(int D, int NCG, int npass, int band, int TR, int TC, int WR, int WC, int S, int sn2, int ls2, long long slab_bytes,
               long long scal_elems, int lds_bytes, int lds_kv_bytes) {
  g_msg[0] = 0;
#define CASE(d, n) if (D == d && NCG == n) return model<Swa2Cfg<d, n>>(TR, TC, WR, WC, S, npass, band, sn2, ls2, slab_bytes, scal_elems, lds_bytes, lds_kv_bytes);
  CASE(64, 4) CASE(64, 6) CASE(64, 8) CASE(64, 10) CASE(128, 4) CASE(128, 6)
#undef CASE
  return fail("no class (%d, %d)", D, NCG);
}
const char* swa2_model_message() { return g_msg; }
int swa2_class_lds(int D, int NCG, int kv) {
#define CASE(d, n) if (D == d && NCG == n) return kv ? Swa2Cfg<d, n>::LDS_KV : Swa2Cfg<d, n>::LDS;
  CASE(64, 4) CASE(64, 6) CASE(64, 8) CASE(64, 10) CASE(128, 4) CASE(128, 6)
#undef CASE
  return -1;
}
}
