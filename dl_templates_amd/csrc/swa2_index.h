// Streaming token-grid kernels: the integer side (geometry of a workgroup, windows, and every byte offset into global
// memory and LDS), shared by the kernels and by a host-compiled model of the staging / operand-read maps
// (tests/swa2_shim.cpp).  No device-only construct lives here.
//
// A workgroup of 8 waves owns a band of 8 grid rows x 16 grid columns; wave w owns the 4x4 patch at rows
// 4 (w >> 2), columns 4 (w & 3).  The halo of the band (8 + 2 WR rows x HCW columns, first halo column = c0 - WC)
// streams through LDS in chunks of 4 halo rows.  Stacked variant (Swa2Plan::band = 16): a band of 16 grid rows, wave w
// owns the two 4x4 patches at rows 8 (w >> 2) and 8 (w >> 2) + 4, columns 4 (w & 3): "row group" rg below is then 0 .. 3.
//
// Tiles of S tokens (1 < S < 16): a grid row then holds TC = tiles * S token slots ("columns" below are slots), a token
// in tile t sees the slots of tiles t - WCt .. t + WCt, i.e. S WCt + (x mod S) slots to its left and S WCt + S - 1 - (x mod S)
// to its right; WC is the largest of these extents, S WCt + S - 1, and positions the halo.  S = 1: WC = WCt.  LDS rows are 2 D bytes with no padding; the 16-byte piece c of token
// row t (t = halo row inside the chunk * HCW + halo column) is stored at piece c ^ (SWZ (t & 7)).
#pragma once
#include "dlt_geom.h"

constexpr int SWA2_THREADS = 512;

template <int D_, int NCG_>
struct Swa2Cfg {
  static constexpr int D = D_, NCG = NCG_;
  static constexpr int NKB = NCG / 2;            // blocks of 32 streamed tokens (two column groups) per chunk
  static constexpr int KC = D / 32;              // 32-dim steps of a product that contracts over the head dim
  static constexpr int VB = D / 16;              // 16-dim blocks of an accumulator
  static constexpr int HCW = 4 * NCG + 12;       // staged halo columns
  static constexpr int TOK = 4 * HCW;            // tokens of a chunk
  static constexpr int ROW = 2 * D;              // bytes of a token row
  static constexpr int PIECES = ROW / 16;        // 16-byte pieces of a row
  static constexpr int SWZ = PIECES / 8;         // swizzle multiplier
  static constexpr int TPI = 64 / PIECES;        // tokens per copy instruction
  static constexpr int NI = (HCW + TPI - 1) / TPI;   // copy instructions per halo row
  static constexpr int REGION = TOK * ROW;       // one tensor of a chunk
  static constexpr int BUF = 2 * REGION;         // both tensors of a chunk
  static constexpr int LDS = 2 * BUF;            // two chunk buffers
  static constexpr int SCAL = 2 * TOK * 4;       // per-token scalars of a chunk (dK/dV kernel): lse2 then delta
  static constexpr int BUF_KV = BUF + SCAL;
  static constexpr int LDS_KV = 2 * BUF_KV;
  static constexpr int TILE = 16 * ROW;          // wave-private tile of the store epilogue
  // issue slots a chunk body offers for the copies of the next chunk (one copy instruction per slot)
  static constexpr int SLOTS_FWD = NCG + NKB * (VB / 4);
  static constexpr int SLOTS_BWD = 4 * NKB;
  static_assert(NCG % 2 == 0 && NCG >= 4, "column groups come in pairs (32-token blocks)");
  static_assert(HCW % 8 == 4, "the operand-read swizzle assumes HCW = 4 mod 8");
  static_assert(HCW <= 64, "one 4-byte copy instruction per halo row of scalars");
  static_assert(NI <= SLOTS_FWD && NI <= SLOTS_BWD, "more copy instructions per halo row than issue slots in a chunk body");
  static_assert(8 * TILE <= LDS, "the store epilogue reuses the chunk buffers");
  static_assert(LDS_KV <= 160 * 1024, "LDS of a CU");
};

struct Swa2Plan {
  int32_t nblk_r, nblk_c;
  uint32_t m_bh, s_bh, m_c, s_c, m_h, s_h;   // exact multiply-shift divisions by nblk_r * nblk_c, nblk_c and H
  int32_t npass;   // column passes: a window of more than NCG column groups is walked in npass slices of NCG groups
  int32_t S, WCt;  // tokens per tile, window half-width in tiles
  uint32_t m_S, s_S;   // division by S
  int32_t band;    // grid rows of a workgroup's band: 8 (one patch per wave) or 16 (two stacked patches per wave)
};

struct Swa2Geom {
  int TR, TC, WR, WC;   // grid rows, token slots per row, window half-height in rows, largest column extent in slots
  int r0, c0;   // first grid row / column of the band
  int b, h;
  int ch_first, ch_last;   // chunks of the band's halo that hold grid rows
  int S, WCt;
  uint32_t m_S, s_S;
};

// plan fields of a token grid (one token per tile)
DLT_HD void swa2_plan_tokens(Swa2Plan& P, int WC) {
  P.S = 1; P.WCt = WC;
  dlt_fastdiv_make(1u, P.m_S, P.s_S);
}

// geometry of workgroup `lin` (its index after the XCD remap); TC: token slots per grid row, WC: S WCt + S - 1
DLT_HD Swa2Geom swa2_geom_at(int TR, int TC, int WR, int WC, int H, const Swa2Plan& P, int lin) {
  Swa2Geom G;
  G.S = P.S; G.WCt = P.WCt; G.m_S = P.m_S; G.s_S = P.s_S;
  const int per_bh = P.nblk_r * P.nblk_c;
  const int bh = (int)dlt_fastdiv((uint32_t)lin, P.m_bh, P.s_bh);
  const int rem = lin - bh * per_bh;
  const int br = (int)dlt_fastdiv((uint32_t)rem, P.m_c, P.s_c);
  G.b = (int)dlt_fastdiv((uint32_t)bh, P.m_h, P.s_h);
  G.h = bh - G.b * H;
  G.TR = TR; G.TC = TC; G.WR = WR; G.WC = WC;
  G.r0 = P.band * br;
  G.c0 = 16 * (rem - br * P.nblk_c);
  const int lo = dlt_imax(0, G.WR - G.r0), hi = dlt_imin(P.band - 1 + 2 * G.WR, G.TR - 1 - G.r0 + G.WR);
  G.ch_first = lo >> 2;
  G.ch_last = hi >> 2;
  return G;
}

// per-lane window of an own token in the coordinates of the band's halo
struct Swa2Win {
  int rlo, rhi;      // visible halo rows [rlo, rhi]
  int clo, cspan;    // visible window columns [clo, clo + cspan] (cspan < 0: the token lies outside the grid)
  int ch_lo, ch_hi;  // chunks that hold visible rows of the wave's patch (wave-uniform)
};

DLT_HD Swa2Win swa2_window(const Swa2Geom& G, int rg, int pc, int n) {
  Swa2Win w;
  const int qr = 4 * rg + (n >> 2), qc = n & 3;
  const int c_p = G.c0 + 4 * pc;
  const bool ok = (G.r0 + qr < G.TR) && (c_p + qc < G.TC);
  w.rlo = dlt_imax(qr, G.WR - G.r0);
  w.rhi = dlt_imin(qr + 2 * G.WR, G.TR - 1 - G.r0 + G.WR);
  // window columns: the wave window starts at slot c_p - WC, the own token sits at window column WC + qc
  const int x = c_p + qc;
  const int xm = x - G.S * (int)dlt_fastdiv((uint32_t)x, G.m_S, G.s_S);   // slot inside its tile
  const int reach = G.S * G.WCt;
  w.clo = dlt_imax(G.WC + qc - reach - xm, G.WC - c_p);
  const int chi = dlt_imin(G.WC + qc + reach + (G.S - 1 - xm), G.TC - 1 - c_p + G.WC);
  w.cspan = ok ? chi - w.clo : -1;
  // halo rows of the patch that hold grid rows
  const int plo = dlt_imax(4 * rg, G.WR - G.r0), phi = dlt_imin(4 * rg + 3 + 2 * G.WR, G.TR - 1 - G.r0 + G.WR);
  const bool patch_ok = (G.r0 + 4 * rg < G.TR) && (c_p < G.TC) && plo <= phi;
  w.ch_lo = patch_ok ? plo >> 2 : 1;
  w.ch_hi = patch_ok ? phi >> 2 : 0;
  return w;
}

// Windows wider than the class (more than NCG column groups per wave) are walked in column passes: pass s covers the
// window columns 4 NCG s .. 4 NCG (s + 1) - 1 of every wave.  Everything that addresses columns sees a pass through a
// geometry whose column half-width is reduced by the pass's offset (halo column 0 of the pass = grid column
// c0 - WC + 4 NCG s) and a window whose first visible column is moved by the same amount; rows are untouched, and the
// running softmax / the gradient accumulators simply carry on from pass to pass.
DLT_HD Swa2Geom swa2_pass_geom(const Swa2Geom& G, int ncg_class, int pass) {
  Swa2Geom P = G;
  P.WC = G.WC - 4 * ncg_class * pass;
  return P;
}
DLT_HD Swa2Win swa2_pass_window(const Swa2Win& W, int ncg_class, int pass) {
  Swa2Win P = W;
  P.clo = W.clo - 4 * ncg_class * pass;
  return P;
}
// column groups of pass `pass` that can hold a visible token (window of WC columns to each side)
DLT_HD int swa2_pass_ncg(int WC, int ncg_class, int pass) { return dlt_imin(ncg_class, ((4 + 2 * WC + 3) >> 2) - ncg_class * pass); }

// visibility of the streamed token (halo row covered by row_vis, window column 4 cg + i) from the lane's own token
DLT_HD bool swa2_visible(const Swa2Win& W, bool row_vis, int cg, int i, int ncg) {
  return row_vis & (cg < ncg) & ((unsigned)(4 * cg + i - W.clo) <= (unsigned)W.cspan);
}

// ---- asynchronous staging -------------------------------------------------------------------------------
// Wave w copies halo row (w & 3) of tensor (w >> 2) of every chunk in NI instructions of 64 lanes; instruction i,
// lane l writes LDS slot 64 i + l of the row = physical piece l % PIECES of halo column TPI i + l / PIECES, and
// therefore fetches the logical piece (l % PIECES) ^ (SWZ (token & 7)) of that token.  Lanes past the last halo
// column of the last instruction stay idle.

// byte offset, inside a grid row of the tensor (token stride sn2 bytes), of the piece lane `lane` fetches in instruction i
template <typename C>
DLT_HD uint32_t swa2_stage_off(const Swa2Geom& G, int wave, int lane, int sn2, int i) {
  const int hc = C::TPI * i + lane / C::PIECES;
  const int tok = (wave & 3) * C::HCW + hc;
  const int cc = dlt_imax(0, dlt_imin(G.c0 - G.WC + hc, G.TC - 1));   // clamped: positions outside the grid are masked
  return (uint32_t)(cc * sn2 + 16 * ((lane % C::PIECES) ^ (C::SWZ * (tok & 7))));
}
// the lane takes part in the last instruction of a halo row
template <typename C>
DLT_HD bool swa2_stage_last_on(int lane) { return C::TPI * (C::NI - 1) + lane / C::PIECES < C::HCW; }
// lane `lane` takes part in instruction i
template <typename C>
DLT_HD bool swa2_stage_on(int lane, int i) { return i + 1 < C::NI || C::HCW % C::TPI == 0 || swa2_stage_last_on<C>(lane); }
// grid row (clamped onto the grid) that wave `wave` copies for chunk ch
DLT_HD int swa2_issue_grid_row(const Swa2Geom& G, int ch, int wave) {
  return dlt_imax(0, dlt_imin(G.r0 - G.WR + 4 * ch + (wave & 3), G.TR - 1));
}
// byte offset inside a chunk buffer of the halo row wave `wave` copies (instruction i starts 1024 i bytes further on)
template <typename C>
DLT_HD int swa2_issue_dst_off(int wave) { return (wave >> 2) * C::REGION + (wave & 3) * (C::HCW * C::ROW); }

// per-token scalars of the dK/dV kernel: lane l < HCW of wave w copies the scalar of halo column l of halo row (w & 3)
// of tensor (w >> 2) (lse2, delta) into the table behind the chunk's rows
DLT_HD int swa2_scal_col(const Swa2Geom& G, int lane) { return dlt_imax(0, dlt_imin(G.c0 - G.WC + lane, G.TC - 1)); }
template <typename C>
DLT_HD int swa2_scal_dst_off(int wave) { return C::BUF + (wave >> 2) * (C::TOK * 4) + (wave & 3) * (C::HCW * 4); }
// byte offset (from the start of the lse2 table; delta: + 4 TOK) of the four scalars of halo row g, window columns
// 4 cg .. 4 cg + 3 of the wave at patch column pc: + 16 cg
template <typename C>
DLT_HD int swa2_scal_lane_off(int g, int pc) { return (g * C::HCW + 4 * pc) * 4; }

// ---- operand reads -----------------------------------------------------------------------------------------
// Lane constants of a wave whose window starts at halo column 4 pc.
template <typename C>
struct Swa2Lane {
  int a[C::KC];    // A operand (token = MFMA row, head dim along k): byte offset of k-piece c of the lane's token row for an
                   // even column group (odd groups: a[c ^ (KC / 2)])
  int tr[C::VB];   // transposing read (head dim = MFMA row, tokens along k): byte offset for dims 16 d .. 16 d + 15
};

template <typename C>
DLT_HD void swa2_lane_init(Swa2Lane<C>& L, int pc, int n, int g) {
  // A operand: lane (n, g) reads token (halo row n >> 2, column 4 (pc + cg) + (n & 3)) of a chunk, pieces 4 c + g;
  // token & 7 = (n & 3) | 4 ((n >> 2) + pc + cg & 1)  (HCW = 4 mod 8)
  const int tok = (n >> 2) * C::HCW + 4 * pc + (n & 3);
  const int par = ((n >> 2) + pc) & 1;
#pragma unroll
  for (int c = 0; c < C::KC; c++) L.a[c] = tok * C::ROW + 16 * ((4 * c + g) ^ (C::SWZ * ((n & 3) | (4 * par))));
  // transposing read: lane (n, g) addresses token (halo row g, column 4 (pc + cg0) + (n >> 2)), cg0 even, 8 bytes at dim
  // 16 d + 4 (n & 3): piece 2 d + ((n & 3) >> 1); token & 7 = (n >> 2) | 4 ((g + pc) & 1)
  const int tok2 = g * C::HCW + 4 * pc + (n >> 2);
  const int sw = C::SWZ * ((n >> 2) | (4 * ((g + pc) & 1)));
#pragma unroll
  for (int d = 0; d < C::VB; d++) L.tr[d] = tok2 * C::ROW + 16 * ((2 * d + ((n & 3) >> 1)) ^ sw) + 8 * (n & 1);
}

// byte offset inside a chunk region of the 16 bytes lane L reads as k-piece c (head dims 32 c + 8 g .. + 7) of the 16
// tokens at column group CG
template <typename C, int CG>
DLT_HD int swa2_read_a_off(const Swa2Lane<C>& L, int c) { return 4 * C::ROW * CG + L.a[(CG & 1) ? (c ^ (C::KC / 2)) : c]; }
// byte offset inside a chunk region of the 8 bytes lane L addresses in the transposing read of head dims 16 d .. + 15 of
// the 32 tokens at column groups 2 KB (half 0) and 2 KB + 1 (half 1)
template <typename C, int KB>
DLT_HD int swa2_read_tr_off(const Swa2Lane<C>& L, int d, int half) {
  return 8 * C::ROW * KB + (half ? 4 * C::ROW + L.tr[d ^ (C::VB / 2)] : L.tr[d]);
}

// ---- store epilogue: wave-private LDS tile [16 tokens][2 D bytes], pieces swizzled with the token index -----------
// 8 bytes lane (n, g) writes for accumulator block d (dims 16 d + 4 g .. + 3 of own token n)
template <typename C>
DLT_HD int swa2_tile_write_off(int n, int g, int d) { return n * C::ROW + 16 * ((2 * d + (g >> 1)) ^ (n & 7)) + 8 * (g & 1); }
// 16 bytes read back as piece c of tile row `row`
template <typename C>
DLT_HD int swa2_tile_read_off(int row, int c) { return row * C::ROW + 16 * (c ^ (row & 7)); }
