// Marching token-grid kernels (b_size == 1, head dim 64, windows up to 13 x 13): shared geometry,
// the LDS ring and its staging, swizzled operand reads and the store epilogue.
//
// A workgroup of 8 waves owns a column strip of 16 grid columns and marches down a band of grid
// rows in steps of 8 rows.  In a step wave w owns the 4x4 patch of own tokens at rows 4 (w >> 2),
// columns 4 (w & 3) of the step's 8 x 16 block.  The tokens of the other side that any of them can
// see (20 halo rows x 28 halo columns) are resident in LDS as 5 chunks of 4 halo rows: chunk c
// holds grid rows band_r0 - WR + 4 c .. + 3 and lives in slot c % 5.  Going to the next step
// replaces the two oldest chunks, so every halo row is fetched once per band instead of once per 4
// own rows, a workgroup's prologue and address set-up are paid once per band, and the chunks of
// the next step travel HBM -> registers while the current step computes.
//
// LDS rows are 2 D bytes with no padding; the 16-byte piece `ch` of token row t is stored at piece
// ch ^ (t & 7) (the low token bits inside a chunk), which keeps the operand reads of a wave (16
// lanes x 16 bytes, or 32 lanes x 8 bytes for the transposing read) on distinct banks.
#pragma once
#include "swa1_common.hpp"

typedef DLT_LDS const char* SwamLds;   // 32-bit LDS address: constant parts of an offset fold into the instruction

constexpr int SWAM_HCW = 28;               // staged halo columns: 16 own + 2 * 6
constexpr int SWAM_TOK = 4 * SWAM_HCW;     // tokens of a chunk
constexpr int SWAM_NSLOT = 5;
constexpr int SWAM_THREADS = 512;
constexpr int swam_region(int d) { return SWAM_TOK * 2 * d; }   // one tensor of a chunk
constexpr int swam_slot(int d) { return 2 * swam_region(d); }    // both tensors of a chunk
constexpr int swam_ring(int d) { return SWAM_NSLOT * swam_slot(d); }

struct SwamPlan {
  int32_t band;     // grid rows per workgroup (a multiple of 8)
  int32_t nbands, nstrips;
  uint32_t m_bh, s_bh, m_st, s_st, m_h, s_h;   // exact multiply-shift divisions by nbands * nstrips, nstrips and H
};

struct SwamGeom {
  int TR, TC, WR, WC;
  int r0, c0;     // first grid row of the band, first grid column of the strip
  int nch;        // chunks a patch window spans: ceil((4 + 2 WR) / 4), 1..4
  int nstep;      // steps of this band that hold grid rows
  int b, h;
};

DLT_DEV SwamGeom swam_geom(const AttnProblem& p, const SwamPlan& P) {
  SwamGeom G;
  const int lin = xcd_remap(blockIdx.x, gridDim.x);
  const int per_bh = P.nbands * P.nstrips;
  const int bh = (int)dlt_fastdiv((uint32_t)lin, P.m_bh, P.s_bh);
  const int rem = lin - bh * per_bh;
  const int band = (int)dlt_fastdiv((uint32_t)rem, P.m_st, P.s_st);
  G.b = (int)dlt_fastdiv((uint32_t)bh, P.m_h, P.s_h);
  G.h = bh - G.b * p.H;
  G.TR = p.g.TR; G.TC = p.g.TC; G.WR = p.g.WR; G.WC = p.g.WC;
  G.r0 = band * P.band;
  G.c0 = 16 * (rem - band * P.nstrips);
  G.nch = (4 + 2 * G.WR + 3) >> 2;
  G.nstep = (dlt_imin(P.band, G.TR - G.r0) + 7) >> 3;
  return G;
}

// ---- staging: one 64-byte item per thread, chunk and tensor --------------------------------------
// Thread t of the lower half of the workgroup (waves 0-3) stages tensor A (the one that may be
// rotated) of even chunks and tensor B of odd chunks, the upper half the other way round, so that
// every wave does the same share of rotation work.  Within a half thread lt stages the piece qd =
// lt & 1 of token lt >> 1: the rotary pair of 16-byte pieces (2 qd, 2 qd + 1) and the unrotated pieces
// (4 + 2 qd, 5 + 2 qd) (head dim 64, 8 rotary pairs per axis: pieces 0, 1 turn by the row angle,
// 2, 3 by the column angle).
struct SwamStage {
  int hr;          // halo row inside a chunk
  int cc;          // grid column, clamped onto the grid
  bool live;       // the thread has a token in every chunk (112 of 128 per tensor)
  bool own_col;    // its column belongs to the strip (and to the grid)
  int qd;
  int lds_off[4];  // byte offsets of its four pieces inside a chunk region
};

DLT_DEV void swam_stage_init(SwamStage& st, const SwamGeom& G, int tid) {
  const int lt = tid & 255;
  int tok = lt >> 1;
  st.qd = lt & 1;
  st.live = tok < SWAM_TOK;
  if (!st.live) tok = 0;
  st.hr = (tok * 147) >> 12;   // tok / 28 for tok < 128
  const int hc = tok - st.hr * SWAM_HCW;
  const int col = G.c0 - G.WC + hc;
  st.cc = dlt_imax(0, dlt_imin(col, G.TC - 1));
  st.own_col = st.live && col >= G.c0 && col < G.c0 + 16 && col < G.TC;
  const int piece[4] = {2 * st.qd, 2 * st.qd + 1, 4 + 2 * st.qd, 5 + 2 * st.qd};
#pragma unroll
  for (int j = 0; j < 4; j++) st.lds_off[j] = tok * 128 + 16 * (piece[j] ^ (tok & 7));
}

// One tensor as the staging threads address it: byte offset of a token piece = row * rowstride + coloff, with the
// thread's column and its first piece folded into coloff; the four pieces lie at +0, +16, +64, +80.
struct SwamSide {
  const char* base;
  uint32_t rowstride;   // bytes between grid rows
  uint32_t coloff;
};

DLT_DEV SwamSide swam_side(const char* base, int sn2, const SwamGeom& G, const SwamStage& st) {
  SwamSide sd;
  sd.base = base;
  sd.rowstride = (uint32_t)(G.TC * sn2);
  sd.coloff = (uint32_t)(st.cc * sn2 + 32 * st.qd);
  return sd;
}

struct SwamItem {
  u32x4 v[4];
  int row;      // unclamped grid row of the token
};

// grid row of halo row `hr` of chunk `c`, clamped onto the grid: positions outside are always masked
// by the window test, so their (finite) values never reach a result
DLT_DEV int swam_item_row(const SwamStage& st, const SwamGeom& G, int c) { return G.r0 - G.WR + 4 * c + st.hr; }

DLT_DEV void swam_issue(SwamItem& it, const SwamStage& st, const SwamGeom& G, int c, const SwamSide& sd) {
  it.row = swam_item_row(st, G, c);
  const int r = dlt_imax(0, dlt_imin(it.row, G.TR - 1));
  const char* p = sd.base + ((uint32_t)r * sd.rowstride + sd.coloff);
  it.v[0] = *reinterpret_cast<const u32x4*>(p);
  it.v[1] = *reinterpret_cast<const u32x4*>(p + 16);
  it.v[2] = *reinterpret_cast<const u32x4*>(p + 64);
  it.v[3] = *reinterpret_cast<const u32x4*>(p + 80);
}

// packed rotary index of the token the thread stages in chunk c
DLT_DEV int32_t swam_issue_idx(const SwamStage& st, const SwamGeom& G, int c, const int32_t* rope_idx) {
  const int r = dlt_imax(0, dlt_imin(swam_item_row(st, G, c), G.TR - 1));
  return rope_idx[r * G.TC + st.cc];
}

DLT_DEV void swam_pin(const SwamItem& it) {
#pragma unroll
  for (int j = 0; j < 4; j++) pin_loaded(it.v[j]);
}

struct SwamTab {
  f32x4 t[4];   // (cos, sin) of the 8 pair elements
  bool rot;
};

DLT_DEV void swam_tab_issue(SwamTab& tb, int32_t id, int axis, const RopeDev& rope) {
  bool rotated;
  const float* tab = rope_table_row(rope, axis, id, rotated);
  tb.rot = rotated;
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const float* tj = tab + 4 * j;
    tb.t[j] = f32x4{tj[0], tj[1], tj[2], tj[3]};
  }
}

// ---- rotary tables resident in LDS --------------------------------------------------------------------
// Both tables (8 rotary pairs: 64 bytes per position) are copied into LDS once per workgroup when they fit
// SWAM_TAB_BYTES: row table first, the column table behind it.  A table row then costs four LDS reads instead of a
// global load that can only be requested once the token's index has arrived (index -> table row is a dependent chain
// in front of every rotation: in the prologue, between the steps, in front of the rotating stores).
constexpr int SWAM_TAB_BYTES = 8192;
DLT_DEV bool swam_tab_fits(const RopeDev& rope) { return (rope.row_len + rope.col_len) * 64 <= SWAM_TAB_BYTES; }

// the 16 bytes thread `tid` of the 512 copies (threads past the tables' end re-read the last row: no access out of bounds)
DLT_DEV f32x4 swam_tab_fetch(const RopeDev& rope, int tid) {
  const int row = tid >> 2, q = tid & 3;
  const int rc = dlt_imin(row, rope.row_len + rope.col_len - 1);
  const float* p = rc < rope.row_len ? rope.row_cs + (int64_t)rc * rope.rs0 : rope.col_cs + (int64_t)(rc - rope.row_len) * rope.cs0;
  p += 4 * q;
  return f32x4{p[0], p[1], p[2], p[3]};
}
DLT_DEV void swam_tab_store(char* tabs, int tid, const f32x4& v) { *reinterpret_cast<f32x4*>(tabs + 16 * tid) = v; }

// table row of a token from the LDS copy (TL) or from global memory
template <bool TL>
DLT_DEV void swam_tab_get(SwamTab& tb, int32_t id, int axis, const RopeDev& rope, SwamLds tabs) {
  if constexpr (TL) {
    int pos = axis == 0 ? dlt_rope_row(id) : dlt_rope_col(id);
    tb.rot = pos >= 0;
    pos = dlt_imax(0, dlt_imin(pos, (axis == 0 ? rope.row_len : rope.col_len) - 1));
    SwamLds p = tabs + ((axis == 0 ? 0 : rope.row_len) + pos) * 64;
#pragma unroll
    for (int j = 0; j < 4; j++) tb.t[j] = *reinterpret_cast<DLT_LDS const f32x4*>(p + 16 * j);
  } else {
    swam_tab_issue(tb, id, axis, rope);
  }
}

// rotate the pair (lo, hi) = (first, second element of each of 8 rotary pairs); `inverse`: transposed rotation
template <typename CT>
DLT_DEV void swam_rotate_pair(u32x4& lo, u32x4& hi, const SwamTab& tb, bool inverse) {
  if (!tb.rot) return;
  float x0[8], x1[8];
  unpack8<CT>(lo, x0);
  unpack8<CT>(hi, x1);
  const unsigned s0 = rope_sign_mask(true, inverse), s1 = rope_sign_mask(false, inverse);
#pragma unroll
  for (int j = 0; j < 8; j++) {
    const float cs = tb.t[j >> 1][2 * (j & 1)], sn = tb.t[j >> 1][2 * (j & 1) + 1];
    const float y0 = rope_mix_signed(x0[j], x1[j], cs, sn, s0);
    const float y1 = rope_mix_signed(x1[j], x0[j], cs, sn, s1);
    x0[j] = y0; x1[j] = y1;
  }
  lo = pack8<CT>(x0);
  hi = pack8<CT>(x1);
}

DLT_DEV void swam_commit(const SwamItem& it, const SwamStage& st, char* region) {
  if (st.live) {
#pragma unroll
    for (int j = 0; j < 4; j++) lds_write16(region + st.lds_off[j], it.v[j]);
  }
}

// ---- operand reads --------------------------------------------------------------------------------
// Lane constants of a wave whose window starts at halo column 4 pc.
struct SwamLane {
  int a_even, a_odd;   // A operand (token = MFMA row, head dim along k): byte offset of k-piece 0 of the lane's
                       // token row for an even / odd column group; k-piece 1 sits at the other one's piece
  int tr[4];           // transposing read (head dim = MFMA row, tokens along k): byte offset for dims 16 d .. + 15
};

DLT_DEV void swam_lane_init(SwamLane& L, int pc, int n, int g) {
  // A operand: lane (n, g) reads token (halo row n >> 2, column 4 (pc + cg) + (n & 3)) of a chunk, pieces g and 4 + g;
  // t & 7 = (n & 3) | 4 * ((n >> 2) + pc + cg & 1)
  const int tok = (n >> 2) * SWAM_HCW + 4 * pc + (n & 3);
  const int par = ((n >> 2) + pc) & 1;
  const int low = 16 * (g ^ (n & 3));
  L.a_even = tok * 128 + low + 64 * par;
  L.a_odd = tok * 128 + low + 64 * (par ^ 1);
  // transposing read: lane (n, g) addresses token (halo row g, column 4 (pc + cg0) + (n >> 2)), cg0 even, 8 bytes at dim
  // 16 d + 4 (n & 3); t & 7 = (n >> 2) | 4 * ((g + pc) & 1)
  const int tok2 = g * SWAM_HCW + 4 * pc + (n >> 2);
  const int x = (n >> 2) | (4 * ((g + pc) & 1));
#pragma unroll
  for (int d = 0; d < 4; d++) {
    const int piece = (2 * d + ((n & 3) >> 1)) ^ x;
    L.tr[d] = tok2 * 128 + 16 * piece + 8 * (n & 1);
  }
}

DLT_DEV u32x4 swam_lds16(SwamLds p) { return *reinterpret_cast<DLT_LDS const u32x4*>(p); }
DLT_DEV u32x2 swam_lds_tr(SwamLds p) {
  s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((DLT_LDS s16x4*)(p));
  return __builtin_bit_cast(u32x2, v);
}

// A-operand pieces of the 64 tokens (4 halo rows x 16 window columns) of a chunk region: ka[2 cg + c] = k-piece c of the
// 16 tokens at column group cg
DLT_DEV void swam_read_a_chunk(SwamLds region, const SwamLane& L, u32x4 (&ka)[8]) {
  SwamLds pe = region + L.a_even, po = region + L.a_odd;
  ka[0] = swam_lds16(pe);        ka[1] = swam_lds16(po);
  ka[2] = swam_lds16(po + 512);  ka[3] = swam_lds16(pe + 512);
  ka[4] = swam_lds16(pe + 1024); ka[5] = swam_lds16(po + 1024);
  ka[6] = swam_lds16(po + 1536); ka[7] = swam_lds16(pe + 1536);
}

// the same for one half of the window columns: column groups 2 kb and 2 kb + 1 (ka[2 i + c] = k-piece c of group 2 kb + i)
template <int KB>
DLT_DEV void swam_read_a_half(SwamLds region, const SwamLane& L, u32x4 (&ka)[4]) {
  SwamLds pe = region + L.a_even, po = region + L.a_odd;
  ka[0] = swam_lds16(pe + 1024 * KB);       ka[1] = swam_lds16(po + 1024 * KB);
  ka[2] = swam_lds16(po + 1024 * KB + 512); ka[3] = swam_lds16(pe + 1024 * KB + 512);
}

// A operands with tokens along k for the 32 tokens (4 halo rows x 8 columns) at column groups 2 kb, 2 kb + 1 of a chunk
// region: va[d] has dims 16 d .. 16 d + 15 as its rows
template <int KB>
DLT_DEV void swam_read_tr_block(SwamLds region, const SwamLane& L, u32x4 (&va)[4]) {
#pragma unroll
  for (int d = 0; d < 4; d++) {
    const u32x2 lo = swam_lds_tr(region + L.tr[d] + 1024 * KB);
    const u32x2 hi = swam_lds_tr(region + L.tr[d ^ 2] + 1024 * KB + 512);
    va[d].x = lo.x; va[d].y = lo.y; va[d].z = hi.x; va[d].w = hi.y;
  }
}

// ---- store epilogue --------------------------------------------------------------------------------
// Accumulators in C layout (lane (n, g) holds dims 16 d + 4 g .. + 3 of own token n, times `mul`) -> a
// wave-private LDS tile [16 tokens][128 bytes] (pieces swizzled with the token index) -> 16-byte pieces:
// out[it] = piece lane & 7 of token (lane >> 3) + 8 it.  With ROT the rotary partner pieces are returned too.
template <typename CT, bool ROT>
DLT_DEV void swam_tile_transpose(char* sW, const f32x4 (&acc)[4], float mul, int lane, u32x4 (&out)[2], u32x4 (&partner)[2]) {
  const int n = lane & 15, g = lane >> 4;
#pragma unroll
  for (int d = 0; d < 4; d++) {
    u32x2 w;
    w.x = pack2<CT>(acc[d][0] * mul, acc[d][1] * mul);
    w.y = pack2<CT>(acc[d][2] * mul, acc[d][3] * mul);
    *reinterpret_cast<u32x2*>(sW + n * 128 + 16 * ((2 * d + (g >> 1)) ^ (n & 7)) + 8 * (g & 1)) = w;
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  const int c = lane & 7;
#pragma unroll
  for (int it = 0; it < 2; it++) {
    const int row = (lane >> 3) + 8 * it;
    out[it] = lds_read16(sW + row * 128 + 16 * (c ^ (row & 7)));
    if (ROT) partner[it] = lds_read16(sW + row * 128 + 16 * ((c ^ 1) ^ (row & 7)));
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
}

// rotate piece c = lane & 7 (< 4: rotary pieces 0-1 row angle, 2-3 column angle) of a transposed tile row
template <typename CT>
DLT_DEV void swam_rotate_piece(u32x4& v, const u32x4& pv, const SwamTab& tb, int c, bool inverse) {
  if (c >= 4 || !tb.rot) return;
  float self[8], partner[8];
  unpack8<CT>(v, self);
  unpack8<CT>(pv, partner);
  const unsigned sm = rope_sign_mask((c & 1) == 0, inverse);
#pragma unroll
  for (int j = 0; j < 8; j++)
    self[j] = rope_mix_signed(self[j], partner[j], tb.t[j >> 1][2 * (j & 1)], tb.t[j >> 1][2 * (j & 1) + 1], sm);
  v = pack8<CT>(self);
}

template <typename TIO>
DLT_DEV void swam_store_rows(TIO* base, int64_t sn, const int (&tok)[2], int lane, const u32x4 (&v)[2]) {
#pragma unroll
  for (int it = 0; it < 2; it++)
    if (tok[it] >= 0) store_stream16(base + (int64_t)tok[it] * sn + 8 * (lane & 7), v[it]);
}
