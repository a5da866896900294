// Streaming token-grid kernels (b_size == 1, head dim 64 or 128, windows up to 21 columns, any number of rows):
// shared geometry, asynchronous staging and swizzled operand reads.
//
// A workgroup of 8 waves owns a band of 8 grid rows x 16 grid columns; wave w owns the 4x4 patch at rows
// 4 (w >> 2), columns 4 (w & 3).  The tokens of the other side that any own token can see (8 + 2 WR halo rows x HCW
// halo columns) stream through LDS in chunks of 4 halo rows.  A chunk is copied HBM -> LDS by the DMA path of the
// vector memory unit (16 bytes per lane, no staging registers: at head dim 128 those were a third of the register
// file) into one of two buffers while the other one is consumed, so a chunk costs one workgroup barrier, every
// halo row is fetched once per 8 own rows, and the registers go to operand read-ahead instead.
//
// A wave's window is NCG column groups of 4 halo columns (NCG = 4: windows up to 13 columns, 6: up to 21), so
// HCW = 16 + 4 NCG - 4 halo columns are staged.  LDS rows are 2 D bytes with no padding; the 16-byte piece c of token
// row t is stored at piece c ^ (m (t & 7)), m = D / 64: operand reads of a wave (16 lanes x 16 bytes, or 32 lanes x
// 8 bytes for the transposing read) then fall on distinct banks, and so do the 64 x 16 bytes a copy instruction writes.
#pragma once
#include <type_traits>
#include "swa1_common.hpp"

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
};

// compile-time loop: f(std::integral_constant<int, I>) for I = I0 .. N - 1
template <int I, int N, typename F>
DLT_DEV void swa2_for(F&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    swa2_for<I + 1, N>(f);
  }
}

typedef DLT_LDS const char* Swa2Lds;
DLT_DEV u32x4 swa2_lds16(Swa2Lds p) { return *reinterpret_cast<DLT_LDS const u32x4*>(p); }
DLT_DEV u32x2 swa2_lds_tr(Swa2Lds p) {
  s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((DLT_LDS s16x4*)(p));
  return __builtin_bit_cast(u32x2, v);
}

struct Swa2Plan {
  int32_t nblk_r, nblk_c;
  uint32_t m_bh, s_bh, m_c, s_c, m_h, s_h;   // exact multiply-shift divisions by nblk_r * nblk_c, nblk_c and H
};

struct Swa2Geom {
  int TR, TC, WR, WC;
  int r0, c0;   // first grid row / column of the band
  int b, h;
  int ch_first, ch_last;   // chunks of the band's halo that hold grid rows
};

DLT_DEV Swa2Geom swa2_geom(const AttnProblem& p, const Swa2Plan& P) {
  Swa2Geom G;
  const int lin = xcd_remap(blockIdx.x, gridDim.x);
  const int per_bh = P.nblk_r * P.nblk_c;
  const int bh = (int)dlt_fastdiv((uint32_t)lin, P.m_bh, P.s_bh);
  const int rem = lin - bh * per_bh;
  const int br = (int)dlt_fastdiv((uint32_t)rem, P.m_c, P.s_c);
  G.b = (int)dlt_fastdiv((uint32_t)bh, P.m_h, P.s_h);
  G.h = bh - G.b * p.H;
  G.TR = p.g.TR; G.TC = p.g.TC; G.WR = p.g.WR; G.WC = p.g.WC;
  G.r0 = 8 * br;
  G.c0 = 16 * (rem - br * P.nblk_c);
  const int lo = dlt_imax(0, G.WR - G.r0), hi = dlt_imin(7 + 2 * G.WR, G.TR - 1 - G.r0 + G.WR);
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

DLT_DEV Swa2Win swa2_window(const Swa2Geom& G, int rg, int pc, int n) {
  Swa2Win w;
  const int qr = 4 * rg + (n >> 2), qc = n & 3;
  const int c_p = G.c0 + 4 * pc;
  const bool ok = (G.r0 + qr < G.TR) && (c_p + qc < G.TC);
  w.rlo = dlt_imax(qr, G.WR - G.r0);
  w.rhi = dlt_imin(qr + 2 * G.WR, G.TR - 1 - G.r0 + G.WR);
  w.clo = dlt_imax(qc, G.WC - c_p);
  const int chi = dlt_imin(qc + 2 * G.WC, G.TC - 1 - c_p + G.WC);
  w.cspan = ok ? chi - w.clo : -1;
  // halo rows of the patch that hold grid rows
  const int plo = dlt_imax(4 * rg, G.WR - G.r0), phi = dlt_imin(4 * rg + 3 + 2 * G.WR, G.TR - 1 - G.r0 + G.WR);
  const bool patch_ok = (G.r0 + 4 * rg < G.TR) && (c_p < G.TC) && plo <= phi;
  w.ch_lo = patch_ok ? plo >> 2 : 1;
  w.ch_hi = patch_ok ? phi >> 2 : 0;
  return w;
}

// visibility of the streamed token (halo row covered by row_vis, window column 4 cg + i) from the lane's own token
DLT_DEV bool swa2_visible(const Swa2Win& W, bool row_vis, int cg, int i, int ncg) {
  return row_vis & (cg < ncg) & ((unsigned)(4 * cg + i - W.clo) <= (unsigned)W.cspan);
}

// One copy instruction as the hardware sees it: 64 lanes x 16 (or 4) bytes from `base + voff` (base wave-uniform)
// to the LDS address `lds` + 16 (4) lane.  It is issued from inline assembly on purpose: the compiler models the
// instruction as a flat access that may touch LDS, and while one is in flight it turns every wait for an LDS read into
// a wait for ALL outstanding LDS reads (lgkmcnt(0)) and for all outstanding copies (vmcnt(0)), which serialises the
// operand read-ahead of the loops that overlap copies with products.  Hidden from its counters, the waits for operand
// reads are exact again; the waits for the copies themselves are explicit (swa2_wait_copies).  M0 (the LDS address of a
// copy) is a reserved register that cannot be named as an operand or a clobber: the statement saves it, sets it, issues
// the copy (which reads M0 at issue) and puts the saved value back, so whatever the compiler itself keeps in M0 (dynamic
// indexing of register arrays, its own LDS-DMA builtin, messages) survives a copy.
DLT_DEV void dlt_copy16_to_lds(const char* base, uint32_t voff, char* lds) {
  const uint32_t m = (uint32_t)(uintptr_t)(DLT_LDS char*)lds;
  uint32_t saved;
  asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %1\n\ts_mov_b32 m0, %0"
               : "=&s"(saved) : "s"(base), "v"(voff), "s"(m) : "memory");
}
DLT_DEV void dlt_copy4_to_lds(const char* base, uint32_t voff, char* lds) {
  const uint32_t m = (uint32_t)(uintptr_t)(DLT_LDS char*)lds;
  uint32_t saved;
  asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %3\n\ts_nop 0\n\tglobal_load_lds_dword %2, %1\n\ts_mov_b32 m0, %0"
               : "=&s"(saved) : "s"(base), "v"(voff), "s"(m) : "memory");
}

// ---- asynchronous staging -------------------------------------------------------------------------------
// Wave w copies halo row (w & 3) of tensor (w >> 2) of every chunk in NI instructions of 64 lanes; instruction i,
// lane l writes LDS slot 64 i + l of the row = physical piece l % PIECES of halo column TPI i + l / PIECES, and
// therefore fetches the logical piece (l % PIECES) ^ (SWZ (token & 7)) of that token.  Lanes past the last halo
// column of the last instruction stay idle.
template <typename C>
struct Swa2Stage {
  uint32_t off[C::NI];   // byte offset of the lane's piece inside a grid row of the tensor, per instruction
  bool last_on;          // the lane takes part in the last instruction
};

template <typename C>
DLT_DEV void swa2_stage_init(Swa2Stage<C>& st, const Swa2Geom& G, int wave, int lane, int sn2) {
#pragma unroll
  for (int i = 0; i < C::NI; i++) {
    const int hc = C::TPI * i + lane / C::PIECES;
    const int tok = (wave & 3) * C::HCW + hc;
    const int cc = dlt_imax(0, dlt_imin(G.c0 - G.WC + hc, G.TC - 1));   // clamped: positions outside the grid are masked
    st.off[i] = (uint32_t)(cc * sn2 + 16 * ((lane % C::PIECES) ^ (C::SWZ * (tok & 7))));
  }
  st.last_on = C::TPI * (C::NI - 1) + lane / C::PIECES < C::HCW;
}

// one of the NI copy instructions of a halo row (to be spread between the products of a chunk: issued together they
// fill the address queue of the memory pipe and stall the wave in front of its first product)
template <typename C, int I>
DLT_DEV void swa2_issue_one(const Swa2Stage<C>& st, const char* row, char* dst) {
  if constexpr (I < C::NI) {
    if (I + 1 < C::NI || C::HCW % C::TPI == 0 || st.last_on)
      dlt_copy16_to_lds(row, st.off[I], dst + 1024 * I);
  }
}
DLT_DEV const char* swa2_issue_row(const Swa2Geom& G, int ch, const char* base, uint32_t rowstride, int wave) {
  const int r = dlt_imax(0, dlt_imin(G.r0 - G.WR + 4 * ch + (wave & 3), G.TR - 1));
  return base + (uint32_t)r * rowstride;   // wave-uniform
}
template <typename C>
DLT_DEV char* swa2_issue_dst(char* buf, int wave) { return buf + (wave >> 2) * C::REGION + (wave & 3) * (C::HCW * C::ROW); }

// copy halo row (wave & 3) of chunk `ch` of the wave's tensor into its place in `buf`
template <typename C>
DLT_DEV void swa2_issue(const Swa2Stage<C>& st, const Swa2Geom& G, int ch, const char* base, uint32_t rowstride, char* buf, int wave) {
  const char* row = swa2_issue_row(G, ch, base, rowstride, wave);
  char* dst = swa2_issue_dst<C>(buf, wave);
  swa2_for<0, C::NI>([&](auto ic) { swa2_issue_one<C, decltype(ic)::value>(st, row, dst); });
}

// every copy this wave issued has landed in LDS (the workgroup barrier that follows makes all of them visible)
DLT_DEV void swa2_wait_copies() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// Groups of instructions in issue order for the scheduler: one matrix instruction, then `nv` vector instructions that
// do not depend on it.  A wave issues in order: vector work placed behind a run of matrix instructions waits for the
// matrix pipe instead of using the issue slots that the pipe leaves free (a matrix instruction holds the pipe for 16
// cycles and the issue port for 8).
#define SWA2_MIX(nm, nv)                                   \
  _Pragma("unroll") for (int i_ = 0; i_ < (nm); i_++) {    \
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);     \
    __builtin_amdgcn_sched_group_barrier(0x002, (nv), 0);  \
  }

// ---- operand reads -----------------------------------------------------------------------------------------
// Lane constants of a wave whose window starts at halo column 4 pc.
template <typename C>
struct Swa2Lane {
  int a[C::KC];    // A operand (token = MFMA row, head dim along k): byte offset of k-piece c of the lane's token row for an
                   // even column group (odd groups: a[c ^ (KC / 2)])
  int tr[C::VB];   // transposing read (head dim = MFMA row, tokens along k): byte offset for dims 16 d .. 16 d + 15
};

template <typename C>
DLT_DEV void swa2_lane_init(Swa2Lane<C>& L, int pc, int n, int g) {
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

// A-operand pieces of the 16 tokens at column group CG of a chunk region: k[c] = head dims 32 c + 8 g .. + 7
template <typename C, int CG>
DLT_DEV void swa2_read_a(Swa2Lds region, const Swa2Lane<C>& L, u32x4 (&k)[C::KC]) {
#pragma unroll
  for (int c = 0; c < C::KC; c++) k[c] = swa2_lds16(region + 4 * C::ROW * CG + L.a[(CG & 1) ? (c ^ (C::KC / 2)) : c]);
}

// A operands with tokens along k for the 32 tokens (4 halo rows x 8 columns) at column groups 2 KB, 2 KB + 1 of a chunk
// region: v[i] has head dims 16 (D0 + i) .. + 15 as its rows
template <typename C, int KB, int D0, int ND>
DLT_DEV void swa2_read_tr(Swa2Lds region, const Swa2Lane<C>& L, u32x4 (&v)[ND]) {
#pragma unroll
  for (int i = 0; i < ND; i++) {
    const int d = D0 + i;
    const u32x2 lo = swa2_lds_tr(region + 8 * C::ROW * KB + L.tr[d]);
    const u32x2 hi = swa2_lds_tr(region + 8 * C::ROW * KB + 4 * C::ROW + L.tr[d ^ (C::VB / 2)]);
    v[i].x = lo.x; v[i].y = lo.y; v[i].z = hi.x; v[i].w = hi.y;
  }
}

// own-token fragments in B-operand layout: lane (n, g) holds head dims 32 c + 8 g .. + 7 of token n
template <int KC>
DLT_DEV void swa2_own_frags(u32x4 (&f)[KC], const char* base, int sn2, int tok, int g) {
  const char* p = base + ((uint32_t)((tok >= 0 ? tok : 0) * sn2) + 16 * g);
#pragma unroll
  for (int c = 0; c < KC; c++) f[c] = *reinterpret_cast<const u32x4*>(p + 64 * c);
}

// ---- store epilogue: accumulators in C layout (lane (n, g): dims 16 d + 4 g .. + 3 of own token n, times `mul`) -> a
// wave-private LDS tile [16 tokens][2 D bytes] (pieces swizzled with the token index) -> 16-byte pieces -> HBM rows
template <typename C, typename TIO, typename CT>
DLT_DEV void swa2_store_own(char* sW, const f32x4 (&acc)[C::VB], float mul, TIO* base, int64_t sn, const Swa2Geom& G, int r_p, int c_p,
                            int lane) {
  const int n = lane & 15, g = lane >> 4;
#pragma unroll
  for (int d = 0; d < C::VB; d++) {
    u32x2 w;
    w.x = pack2<CT>(acc[d][0] * mul, acc[d][1] * mul);
    w.y = pack2<CT>(acc[d][2] * mul, acc[d][3] * mul);
    *reinterpret_cast<u32x2*>(sW + n * C::ROW + 16 * ((2 * d + (g >> 1)) ^ (n & 7)) + 8 * (g & 1)) = w;
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  constexpr int RPI = 64 / C::PIECES;   // tile rows per pass of the wave
  const int c = lane % C::PIECES;
#pragma unroll
  for (int it = 0; it < 16 / RPI; it++) {
    const int row = lane / C::PIECES + RPI * it;
    const u32x4 v = lds_read16(sW + row * C::ROW + 16 * (c ^ (row & 7)));
    const int r = r_p + (row >> 2), col = c_p + (row & 3);
    if (r < G.TR && col < G.TC) *reinterpret_cast<u32x4*>(base + (int64_t)(r * G.TC + col) * sn + 8 * c) = v;
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
}
