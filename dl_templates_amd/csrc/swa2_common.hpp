// Streaming token-grid kernels for head dim 128 (b_size == 1, windows up to 21 columns, any number of rows):
// shared geometry, asynchronous staging and swizzled operand reads.
//
// A workgroup of 8 waves owns a band of 8 grid rows x 16 grid columns; wave w owns the 4x4 patch at rows
// 4 (w >> 2), columns 4 (w & 3).  The tokens of the other side that any own token can see (8 + 2 WR halo rows x 36
// halo columns) stream through LDS in chunks of 4 halo rows.  A chunk is copied HBM -> LDS by the DMA path of the
// vector memory unit (16 bytes per lane, no staging registers: at head dim 128 those were a third of the register
// file) into one of two buffers while the other one is consumed, so a chunk costs one workgroup barrier, every
// halo row is fetched once per 8 own rows, and the registers go to operand read-ahead instead.
//
// LDS rows are 2 D = 256 bytes with no padding; the 16-byte piece `ch` of token row t is stored at piece
// ch ^ (2 (t & 7)): operand reads of a wave (16 lanes x 16 bytes, or 32 lanes x 8 bytes for the transposing read)
// then fall on distinct banks, and so do the 64 x 16 bytes a copy instruction writes.
#pragma once
#include "swa1_common.hpp"

constexpr int SWA2_HCW = 36;                 // staged halo columns: 16 own + 2 * 10
constexpr int SWA2_TOK = 4 * SWA2_HCW;       // tokens of a chunk
constexpr int SWA2_THREADS = 512;
constexpr int SWA2_ROW = 256;                // bytes of a token row (head dim 128, 2-byte elements)
constexpr int SWA2_REGION = SWA2_TOK * SWA2_ROW;   // one tensor of a chunk
constexpr int SWA2_BUF = 2 * SWA2_REGION;          // both tensors of a chunk
constexpr int SWA2_LDS = 2 * SWA2_BUF;             // two chunk buffers

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

// ---- asynchronous staging -------------------------------------------------------------------------------
// Wave w copies halo row (w & 3) of tensor (w >> 2) of every chunk: 36 tokens x 16 pieces = 9 instructions of 64
// lanes; instruction i, lane l writes LDS slot 64 i + l of the row = physical piece l & 15 of halo column
// 4 i + (l >> 4), and therefore fetches the logical piece (l & 15) ^ (2 (token & 7)) of that token.
struct Swa2Stage {
  uint32_t off[9];   // byte offset of the lane's piece inside a grid row of the tensor, per instruction
};

DLT_DEV void swa2_stage_init(Swa2Stage& st, const Swa2Geom& G, int wave, int lane, int sn2) {
#pragma unroll
  for (int i = 0; i < 9; i++) {
    const int hc = 4 * i + (lane >> 4);
    const int tok = (wave & 3) * SWA2_HCW + hc;
    const int cc = dlt_imax(0, dlt_imin(G.c0 - G.WC + hc, G.TC - 1));   // clamped: positions outside the grid are masked
    st.off[i] = (uint32_t)(cc * sn2 + 16 * ((lane & 15) ^ (2 * (tok & 7))));
  }
}

// copy halo row (wave & 3) of chunk `ch` of the wave's tensor into its place in `buf`
DLT_DEV void swa2_issue(const Swa2Stage& st, const Swa2Geom& G, int ch, const char* base, uint32_t rowstride, char* buf, int wave) {
  const int r = dlt_imax(0, dlt_imin(G.r0 - G.WR + 4 * ch + (wave & 3), G.TR - 1));
  const char* row = base + (uint32_t)r * rowstride;   // wave-uniform
  char* dst = buf + (wave >> 2) * SWA2_REGION + (wave & 3) * (SWA2_HCW * SWA2_ROW);
#pragma unroll
  for (int i = 0; i < 9; i++)
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(row + st.off[i]),
                                     (DLT_LDS void*)(dst + 1024 * i), 16, 0, 0);
}

// one of the nine copy instructions of swa2_issue (to be spread between the products of a chunk: issued together they
// fill the address queue of the memory pipe and stall the wave in front of its first product)
template <int I>
DLT_DEV void swa2_issue_one(const Swa2Stage& st, const char* row, char* dst) {
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(row + st.off[I]), (DLT_LDS void*)(dst + 1024 * I), 16, 0,
                                   0);
}
DLT_DEV const char* swa2_issue_row(const Swa2Geom& G, int ch, const char* base, uint32_t rowstride, int wave) {
  const int r = dlt_imax(0, dlt_imin(G.r0 - G.WR + 4 * ch + (wave & 3), G.TR - 1));
  return base + (uint32_t)r * rowstride;
}
DLT_DEV char* swa2_issue_dst(char* buf, int wave) { return buf + (wave >> 2) * SWA2_REGION + (wave & 3) * (SWA2_HCW * SWA2_ROW); }

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
struct Swa2Lane {
  int a[4];    // A operand (token = MFMA row, head dim along k): byte offset of k-piece c of the lane's token row for an
               // even column group (odd groups: a[c ^ 2])
  int tr[8];   // transposing read (head dim = MFMA row, tokens along k): byte offset for dims 16 d .. 16 d + 15
};

DLT_DEV void swa2_lane_init(Swa2Lane& L, int pc, int n, int g) {
  // A operand: lane (n, g) reads token (halo row n >> 2, column 4 (pc + cg) + (n & 3)) of a chunk, pieces 4 c + g;
  // token & 7 = (n & 3) | 4 ((n >> 2) + pc + cg & 1)  (36 = 4 mod 8)
  const int tok = (n >> 2) * SWA2_HCW + 4 * pc + (n & 3);
  const int par = ((n >> 2) + pc) & 1;
#pragma unroll
  for (int c = 0; c < 4; c++) L.a[c] = tok * SWA2_ROW + 16 * ((4 * c + g) ^ (2 * (n & 3)) ^ (8 * par));
  // transposing read: lane (n, g) addresses token (halo row g, column 4 (pc + cg0) + (n >> 2)), cg0 even, 8 bytes at dim
  // 16 d + 4 (n & 3): piece 2 d + ((n & 3) >> 1); token & 7 = (n >> 2) | 4 ((g + pc) & 1)
  const int tok2 = g * SWA2_HCW + 4 * pc + (n >> 2);
  const int sw = 2 * ((n >> 2) | (4 * ((g + pc) & 1)));
#pragma unroll
  for (int d = 0; d < 8; d++) L.tr[d] = tok2 * SWA2_ROW + 16 * ((2 * d + ((n & 3) >> 1)) ^ sw) + 8 * (n & 1);
}

// A-operand pieces of the 16 tokens at column group CG of a chunk region: k[c] = head dims 32 c + 8 g .. + 7
template <int CG>
DLT_DEV void swa2_read_a(Swa2Lds region, const Swa2Lane& L, u32x4 (&k)[4]) {
#pragma unroll
  for (int c = 0; c < 4; c++) k[c] = swa2_lds16(region + 1024 * CG + L.a[(CG & 1) ? (c ^ 2) : c]);
}

// A operands with tokens along k for the 32 tokens (4 halo rows x 8 columns) at column groups 2 KB, 2 KB + 1 of a chunk
// region: v[i] has head dims 16 (D0 + i) .. + 15 as its rows
template <int KB, int D0, int ND>
DLT_DEV void swa2_read_tr(Swa2Lds region, const Swa2Lane& L, u32x4 (&v)[ND]) {
#pragma unroll
  for (int i = 0; i < ND; i++) {
    const int d = D0 + i;
    const u32x2 lo = swa2_lds_tr(region + 2048 * KB + L.tr[d]);
    const u32x2 hi = swa2_lds_tr(region + 2048 * KB + 1024 + L.tr[d ^ 4]);
    v[i].x = lo.x; v[i].y = lo.y; v[i].z = hi.x; v[i].w = hi.y;
  }
}

// ---- store epilogue: accumulators in C layout (lane (n, g): dims 16 d + 4 g .. + 3 of own token n, times `mul`) -> a
// wave-private LDS tile [16 tokens][256 bytes] (pieces swizzled with the token index) -> 16-byte pieces -> HBM rows
template <typename TIO, typename CT>
DLT_DEV void swa2_store_own(char* sW, const f32x4 (&acc)[8], float mul, TIO* base, int64_t sn, const Swa2Geom& G, int r_p, int c_p,
                            int lane) {
  const int n = lane & 15, g = lane >> 4;
#pragma unroll
  for (int d = 0; d < 8; d++) {
    u32x2 w;
    w.x = pack2<CT>(acc[d][0] * mul, acc[d][1] * mul);
    w.y = pack2<CT>(acc[d][2] * mul, acc[d][3] * mul);
    *reinterpret_cast<u32x2*>(sW + n * 256 + 16 * ((2 * d + (g >> 1)) ^ (n & 7)) + 8 * (g & 1)) = w;
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  const int c = lane & 15;
#pragma unroll
  for (int it = 0; it < 4; it++) {
    const int row = (lane >> 4) + 4 * it;
    const u32x4 v = lds_read16(sW + row * 256 + 16 * (c ^ (row & 7)));
    const int r = r_p + (row >> 2), col = c_p + (row & 3);
    if (r < G.TR && col < G.TC) *reinterpret_cast<u32x4*>(base + (int64_t)(r * G.TC + col) * sn + 8 * c) = v;
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
}
