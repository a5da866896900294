// Token-grid (b_size == 1) sliding-window kernels: shared geometry and halo staging.
//
// A workgroup of 4 waves owns a band of 4 grid rows x 16 grid columns; wave w owns the 4x4
// patch at columns 4w..4w+3 (lane n <-> query (n >> 2, n & 3) of the patch).  The tokens of the
// other side that any owned token can see form the halo: (4 + 2 WR) rows x (16 + 2 WC)
// columns, of which each wave uses a window of 4 * NCG columns starting at halo column 4w.
// The halo is streamed through LDS in chunks of CR rows (a multiple of 8).  A wave walks its
// window in blocks of 8 rows x 4 columns (32 tokens): two MFMA row blocks of 4x4 tokens.  In
// the 16x16 result layout lane group g then holds halo row g of each 4x4 block and element i
// holds column i, so the window test splits into a per-row and a per-column part.
#pragma once
#include "attn_common.hpp"

struct Swa1Plan {
  int32_t HRP;      // halo rows, padded to a multiple of 8 (chunks hold 8 halo rows)
  int32_t ncg;      // 4-column groups per wave window that can hold a visible token
  int32_t nblk_r, nblk_c;
  int32_t lds_bytes;
};

// halo columns staged per row for a window class of NCGMAX column groups: the kernels are
// compiled for the class, narrower windows stage (and mask) the surplus columns
constexpr int swa1_hcw(int ncgmax) { return 12 + 4 * ncgmax; }

// 64-byte items (4 chunks of 8 dims of one token) a thread stages per 8-row chunk of one tensor
constexpr int swa1_items(int d, int hcw) { return (8 * hcw * (d / 32) + 255) / 256; }

// One thread's share of a halo chunk in flight between HBM and LDS.  An item is 64 contiguous
// bytes of one token; rotary partners (8 or 16 dims apart) live in the same item, so the
// rotation needs no second load.
template <int NI>
struct StageRegs {
  u32x4 v[NI][4];
  int32_t id[NI];  // packed rotary index of the token (-1: no rotation / outside the grid)
};

struct Swa1Geom {
  int r0, c0;      // first grid row / column of the workgroup's band
  int TR, TC, WR, WC;
};

// Issue the global loads of halo rows [cr0, cr0 + 8) into registers (zeros outside the grid).
// Offsets are 32-bit element offsets from `base` (the host checks that a [N, D] slab fits).
template <typename TIO, int D, int HCW>
DLT_DEV void swa1_issue(StageRegs<swa1_items(D, HCW)>& sr, const TIO* base, int sn, int dact, const Swa1Geom& G,
                        int cr0, const int32_t* rope_idx, int tid) {
  constexpr int QUADS = D / 32;
  constexpr int TOTAL = 8 * HCW * QUADS;
  const int rbase = G.r0 - G.WR + cr0, cbase = G.c0 - G.WC;
#pragma unroll
  for (int it = 0; it < swa1_items(D, HCW); it++) {
    const int idx = tid + 256 * it;
#pragma unroll
    for (int j = 0; j < 4; j++) sr.v[it][j] = u32x4{0u, 0u, 0u, 0u};
    sr.id[it] = -1;
    if (TOTAL % 256 == 0 || it + 1 < swa1_items(D, HCW) || idx < TOTAL) {
      const int key = idx / QUADS, qd = idx % QUADS;
      const int hr = key / HCW, hc = key - hr * HCW;
      const int r = rbase + hr, c = cbase + hc;
      if ((unsigned)r < (unsigned)G.TR && (unsigned)c < (unsigned)G.TC) {
        const int tok = r * G.TC + c;
        const TIO* p = base + (tok * sn + 32 * qd);
#pragma unroll
        for (int j = 0; j < 4; j++)
          if (32 * qd + 8 * j < dact) sr.v[it][j] = *reinterpret_cast<const u32x4*>(p + 8 * j);
        if (rope_idx != nullptr) sr.id[it] = rope_idx[tok];
      }
    }
  }
}

// Rotate (K / Q side only) and write the staged registers into an LDS chunk.
// pbit: chunk distance between rotary partners (1 or 2).
template <typename CT, int D, int HCW>
DLT_DEV void swa1_commit(StageRegs<swa1_items(D, HCW)>& sr, char* s, int pitch, int pbit, const RopeDev& rope,
                         bool use_rope, int tid) {
  constexpr int QUADS = D / 32;
  constexpr int TOTAL = 8 * HCW * QUADS;
#pragma unroll
  for (int it = 0; it < swa1_items(D, HCW); it++) {
    const int idx = tid + 256 * it;
    if (TOTAL % 256 == 0 || it + 1 < swa1_items(D, HCW) || idx < TOTAL) {
      const int key = idx / QUADS, qd = idx % QUADS;
      if (use_rope && sr.id[it] != -1 && 32 * qd < 4 * rope.R) {
        const int r8 = rope.R >> 3;
#pragma unroll
        for (int pr = 0; pr < 2; pr++) {
          // pbit 1: pairs (0,1), (2,3); pbit 2: pairs (0,2), (1,3)
          const int ja = pbit == 1 ? 2 * pr : pr, jb = ja + pbit;
          const int c0 = 4 * qd + ja;
          if (8 * c0 < 4 * rope.R) {
            const int region = c0 / r8, ci = c0 - region * r8;
            bool rotated;
            const float* tab = rope_table_row(rope, region >> 1, sr.id[it], rotated) + 16 * ci;
            if (rotated) {
              u32x4 lo = pbit == 1 ? (pr == 0 ? sr.v[it][0] : sr.v[it][2]) : (pr == 0 ? sr.v[it][0] : sr.v[it][1]);
              u32x4 hi = pbit == 1 ? (pr == 0 ? sr.v[it][1] : sr.v[it][3]) : (pr == 0 ? sr.v[it][2] : sr.v[it][3]);
              float x0[8], x1[8];
              unpack8<CT>(lo, x0);
              unpack8<CT>(hi, x1);
#pragma unroll
              for (int j = 0; j < 8; j++) {
                const float cs = tab[2 * j], sn = tab[2 * j + 1];
                const float y0 = rope_mix(x0[j], x1[j], cs, sn, true);
                const float y1 = rope_mix(x1[j], x0[j], cs, sn, false);
                x0[j] = y0; x1[j] = y1;
              }
              lo = pack8<CT>(x0);
              hi = pack8<CT>(x1);
              if (pbit == 1) {
                if (pr == 0) { sr.v[it][0] = lo; sr.v[it][1] = hi; } else { sr.v[it][2] = lo; sr.v[it][3] = hi; }
              } else {
                if (pr == 0) { sr.v[it][0] = lo; sr.v[it][2] = hi; } else { sr.v[it][1] = lo; sr.v[it][3] = hi; }
              }
            }
          }
        }
      }
      char* row = s + key * pitch + 64 * qd;
#pragma unroll
      for (int j = 0; j < 4; j++) lds_write16(row + 16 * j, sr.v[it][j]);
    }
  }
}

// A operand for a product that contracts over the 32 tokens of an 8x4 block: dims
// dim0..dim0+15 of the [token][dim] chunk become the operand rows.  `key0` is the LDS token
// index of the block's first row at the wave's column group.
DLT_DEV u32x4 swa1_read_tokens_as_k(const char* tile, int pitch, int hcw, int key0, int dim0, int n, int g) {
  const char* p = tile + (key0 + g * hcw + (n >> 2)) * pitch + (dim0 + 4 * (n & 3)) * 2;
  const u32x2 lo = lds_read_tr16(p);
  const u32x2 hi = lds_read_tr16(p + 4 * hcw * pitch);
  u32x4 r;
  r.x = lo.x; r.y = lo.y; r.z = hi.x; r.w = hi.y;
  return r;
}
