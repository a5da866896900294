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

// LDS row pitch of a staged chunk.  16-byte LDS accesses of a wave are served 16 lanes at a time,
// lanes {0-7, 16-23}, {8-15, 24-31}, ... together (measured with a probe); with 64 banks of 4 bytes
// a pitch of 16 k bytes keeps the reads of such a group on distinct banks iff k = 2 (mod 4):
// 32 bytes of padding for head dims 64 and 128, where 16 bytes make every read a 2-way conflict.
// `wide`: the layout with 32 bytes of padding and the bank-spreading write map (kernels without
// rotation).  At D = 128 the wide window class cannot afford it for both regions within two
// workgroups per CU: its second region keeps 16 bytes (and the dK/dV kernel, which also stages
// lse2 / delta, keeps 16 bytes for both).
constexpr int swa1_pitch(int d, int ncgmax, int region, bool wide, bool kv = false) {
  return d * 2 + ((!wide || (d == 128 && ncgmax > 4 && (region == 1 || kv))) ? 16 : 32);
}

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
constexpr int swa1_items(int d, int hcw, int cr = 8) { return (cr * hcw * (d / 32) + 255) / 256; }
// Tail staging: when the 64-byte items of a chunk do not divide evenly over the 256 threads and the
// remainder is at most 256 16-byte chunks, the remainder is staged one 16-byte chunk per thread
// instead of one more (mostly idle) 64-byte item: 4 staging registers per tensor instead of 16.
// Only without rotation (a rotary pair must sit in one thread).
constexpr bool swa1_use_tail(int d, int hcw, int cr) {
  return (cr * hcw * (d / 32)) / 256 >= 1 && (cr * hcw * (d / 32)) % 256 != 0 && ((cr * hcw * (d / 32)) % 256) * 4 <= 256;
}
constexpr int swa1_items_t(int d, int hcw, int cr, bool tail) { return tail ? (cr * hcw * (d / 32)) / 256 : swa1_items(d, hcw, cr); }

struct Swa1Geom {
  int r0, c0;      // first grid row / column of the workgroup's band
  int TR, TC, WR, WC;
};

// Chunk-invariant part of a thread's staging work.  Item `it` of a thread is the 64-byte piece
// `qd` of halo token (hr[it], column cc[it]); halo positions outside the grid are CLAMPED onto
// the nearest grid token instead of being zero-filled: such positions are always masked by the
// -inf window bias, so their (finite) values never reach a result, and the loads need neither
// a branch nor a zero fill.
//
// A token row of D dims is staged by D / 32 neighbouring threads, four 16-byte chunks each.
// Plain mapping: thread qd takes chunks 4 qd .. 4 qd + 3.  Balanced mapping (`bal_r8` > 0, used
// when the rotary encoding covers exactly half of the head dim, R = D / 8 = 8 bal_r8): there are
// as many rotary pairs of chunks as threads, so thread qd takes pair qd (chunks x0, x0 + bal_r8)
// plus two of the unrotated chunks, and every lane rotates one pair instead of half of the
// lanes rotating two.
template <int NI>
struct StagePlan {
  int hr[NI];    // halo row inside the chunk (0..7)
  int cc[NI];    // grid column, clamped
  int lkey[NI];  // token row inside the LDS chunk, -1: no such item
  int coff[4];   // byte offsets of the thread's four 16-byte chunks inside a token row
  int t_hr, t_cc;  // tail chunk: halo row and clamped grid column of its token
  int t_key;       // tail chunk: token row inside the LDS chunk, -1: this thread has none
  int t_off;       // tail chunk: byte offset inside the token row
  int jx16[2];   // wide layout, per region: register j holds chunk j ^ (jx16 / 16) of the piece (0: in order)
  int bal;       // balanced mapping: chunks 0 and 1 are a rotary pair
  int axis;      // balanced: 0 row angle, 1 column angle
  int tab_off;   // balanced: float offset of the pair's (cos, sin) values inside a table row
};

// WIDE: thread -> token map with lane bits 3 and 4 swapped, and for a region of pitch 2 D + 32 the
// chunk order of a piece flipped on every other thread (D = 64) or token pair (D = 128): the 16 writes
// of a lane group then land on 16 distinct bank quads (PA / PB: the pitches of the two regions).
template <int D, int HCW, int CR, bool BAL, bool TAIL = false, bool WIDE = false, int PA = 0, int PB = 0>
DLT_DEV void swa1_plan_init(StagePlan<swa1_items_t(D, HCW, CR, TAIL)>& sp, const Swa1Geom& G, int tid_, int bal_r8) {
  constexpr int QUADS = D / 32;
  const int tid = WIDE ? ((tid_ & ~0x18) | ((tid_ & 8) << 1) | ((tid_ & 16) >> 1)) : tid_;
  const int qd = tid % QUADS, key0 = tid / QUADS;
  {
    const int jx = WIDE ? 16 * (QUADS == 2 ? (qd & 1) : ((key0 >> 1) & 1)) : 0;
    sp.jx16[0] = PA == 2 * D + 32 ? jx : 0;
    sp.jx16[1] = PB == 2 * D + 32 ? jx : 0;
  }
  sp.t_hr = 0; sp.t_cc = dlt_imax(0, dlt_imin(G.c0 - G.WC, G.TC - 1)); sp.t_key = -1; sp.t_off = 0;
  if (TAIL) {
    constexpr int FULL = (CR * HCW * QUADS) / 256, REM = (CR * HCW * QUADS) % 256;
    if (tid_ < REM * 4) {
      const int ti = FULL * 256 + (tid_ >> 2);
      const int key = ti / QUADS;
      sp.t_off = 64 * (ti % QUADS) + 16 * (tid_ & 3);
      sp.t_hr = key / HCW;
      sp.t_cc = dlt_imax(0, dlt_imin(G.c0 - G.WC + (key - sp.t_hr * HCW), G.TC - 1));
      sp.t_key = key;
    }
  }
  sp.bal = BAL;
  if (BAL) {
    const int region2 = qd / bal_r8, ci = qd - region2 * bal_r8;
    const int x0 = 2 * region2 * bal_r8 + ci;
    sp.coff[0] = 16 * x0;
    sp.coff[1] = 16 * (x0 + bal_r8);
    sp.coff[2] = 16 * (4 * bal_r8 + 2 * qd);
    sp.coff[3] = sp.coff[2] + 16;
    sp.axis = region2;
    sp.tab_off = 16 * ci;
  } else {
#pragma unroll
    for (int j = 0; j < 4; j++) sp.coff[j] = 64 * qd + 16 * j;
    sp.axis = 0;
    sp.tab_off = 0;
  }
#pragma unroll
  for (int it = 0; it < swa1_items_t(D, HCW, CR, TAIL); it++) {
    const int key = key0 + it * (256 / QUADS);
    const bool live = key < CR * HCW;
    const int k = live ? key : 0;
    const int hr = k / HCW, hc = k - hr * HCW;
    sp.hr[it] = hr;
    sp.cc[it] = dlt_imax(0, dlt_imin(G.c0 - G.WC + hc, G.TC - 1));
    sp.lkey[it] = live ? k : -1;
  }
}

// One thread's share of a halo chunk in flight between HBM and LDS (rotary partners, 8 or 16
// dims apart, live in the same 64-byte item, so the rotation needs no second load).
template <int NI>
struct StageRegs {
  u32x4 v[NI][4];
  int32_t id[NI];  // packed rotary index of the token
  u32x4 tv;        // tail chunk
};

template <int NI>
DLT_DEV void swa1_regs_zero(StageRegs<NI>& sr) {
#pragma unroll
  for (int it = 0; it < NI; it++) {
#pragma unroll
    for (int j = 0; j < 4; j++) sr.v[it][j] = u32x4{0u, 0u, 0u, 0u};
    sr.id[it] = -1;
  }
  sr.tv = u32x4{0u, 0u, 0u, 0u};
}

// Issue the global loads of halo rows [cr0, cr0 + 8) into registers.  `sn2` is the token stride
// in BYTES; offsets are 32-bit (the host checks that a [N, D] slab stays below 2 GiB).  `on`:
// the thread's 64-byte piece lies below the actual head dim (pieces above it stay zero).
template <int NI, bool BAL, bool TAIL = false, int REG = 0>
DLT_DEV void swa1_issue(StageRegs<NI>& sr, const StagePlan<NI>& sp, bool on, const void* base, int sn2, const Swa1Geom& G,
                        int cr0, const int32_t* rope_idx, bool tail_on = false) {
  const int rbase = G.r0 - G.WR + cr0;
  if (TAIL) {
    // always a valid address (threads without a tail chunk re-read a token of the chunk)
    const int r = dlt_imax(0, dlt_imin(rbase + sp.t_hr, G.TR - 1));
    const char* p = reinterpret_cast<const char*>(base) + (uint32_t)((r * G.TC + sp.t_cc) * sn2 + (tail_on ? sp.t_off : 0));
    sr.tv = *reinterpret_cast<const u32x4*>(p);
  }
#pragma unroll
  for (int it = 0; it < NI; it++) {
    const int r = dlt_imax(0, dlt_imin(rbase + sp.hr[it], G.TR - 1));
    const int tok = r * G.TC + sp.cc[it];
    if (on) {
      const char* p = reinterpret_cast<const char*>(base) + (uint32_t)(tok * sn2);
#pragma unroll
      for (int j = 0; j < 4; j++) sr.v[it][j] = *reinterpret_cast<const u32x4*>(p + (BAL ? sp.coff[j] : sp.coff[0] + ((16 * j) ^ sp.jx16[REG])));
    }
    if (rope_idx != nullptr) sr.id[it] = rope_idx[tok];
  }
}

// Table values of the rotary pair each staged item of the balanced map needs, fetched ahead of
// the commit: the load depends on the token index that arrived with the chunk, and issuing it before
// the workgroup barrier lets its latency overlap the wait for the other waves.
template <int NI>
struct TabRegs {
  f32x4 t[NI][4];   // (cos, sin) of the 8 pair elements
  bool rot[NI];     // the token has this axis rotated
};

template <int NI>
DLT_DEV void swa1_tab_issue(TabRegs<NI>& tr, const StageRegs<NI>& sr, const StagePlan<NI>& sp, const RopeDev& rope) {
#pragma unroll
  for (int it = 0; it < NI; it++) {
    bool rotated;
    const float* tab = rope_table_row(rope, sp.axis, sr.id[it], rotated) + sp.tab_off;
    tr.rot[it] = rotated;
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const float* tj = tab + 4 * j;
      tr.t[it][j] = f32x4{tj[0], tj[1], tj[2], tj[3]};
    }
  }
}

// Rotate (K / Q side only) and write the staged registers into an LDS chunk.
// ROT: 0 no rotation, 1 rotation with the plain chunk mapping, 2 rotation of the balanced
// mapping's pair (chunks 0 and 1).  pbit: chunk distance between rotary partners (1 or 2).
template <typename CT, int NI, bool BAL, int ROT, bool TAIL, int REG, int PITCH>
DLT_DEV void swa1_commit(StageRegs<NI>& sr, const StagePlan<NI>& sp, char* s, int pbit, const RopeDev& rope, bool use_rope,
                         const TabRegs<NI>* tr = nullptr, bool tail_on = false) {
  static_assert(ROT != 2 || BAL, "pair rotation needs the balanced mapping");
  static_assert(!TAIL || ROT == 0, "tail staging splits rotary pairs");
  if (TAIL) {
    pin_loaded(sr.tv);
    if (sp.t_key >= 0) lds_write16(s + sp.t_key * PITCH + sp.t_off, tail_on ? sr.tv : u32x4{0u, 0u, 0u, 0u});
  }
  // wait for the staged loads HERE, on every path: a wait placed inside the per-thread `if` below
  // would be skipped when no lane has an item, and the compiler would then treat the loads as
  // possibly pending in the next iteration (a full wait in front of every new load)
#pragma unroll
  for (int it = 0; it < NI; it++) {
#pragma unroll
    for (int j = 0; j < 4; j++) pin_loaded(sr.v[it][j]);
    if (ROT != 0) asm volatile("" ::"v"(sr.id[it]));
    if (ROT == 2) {
#pragma unroll
      for (int j = 0; j < 4; j++) asm volatile("" ::"v"(tr->t[it][j]));
    }
  }
#pragma unroll
  for (int it = 0; it < NI; it++) {
    if (sp.lkey[it] < 0) continue;
    if (ROT == 2 && use_rope) {
      if (tr->rot[it]) {
        float x0[8], x1[8];
        unpack8<CT>(sr.v[it][0], x0);
        unpack8<CT>(sr.v[it][1], x1);
#pragma unroll
        for (int j = 0; j < 8; j++) {
          const float cs = tr->t[it][j >> 1][2 * (j & 1)], sn = tr->t[it][j >> 1][2 * (j & 1) + 1];
          const float y0 = rope_mix(x0[j], x1[j], cs, sn, true);
          const float y1 = rope_mix(x1[j], x0[j], cs, sn, false);
          x0[j] = y0; x1[j] = y1;
        }
        sr.v[it][0] = pack8<CT>(x0);
        sr.v[it][1] = pack8<CT>(x1);
      }
    } else if (ROT == 1 && use_rope && sp.coff[0] < 8 * rope.R) {
      const int r8 = rope.R >> 3;
      const int qd4 = sp.coff[0] >> 4;  // first chunk of this piece
#pragma unroll
      for (int pr = 0; pr < 2; pr++) {
        // pbit 1: pairs (0,1), (2,3); pbit 2: pairs (0,2), (1,3)
        const int ja = pbit == 1 ? 2 * pr : pr;
        const int c0 = qd4 + ja;
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
    char* row = s + sp.lkey[it] * PITCH;
#pragma unroll
    for (int j = 0; j < 4; j++) lds_write16(row + (BAL ? sp.coff[j] : sp.coff[0] + ((16 * j) ^ sp.jx16[REG])), sr.v[it][j]);
  }
}

// B-operand fragments of one OWN token (head dim along k) straight from HBM: lane group g
// holds dims 32c + 8g .. +7 of chunk c.  Rotated on the way in when `use_rope`.
template <typename TIO, typename CT, int D>
DLT_DEV void swa1_load_own(u32x4 (&f)[D / 32], const TIO* base, int64_t sn, int dact, int64_t tok, int g,
                           const RopeDev& rope, bool use_rope) {
#pragma unroll
  for (int c = 0; c < D / 32; c++) {
    const int ch = 4 * c + g;
    f[c] = u32x4{0u, 0u, 0u, 0u};
    if (tok >= 0 && 8 * ch < dact) f[c] = *reinterpret_cast<const u32x4*>(base + tok * sn + 8 * ch);
  }
  if (use_rope && tok >= 0) {
    const int32_t id = rope.idx[tok];
#pragma unroll
    for (int c = 0; c < D / 32; c++) {
      const int ch = 4 * c + g;
      const RopeChunk rc = rope_chunk_setup(rope, ch, true);
      if (rc.mode == 1) {
        float self[8], partner[8];
        unpack8<CT>(f[c], self);
        unpack8<CT>(*reinterpret_cast<const u32x4*>(base + tok * sn + 8 * rc.partner_c), partner);
        rope_apply8(rope, rc, ch, id, self, partner, [](int) { return 0.f; });
        f[c] = pack8<CT>(self);
      }
    }
  }
}

// A operand for a product that contracts over the 32 tokens of an 8x4 block: dims
// dim0..dim0+15 of the [token][dim] chunk become the operand rows.  `key0` is the LDS token
// index of the block's first row at the wave's column group.
// `mb_step`: token distance between the two 4x4 halves of the block (4 * hcw: the half below,
// 4: the half to the right).
DLT_DEV u32x4 swa1_read_tokens_as_k(const char* tile, int pitch, int hcw, int key0, int dim0, int n, int g, int mb_step) {
  const char* p = tile + (key0 + g * hcw + (n >> 2)) * pitch + (dim0 + 4 * (n & 3)) * 2;
  const u32x2 lo = lds_read_tr16(p);
  const u32x2 hi = lds_read_tr16(p + mb_step * pitch);
  u32x4 r;
  r.x = lo.x; r.y = lo.y; r.z = hi.x; r.w = hi.y;
  return r;
}

// Epilogue: accumulators in C layout (lane (n, g) holds dims 16 d + 4 g .. +3 of own token n,
// scaled by `mul`) -> wave-private LDS tile [16 tokens][D] of output elements -> 16-byte pieces
// -> HBM rows (element stride 1, 16-byte aligned rows).  A wave reads back only what it wrote
// itself, so no workgroup barrier is involved; LDS operations of one wave execute in order.
// With `use_rope` the rotation selected by rope.inverse is applied to the rounded values, exactly
// as the standalone operator would see them.
template <typename TIO, typename CT, int D>
DLT_DEV void swa1_store_own(char* sW, const f32x4 (&acc)[D / 16], float mul, TIO* base, int64_t sn, int dact,
                            const Swa1Geom& G, int wave, int lane, const RopeDev& rope, bool use_rope) {
  constexpr int PT = D * 2 + 16, CH = D / 8;
  const int n = lane & 15, g = lane >> 4;
#pragma unroll
  for (int d = 0; d < D / 16; d++) {
    u32x2 w;
    w.x = pack2<CT>(acc[d][0] * mul, acc[d][1] * mul);
    w.y = pack2<CT>(acc[d][2] * mul, acc[d][3] * mul);
    *reinterpret_cast<u32x2*>(sW + n * PT + (16 * d + 4 * g) * 2) = w;
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  constexpr int NIT = 16 * CH / 64;
  int tok[NIT];
  bool ok[NIT];
#pragma unroll
  for (int it = 0; it < NIT; it++) {
    const int p = lane + 64 * it;
    const int row = p / CH, c = p % CH;
    const int r = G.r0 + (row >> 2), col = G.c0 + 4 * wave + (row & 3);
    ok[it] = r < G.TR && col < G.TC && 8 * c < dact;
    tok[it] = ok[it] ? r * G.TC + col : 0;
  }
  if (use_rope) {
    // The rotation needs two dependent global loads per piece (token index, then its table row).
    // They are issued in phases over all pieces of the lane, with clamped addresses instead of
    // branches, so that their latencies overlap instead of adding up.
    int32_t id[NIT];
#pragma unroll
    for (int it = 0; it < NIT; it++) id[it] = rope.idx[tok[it]];
    RopeChunk rc[NIT];
    bool rot[NIT];
    f32x4 tv[NIT][4];
#pragma unroll
    for (int it = 0; it < NIT; it++) {
      const int c = (lane + 64 * it) % CH;
      rc[it] = rope_chunk_setup(rope, c, true);
      bool rotated;
      const float* tab = rope_table_row(rope, rc[it].axis, id[it], rotated) + rc[it].tab_off;
      rot[it] = ok[it] && rc[it].mode == 1 && rotated;
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const float* tj = tab + 4 * j;
        tv[it][j] = f32x4{tj[0], tj[1], tj[2], tj[3]};
      }
    }
#pragma unroll
    for (int it = 0; it < NIT; it++) {
      const int p = lane + 64 * it;
      const int row = p / CH, c = p % CH;
      const char* lrow = sW + row * PT;
      u32x4 v = lds_read16(lrow + 16 * c);
      if (rot[it]) {
        float self[8], partner[8];
        unpack8<CT>(v, self);
        unpack8<CT>(lds_read16(lrow + 16 * rc[it].partner_c), partner);
#pragma unroll
        for (int j = 0; j < 8; j++) {
          const float cs = tv[it][j >> 1][2 * (j & 1)], sn_ = tv[it][j >> 1][2 * (j & 1) + 1];
          self[j] = rope_mix_signed(self[j], partner[j], cs, sn_, rope_sign_mask(rc[it].is_x0 != 0, rope.inverse != 0));
        }
        v = pack8<CT>(self);
      }
      if (ok[it]) store_stream16(base + (int64_t)tok[it] * sn + 8 * c, v);
    }
  } else {
#pragma unroll
    for (int it = 0; it < NIT; it++) {
      const int p = lane + 64 * it;
      const int row = p / CH, c = p % CH;
      if (ok[it]) *reinterpret_cast<u32x4*>(base + (int64_t)tok[it] * sn + 8 * c) = lds_read16(sW + row * PT + 16 * c);
    }
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
}
