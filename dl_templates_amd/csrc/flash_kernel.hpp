// Dense, causal and tile-window flash attention forward for gfx950 with separate qk / vo head dims.
//
// MODE 0 dense, 1 causal, 2 and 3 tiled 2D sliding window with b_size a multiple of 16 (3: the tensors are
// images, tokens are addressed through the pixel map of DltTokMap; the regime
// tiled_swa_fwd_large_kernel was written for, src/tiled_swa.py:142-244): a block of 16 own tokens
// lies inside one tile and every 16-token half of a streamed block lies inside one tile, so the
// window test is wave-uniform per half: no per-element mask exists, invisible blocks are skipped.
//
// Replaces _attn_fwd_inner / _attn_fwd (src/flash_attn.py:9-172) and extends the non-causal case
// to Lq != Lk.  CAUSAL (Lq == Lk, query i sees keys j <= i; the STAGE logic of
// src/flash_attn.py:17-24,152-166): a workgroup stops at its last query, a wave skips chunks
// that lie entirely above its queries, and only chunks that cross the diagonal pay for a mask.  A workgroup of 4 waves owns 64*NP consecutive queries of one
// (batch, head); a wave owns NP blocks of 16 queries whose fragments come straight from HBM.
// K and V stream through LDS in chunks of CK keys; the next chunk travels HBM -> registers
// while the current one is consumed.  Per chunk and query block: S^T = K Q^T for all 32-key
// blocks, ONE online-softmax update on the raw scores (p = exp2(fma(s, c, -m c))), then
// O^T += V^T P^T with the K / V^T operand fragments shared by the NP query blocks and the row
// sums produced by one extra MFMA against a row of ones.  Keys past Lk are clamped loads
// masked by an additive -inf bias that only the last chunk applies.
#pragma once
#include <type_traits>
#include "swa1_common.hpp"

struct FlashTailDyn {};   // tag: whether a chunk needs the per-pair bound test is decided at run time

// Streamed chunks in LDS: rows of 2 D + 32 bytes.  16-byte LDS accesses of a wave are served 16
// lanes at a time, lanes {0-7, 16-23}, {8-15, 24-31}, ... together; with 64 banks a pitch of 16 k
// bytes keeps the operand reads (16 rows x 16 bytes, and the transposing 8-byte reads) of such a group
// on distinct banks iff k = 2 (mod 4).  The staging writes (thread -> 16-byte vector t % CH of token
// t / CH) then need the tokens of a lane group a quarter or half of the bank space apart: one pair
// of thread-index bits is swapped per row length.
#ifndef FLASH_PAD
#define FLASH_PAD 32
#endif
template <int CH>
DLT_DEV int flash_stage_tid(int tid) {
  constexpr int A = CH == 4 ? 2 : 4, B = CH == 4 ? 3 : (CH == 8 ? 5 : 6);  // bits to swap
  if (FLASH_PAD != 32) return tid;
  const int x = ((tid >> A) ^ (tid >> B)) & 1;
  return tid ^ ((x << A) | (x << B));
}

#ifndef FLASH_NP_DEF
#define FLASH_NP_DEF 2
#endif
constexpr int FLASH_NP = FLASH_NP_DEF;  // 16-query blocks per wave (forward and dQ)
// Streamed tokens per LDS chunk, per kernel and head-dim class.  128 halves the barriers per key but
// doubles the staging registers and the score registers of a chunk: it pays where the register
// allocation still fits the occupancy target below (measured per class: forward at 64/128 -4 %, dQ at
// 32/32 -8 % in tile mode, dK/dV at 128/128 -8 % in tile mode; elsewhere it spills or changes nothing).
#ifndef FLASH_CK_FWD
#define FLASH_CK_FWD(dk, dv) ((dk) == 64 && (dv) == 128 ? 128 : 64)
#endif
#ifndef FLASH_CK_Q
#define FLASH_CK_Q(dk, dv) ((dk) + (dv) <= 64 ? 128 : 64)
#endif
#ifndef FLASH_CK_KV
#define FLASH_CK_KV(dk, dv) ((dk) + (dv) > 192 ? 128 : 64)
#endif
constexpr int flash_ck_fwd(int dk, int dv) { return FLASH_CK_FWD(dk, dv); }
constexpr int flash_ck_q(int dk, int dv) { return FLASH_CK_Q(dk, dv); }
constexpr int flash_ck_kv(int dk, int dv) { return FLASH_CK_KV(dk, dv); }
// key blocks per wave in the dK/dV kernel: its two accumulator sets only fit twice for small dims
#ifndef FLASH_NP_KV
#define FLASH_NP_KV(dk, dv) ((dk) + (dv) > 192 ? 1 : 2)
#endif
constexpr int flash_np_kv(int dk, int dv) { return FLASH_NP_KV(dk, dv); }
// query blocks per wave in the dQ kernel: one at 128/128 (accumulators, q and dO fragments of two blocks do not fit 256 registers)
constexpr int flash_np_q(int dk, int dv) { return dk + dv > 192 ? 1 : FLASH_NP_DEF; }
// resident workgroups per CU the register allocation aims for (spill-free at these settings)
constexpr int flash_occ_fwd(int dk, int dv) { return dk + dv <= 64 ? 4 : (dk + dv <= 128 ? 3 : 2); }
constexpr int flash_occ_q(int dk, int dv) { return dk + dv <= 64 ? 4 : (dk + dv <= 128 ? 3 : 2); }
constexpr int flash_occ_kv(int dk, int dv, int mode) {
  return dk + dv <= 64 ? 4 : 2;
}

// One chunk of streamed tokens: first token (index inside the [N, D] slab), its x inside the grid
// row (tile mode) or the sequence, and how many of the CK staged tokens exist.
struct FlashChunk { int tok0, x, nvalid, row; };

// Streamed tokens a workgroup visits.  Dense / causal: [first, len) of the sequence.  Tile mode:
// for every grid row in [rlo, rhi] the x range [X0, X1) that some own token can see, CK at a time.
template <int MODE, int CK>
struct FlashWalk {
  int first, nchunks;
  int len;                    // dense / causal
  int nxc, X0, X1, rlo, XL;   // tile mode
  DLT_DEV void init_seq(int first_, int len_) {
    first = first_; len = len_;
    nchunks = len_ > first_ ? (len_ - first_ + CK - 1) / CK : 0;
    nxc = 1; X0 = X1 = rlo = XL = 0;
  }
  // own tokens: grid row r, x in [x0, x0 + own); `transpose`: the own side are keys
  DLT_DEV void init_tile(const DltGeom& g, int r, int x0, int own, bool transpose) {
    const int XLo = transpose ? g.XLk : g.XLq;
    int rl, rh, xl0, xh0, xl1, xh1;
    const int xa = dlt_imin(x0, XLo - 1), xb = dlt_imin(x0 + own - 1, XLo - 1);
    if (transpose) { dlt_query_range(g, r, xa, rl, rh, xl0, xh0); dlt_query_range(g, r, xb, rl, rh, xl1, xh1); }
    else { dlt_key_range(g, r, xa, rl, rh, xl0, xh0); dlt_key_range(g, r, xb, rl, rh, xl1, xh1); }
    X0 = xl0; X1 = xh1; rlo = rl;
    XL = transpose ? g.XLq : g.XLk;
    nxc = (X1 - X0 + CK - 1) / CK;
    nchunks = (rh - rl + 1) * nxc;
    first = 0; len = 0;
  }
  // the chunk after c (the loops walk the chunks in order: no division per chunk)
  DLT_DEV FlashChunk next(const FlashChunk& c) const {
    FlashChunk n;
    n.x = c.x + CK;
    n.row = c.row;
    if (MODE >= 2) {
      if (n.x >= X1) { n.x = X0; n.row = c.row + 1; }
      n.tok0 = n.row * XL + n.x;
      n.nvalid = dlt_imin(CK, X1 - n.x);
    } else {
      n.tok0 = n.x;
      n.nvalid = dlt_imin(CK, len - n.x);
    }
    return n;
  }
  DLT_DEV FlashChunk at(int i) const {
    FlashChunk c;
    if (MODE >= 2) {
      const int ri = i / nxc;
      c.x = X0 + (i - ri * nxc) * CK;
      c.row = rlo + ri;
      c.tok0 = c.row * XL + c.x;
      c.nvalid = dlt_imin(CK, X1 - c.x);
    } else {
      c.x = first + i * CK;
      c.row = 0;
      c.tok0 = c.x;
      c.nvalid = dlt_imin(CK, len - c.x);
    }
    return c;
  }
};

// Byte offset of streamed token j of chunk c inside its (batch, head) slab: a plain token stride, or
// (IMG) the pixel map applied to the token's slot inside its grid row (two exact divisions; the
// row part is wave-uniform).
template <bool IMG>
struct FlashAddr;
template <>
struct FlashAddr<false> {
  int sn2;  // bytes between tokens
  DLT_DEV uint32_t operator()(const FlashChunk& c, int j) const { return (uint32_t)((c.tok0 + j) * sn2); }
};
template <>
struct FlashAddr<true> {
  int sn2, sy2;  // bytes between pixel columns and between pixel rows
  const DltTokMap* tm;
  DLT_DEV uint32_t operator()(const FlashChunk& c, int j) const {
    uint32_t i, x;
    dlt_slot_pixel(*tm, (uint32_t)(c.x + j), i, x);
    return (uint32_t)(((uint32_t)c.row * tm->bh + i) * (uint32_t)sy2 + x * (uint32_t)sn2);
  }
};
template <bool IMG>
DLT_DEV FlashAddr<IMG> flash_addr(const int64_t (&st)[5], const DltTokMap& tm) {
  if constexpr (IMG) return FlashAddr<true>{(int)st[2] * 2, (int)st[4] * 2, &tm};
  else return FlashAddr<false>{(int)st[2] * 2};
}
// what the tile writers take as the token stride: the plain stride, or (IMG) the pixel map
template <bool IMG>
DLT_DEV auto flash_tok(const int64_t (&st)[5], const DltTokMap& tm) {
  if constexpr (IMG) return tok_addr(st, tm);
  else return st[2];
}
// element offset of own token t (-1: none) for the loaders that take (base, stride, token)
template <bool IMG>
DLT_DEV int64_t flash_own_off(const int64_t (&st)[5], const DltTokMap& tm, int64_t t) {
  if (t < 0) return t;
  return IMG ? tok_addr(st, tm)(t) : t * st[2];
}

// workgroup -> (batch * head, grid row, first own x)
DLT_DEV void flash_block(int lin, int nblk, int TR, int own, int& bh, int& r, int& x0) {
  const int per = nblk * TR;
  bh = lin / per;
  const int rem = lin - bh * per;
  r = rem / nblk;
  const int xb = rem - r * nblk;
  x0 = xb * own;
}

// Causal mask: the work of a block grows with its position, and blocks are handed to free CUs in launch order.  Taken
// (batch, head) by (batch, head), the heavy blocks of the last heads start late and finish alone; here `G` heads at a
// time are interleaved, heaviest blocks of all of them first.  The host sizes G so that the streamed tensors of a group
// fit the 4 MB L2 of an XCD (`flash_causal_group`): larger groups balance better but then stream from the infinity
// cache (measured at N = 4096: d = 64 -6 % with 4 heads, d = 128 -5 % with 2 or 4 and +13 % / +30 % with 8 / 16).
// `rev`: the last block is the heaviest (own = queries), otherwise the first (own = keys).
DLT_DEV void flash_block_causal(int lin, int nblk, int nbh, int G, int own, bool rev, int& bh, int& r, int& x0) {
  const int grp = lin / (G * nblk);
  const int rem = lin - grp * (G * nblk);
  const int gc = dlt_imin(G, nbh - grp * G);   // the last group may hold fewer heads
  const int rank = rem / gc;
  bh = grp * G + (rem - rank * gc);
  r = 0;
  x0 = (rev ? nblk - 1 - rank : rank) * own;
}
inline int flash_causal_group(int L, int dk, int dv) {
  const int64_t per_head = (int64_t)L * (dk + dv) * 2;
  const int64_t g = (4 << 20) / (per_head > 0 ? per_head : 1);
  return (int)(g < 1 ? 1 : (g > 16 ? 16 : g));
}

struct FlashArgs {
  const void *q, *k, *v;
  void* o;
  float* lse;
  int64_t qs[5], ks[5], vs[5], os[5], ls[3];
  DltTokMap tm;
  int32_t B, H, Lq, Lk, dk, dv;
  int32_t nblk;       // workgroups per (batch, head) and grid row
  int32_t causal, causal_group;   // causal_group: see flash_block_causal
  int32_t tile;       // MODE 2: Lq = Lk = tokens per grid row, geometry in g
  DltGeom g;
  int32_t o_vec;
  int32_t lds_bytes;
  float scale_log2;
};

template <typename TIO, int DK, int DV, int NP, int CK, int MODE>
__global__ __launch_bounds__(256, flash_occ_fwd(DK, DV)) void flash_fwd_kernel(const FlashArgs a) {
  typedef typename ComputeOf<TIO>::type CT;
  typedef typename TileOf<TIO>::type TL;
  extern __shared__ __align__(16) char smem[];
  constexpr bool CAUSAL = MODE == 1, TILE = MODE >= 2, IMG = MODE == 3;
  constexpr int PK = DK * 2 + FLASH_PAD, PV = DV * 2 + FLASH_PAD, PO = DV * (int)sizeof(TL) + 16;
  constexpr int KC = DK / 32, VB = DV / 16, NKB = CK / 32;
  constexpr int OWN = 64 * NP;
  constexpr int KCH = DK / 8, VCH = DV / 8;                    // 16-byte vectors per token
  constexpr int NKI = CK * KCH / 256, NVI = CK * VCH / 256;    // vectors per thread and chunk
  static_assert(CK * KCH % 256 == 0 && CK * VCH % 256 == 0, "chunk must split evenly over 256 threads");

  const int tid = threadIdx.x;
  const int lane = tid & 63, n = lane & 15, g = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  char* sK = smem;
  char* sV = smem + CK * PK;

  const int lin = xcd_remap(blockIdx.x, gridDim.x);
  int bh, r_own, x0;
  // causal: the blocks with the most keys to visit are launched first
  if constexpr (CAUSAL) flash_block_causal(lin, a.nblk, a.B * a.H, a.causal_group, OWN, true, bh, r_own, x0);
  else flash_block(lin, a.nblk, TILE ? a.g.TR : 1, OWN, bh, r_own, x0);
  const int wq0 = x0 + wave * 16 * NP;                            // first query of this wave
  const int b = bh / a.H, h = bh - b * a.H;
  const TIO* qb = reinterpret_cast<const TIO*>(a.q) + b * a.qs[0] + h * a.qs[1];
  const char* kb_ = reinterpret_cast<const char*>(reinterpret_cast<const TIO*>(a.k) + b * a.ks[0] + h * a.ks[1]);
  const char* vb_ = reinterpret_cast<const char*>(reinterpret_cast<const TIO*>(a.v) + b * a.vs[0] + h * a.vs[1]);
  TIO* ob = reinterpret_cast<TIO*>(a.o) + b * a.os[0] + h * a.os[1];
  const FlashAddr<IMG> ak = flash_addr<IMG>(a.ks, a.tm), av = flash_addr<IMG>(a.vs, a.tm);
  RopeDev no_rope = RopeDev{};
  const int own_base = TILE ? r_own * a.Lq : 0;                   // token index of own x = 0

  FlashWalk<MODE, CK> W;
  if (TILE) W.init_tile(a.g, r_own, x0, OWN, false);
  else W.init_seq(0, CAUSAL ? dlt_imin(a.Lk, x0 + OWN) : a.Lk);   // causal: keys up to the last own query

  // ---- staging plan (chunk invariant): vector `it` of this thread = chunk ck*/vc* of key kkey/vkey + it * step
  const int tk = flash_stage_tid<KCH>(tid), tv = flash_stage_tid<VCH>(tid);
  const int kc_ = tk % KCH, kkey0 = tk / KCH;
  const int vc_ = tv % VCH, vkey0 = tv / VCH;
  const bool on_k = 8 * kc_ < a.dk, on_v = 8 * vc_ < a.dv;
  u32x4 rk[NKI], rv[NVI];
#pragma unroll
  for (int it = 0; it < NKI; it++) rk[it] = u32x4{0u, 0u, 0u, 0u};
#pragma unroll
  for (int it = 0; it < NVI; it++) rv[it] = u32x4{0u, 0u, 0u, 0u};
  // tokens past the end of a chunk are clamped onto its last token (they are masked or skipped)
  auto issue = [&](const FlashChunk& c) {
#pragma unroll
    for (int it = 0; it < NKI; it++) {
      const uint32_t off = ak(c, dlt_imin(kkey0 + it * (256 / KCH), c.nvalid - 1));
      if (on_k) rk[it] = *reinterpret_cast<const u32x4*>(kb_ + (off + 16 * kc_));
    }
#pragma unroll
    for (int it = 0; it < NVI; it++) {
      const uint32_t off = av(c, dlt_imin(vkey0 + it * (256 / VCH), c.nvalid - 1));
      if (on_v) rv[it] = *reinterpret_cast<const u32x4*>(vb_ + (off + 16 * vc_));
    }
  };
  auto commit = [&]() {
    pin_loaded(rk);
    pin_loaded(rv);
#pragma unroll
    for (int it = 0; it < NKI; it++) lds_write16(sK + (kkey0 + it * (256 / KCH)) * PK + 16 * kc_, rk[it]);
#pragma unroll
    for (int it = 0; it < NVI; it++) lds_write16(sV + (vkey0 + it * (256 / VCH)) * PV + 16 * vc_, rv[it]);
  };
  if (W.nchunks > 0) issue(W.at(0));

  // ---- own queries -> B-operand fragments
  u32x4 qf[NP][KC];
  int64_t tq[NP];
  int klim[NP];           // dense / causal: last key this lane's query may see
  int vlo[NP], vhi[NP];   // tile mode: x interval this query block sees in every visited row (wave-uniform)
#pragma unroll
  for (int p = 0; p < NP; p++) {
    const int xq = wq0 + 16 * p + n;
    tq[p] = xq < a.Lq ? (int64_t)(own_base + xq) : (int64_t)-1;
    klim[p] = CAUSAL ? dlt_imin(xq, a.Lk - 1) : a.Lk - 1;
    vlo[p] = vhi[p] = 0;
    if (TILE && wq0 + 16 * p < a.Lq) {
      int rl, rh;
      dlt_key_range(a.g, r_own, wq0 + 16 * p, rl, rh, vlo[p], vhi[p]);
    }
    swa1_load_own<TIO, CT, DK>(qf[p], qb, 1, a.dk, flash_own_off<IMG>(a.qs, a.tm, tq[p]), g, no_rope, false);
  }

  float m_run[NP];
  f32x4 acc[NP][VB], acc_l[NP];
#pragma unroll
  for (int p = 0; p < NP; p++) {
    m_run[p] = -INFINITY;
    acc_l[p] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int d = 0; d < VB; d++) acc[p][d] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  const float scale = a.scale_log2;
  const unsigned one2 = pack2<CT>(1.f, 1.f);
  const u32x4 ones = n == 0 ? u32x4{one2, one2, one2, one2} : u32x4{0u, 0u, 0u, 0u};

  if (W.nchunks > 0) commit();
  __syncthreads();
  pin_loaded(qf);

  // products and softmax update of the chunk resident in LDS
  // `tail` (dense / causal): some keys of the chunk lie past the end or (causal) above the wave's first query, and every
  // pair is tested.  A compile-time tag: without a causal mask only the last chunk can be short, and the loop body then
  // holds no test at all.
  auto chunk_tail = [&](const FlashChunk& c) {
    return !TILE && (c.nvalid < CK || (CAUSAL && c.x + CK - 1 > wq0));
  };
  auto consume_t = [&](const FlashChunk& c, auto tail_tag) __attribute__((always_inline)) {
    // the tag is true_type / false_type (dense: known per call site) or FlashTailDyn (causal: tested per chunk)
    bool tail;
    if constexpr (std::is_same<decltype(tail_tag), FlashTailDyn>::value) tail = chunk_tail(c);
    else tail = decltype(tail_tag)::value;
    const int k0 = c.x;
    // causal: every key of the chunk lies above every query of this wave (wave-uniform)
    bool live = !CAUSAL || k0 <= wq0 + 16 * NP - 1;
    // tile mode: which 32-key blocks hold a 16-key half that query block p sees (wave-uniform)
    bool bv[NP][NKB], any[NP];
#pragma unroll
    for (int p = 0; p < NP; p++) {
      any[p] = !TILE;
#pragma unroll
      for (int kb = 0; kb < NKB; kb++) {
        bv[p][kb] = !TILE || (k0 + 32 * kb + 32 > vlo[p] && k0 + 32 * kb < vhi[p]);
        any[p] = any[p] || bv[p][kb];
      }
    }
    if (TILE) {
      live = false;
#pragma unroll
      for (int p = 0; p < NP; p++) live = live || any[p];
    }

    u32x4 pb[NP][NKB];
    if (live) {
      float t[NP][NKB][8];
#pragma unroll
      for (int kb = 0; kb < NKB; kb++) {
        u32x4 ka[2][KC];
#pragma unroll
        for (int mb = 0; mb < 2; mb++)
#pragma unroll
          for (int c_ = 0; c_ < KC; c_++) ka[mb][c_] = lds_read16(sK + (32 * kb + 16 * mb + n) * PK + (32 * c_ + 8 * g) * 2);
#pragma unroll
        for (int p = 0; p < NP; p++) {
          if (bv[p][kb]) {
            f32x4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c_ = 0; c_ < KC; c_++) {
              s0 = Mma<CT>::mfma(ka[0][c_], qf[p][c_], s0);
              s1 = Mma<CT>::mfma(ka[1][c_], qf[p][c_], s1);
            }
            // tile mode: a 16-key half outside the window of the block is dropped as a whole
            const bool h0 = !TILE || (k0 + 32 * kb >= vlo[p] && k0 + 32 * kb < vhi[p]);
            const bool h1 = !TILE || (k0 + 32 * kb + 16 >= vlo[p] && k0 + 32 * kb + 16 < vhi[p]);
#pragma unroll
            for (int i = 0; i < 4; i++) { t[p][kb][i] = h0 ? s0[i] : -INFINITY; t[p][kb][4 + i] = h1 ? s1[i] : -INFINITY; }
          } else {
#pragma unroll
            for (int i = 0; i < 8; i++) t[p][kb][i] = -INFINITY;
          }
        }
        if (tail) {
#pragma unroll
          for (int p = 0; p < NP; p++)
#pragma unroll
            for (int i = 0; i < 8; i++) {
              const int key = k0 + 32 * kb + 16 * (i >> 2) + 4 * g + (i & 3);
              t[p][kb][i] = key <= klim[p] ? t[p][kb][i] : -INFINITY;
            }
        }
      }
#pragma unroll
      for (int p = 0; p < NP; p++) {
        if (!any[p]) continue;
        // four independent chains, two new values per instruction (v_max3_f32)
        float mx[4] = {-INFINITY, -INFINITY, -INFINITY, -INFINITY};
#pragma unroll
        for (int kb = 0; kb < NKB; kb++)
#pragma unroll
          for (int i = 0; i < 4; i++) mx[i] = fmaxf(fmaxf(mx[i], t[p][kb][2 * i]), t[p][kb][2 * i + 1]);
        float mloc = wave_max4(fmaxf(fmaxf(mx[0], mx[1]), fmaxf(mx[2], mx[3])));
        // The reference maximum only moves when a score exceeds it by more than 2^8 after scaling: p stays below 2^8,
        // well inside the range of the 16-bit operand and of the fp32 sums, and most chunks skip the rescaling of the
        // accumulators.  o and lse do not depend on which reference was used.
        if (__builtin_amdgcn_ballot_w64((mloc - m_run[p]) * scale > 8.f)) {
          keep_branch();
          const float m_new = fmaxf(m_run[p], mloc);   // finite here
          const float alpha = fast_exp2((m_run[p] - m_new) * scale);
          m_run[p] = m_new;
#pragma unroll
          for (int d = 0; d < VB; d++) acc[p][d] *= alpha;
          acc_l[p] *= alpha;
        }
        const float neg_m2 = m_run[p] == -INFINITY ? 0.f : -m_run[p] * scale;   // -inf: a block that has seen no key yet
#pragma unroll
        for (int kb = 0; kb < NKB; kb++) {
#pragma unroll
          for (int i = 0; i < 8; i++) t[p][kb][i] = fast_exp2(fmaf(t[p][kb][i], scale, neg_m2));
          pb[p][kb] = pack8<CT>(t[p][kb]);
        }
      }
    }
    if (live) {
#pragma unroll
      for (int kb = 0; kb < NKB; kb++) {
        bool need = false;
#pragma unroll
        for (int p = 0; p < NP; p++) need = need || bv[p][kb];
        if (!need) continue;
#pragma unroll
        for (int d = 0; d < VB; d++) {
          const u32x4 vt = lds_read_tokens_as_k(sV, PV, 32 * kb, 16 * d, n, g);
#pragma unroll
          for (int p = 0; p < NP; p++)
            if (bv[p][kb]) acc[p][d] = Mma<CT>::mfma(vt, pb[p][kb], acc[p][d]);
        }
#pragma unroll
        for (int p = 0; p < NP; p++)
          if (bv[p][kb]) acc_l[p] = Mma<CT>::mfma(ones, pb[p][kb], acc_l[p]);
      }
    }
  };
  // The last chunk is peeled off so that prefetch and commit are unconditional inside the loop:
  // with `if (has_next)` around each, the compiler sees a path on which loads stay pending across
  // the back edge and guards every later load with a full vmcnt(0) wait.
  auto consume = [&](const FlashChunk& c) __attribute__((always_inline)) {
    if (CAUSAL) consume_t(c, FlashTailDyn{});
    else if (chunk_tail(c)) consume_t(c, std::true_type{});
    else consume_t(c, std::false_type{});
  };
  FlashChunk cc = W.at(0);
  for (int ci = 0; ci + 1 < W.nchunks; ci++) {
    const FlashChunk cn = W.next(cc);
    issue(cn);
    if (CAUSAL) consume(cc);
    else consume_t(cc, std::false_type{});
    __syncthreads();
    commit();
    __syncthreads();
    cc = cn;
  }
  if (W.nchunks > 0) consume(cc);
  __syncthreads();

  // ---- epilogue: normalise, O^T fragments -> LDS tile -> coalesced rows
#pragma unroll
  for (int p = 0; p < NP; p++) {
    const float lt = wave_sum4(acc_l[p][0]);   // only row 0 of the ones operand is set: the other lane groups hold zeros
    const float inv = lt > 0.f ? fast_rcp(lt) : 0.f;
    TL* orow = reinterpret_cast<TL*>(smem + (wave * 16 * NP + 16 * p + n) * PO);
#pragma unroll
    for (int d = 0; d < VB; d++)
#pragma unroll
      for (int i = 0; i < 4; i++) orow[16 * d + 4 * g + i] = (TL)(acc[p][d][i] * inv);
    if (g == 0 && tq[p] >= 0) store_stream4(a.lse + (b * a.ls[0] + h * a.ls[1] + tq[p] * a.ls[2]), m_run[p] * scale + fast_log2(lt));
  }
  __syncthreads();
  int tw = tid;   // opaque copy: keeps the tile writer's addresses out of the registers that live across the chunk loop
  asm volatile("" : "+v"(tw));
  store_tile<TIO, TL, DV>(smem, PO, ob, flash_tok<IMG>(a.os, a.tm), a.os[3], a.dv, a.o_vec != 0, OWN,
                          [&](int row) { return x0 + row < a.Lq ? (int64_t)(own_base + x0 + row) : (int64_t)-1; }, no_rope, tw);
}

// =============================================================================================
// Dense and causal backward: replaces _attn_bwd_dkdv / _attn_bwd_dq / _attn_bwd
// (src/flash_attn.py:204-449; causal masking :361-379, :416-434), Lq != Lk allowed when not
// causal, with the decoupled structure of the reference
// (dK/dV pass over key blocks, dQ pass over query blocks) as two kernels; no host-side
// pre-scaling pass over k (src/flash_attn.py:509-510), no atomics.
struct FlashBwdArgs {
  const void *q, *k, *v, *o, *d_o;
  const float *lse, *delta;
  float* delta_out;   // fuse_delta: the dQ kernel (launched first) stores delta = rowsum(o * dO) of its own queries
  void *dq, *dk, *dv;
  int64_t qs[5], ks[5], vs[5], os[5], dos[5], dqs[5], dks[5], dvs[5], ls[3];
  DltTokMap tm;
  int32_t fuse_delta;
  int32_t B, H, Lq, Lk, dk_, dv_;
  int32_t nblk_q, nblk_k;
  int32_t causal, causal_group;   // causal_group: see flash_block_causal
  int32_t tile;
  DltGeom g;
  int32_t dq_vec, dk_vec, dv_vec;
  int32_t lds_q, lds_kv;
  float scale_log2, sm_scale;
};

// Staging of one chunk of CK tokens of two [token][dim] tensors (dims DA and DB) through registers.
template <int DA, int DB, int CK>
struct PairStage {
  static constexpr int ACH = DA / 8, BCH = DB / 8;
  static constexpr int NAI = CK * ACH / 256, NBI = CK * BCH / 256;
  static_assert(CK * ACH % 256 == 0 && CK * BCH % 256 == 0, "chunk must split evenly over 256 threads");
  u32x4 ra[NAI], rb[NBI];
  int ac, akey0, bc, bkey0;
  bool on_a, on_b;

  DLT_DEV void init(int tid, int dact_a, int dact_b) {
    const int ta = flash_stage_tid<ACH>(tid), tb = flash_stage_tid<BCH>(tid);
    ac = ta % ACH; akey0 = ta / ACH;
    bc = tb % BCH; bkey0 = tb / BCH;
    on_a = 8 * ac < dact_a; on_b = 8 * bc < dact_b;
#pragma unroll
    for (int it = 0; it < NAI; it++) ra[it] = u32x4{0u, 0u, 0u, 0u};
#pragma unroll
    for (int it = 0; it < NBI; it++) rb[it] = u32x4{0u, 0u, 0u, 0u};
  }
  // tokens past the end of the chunk are clamped onto its last token (the caller masks them)
  template <typename AD>
  DLT_DEV void issue(const char* a, const AD& ada, const char* b, const AD& adb, const FlashChunk& c) {
#pragma unroll
    for (int it = 0; it < NAI; it++) {
      const uint32_t off = ada(c, dlt_imin(akey0 + it * (256 / ACH), c.nvalid - 1));
      if (on_a) ra[it] = *reinterpret_cast<const u32x4*>(a + (off + 16 * ac));
    }
#pragma unroll
    for (int it = 0; it < NBI; it++) {
      const uint32_t off = adb(c, dlt_imin(bkey0 + it * (256 / BCH), c.nvalid - 1));
      if (on_b) rb[it] = *reinterpret_cast<const u32x4*>(b + (off + 16 * bc));
    }
  }
  DLT_DEV void commit(char* sa, int pa, char* sb, int pb) const {
    pin_loaded(ra);
    pin_loaded(rb);
#pragma unroll
    for (int it = 0; it < NAI; it++) lds_write16(sa + (akey0 + it * (256 / ACH)) * pa + 16 * ac, ra[it]);
#pragma unroll
    for (int it = 0; it < NBI; it++) lds_write16(sb + (bkey0 + it * (256 / BCH)) * pb + 16 * bc, rb[it]);
  }
};

// accumulators (C layout, [dim][own token]) of NP blocks -> LDS tile -> HBM rows
template <typename TIO, int D, int NP, typename SN>
DLT_DEV void flash_write_grad(char* sT, f32x4 (&acc)[NP][D / 16], float mul, TIO* base, const SN& sn, int64_t sd, int dact,
                              bool vec, int own_base, int x0, int len, int wave, int n, int g, int tid, int nrows = 64 * NP) {
  typedef typename TileOf<TIO>::type TL;
  constexpr int PT = D * (int)sizeof(TL) + 16;
  RopeDev no_rope = RopeDev{};
#pragma unroll
  for (int p = 0; p < NP; p++) {
    TL* row = reinterpret_cast<TL*>(sT + (wave * 16 * NP + 16 * p + n) * PT);
#pragma unroll
    for (int d = 0; d < D / 16; d++)
#pragma unroll
      for (int i = 0; i < 4; i++) row[16 * d + 4 * g + i] = (TL)(acc[p][d][i] * mul);
  }
  __syncthreads();
  // the tile writer's addresses are computed from an opaque copy of the thread id: computed from `tid` itself they are
  // hoisted above the chunk loop and occupy (or spill) registers across it
  int tw = tid;
  asm volatile("" : "+v"(tw));
  if (tw < 256)   // the tile writer walks the rows with 256 threads
    store_tile<TIO, TL, D>(sT, PT, base, sn, sd, dact, vec, nrows,
                           [&](int r) { return x0 + r < len ? (int64_t)(own_base + x0 + r) : (int64_t)-1; }, no_rope, tw);
  __syncthreads();
}

// ---- dQ: own = queries, K and V stream
template <typename TIO, int DK, int DV, int NP, int CK, int MODE>
__global__ __launch_bounds__(256, flash_occ_q(DK, DV)) void flash_bwd_q_kernel(const FlashBwdArgs a) {
  typedef typename ComputeOf<TIO>::type CT;
  extern __shared__ __align__(16) char smem[];
  constexpr bool CAUSAL = MODE == 1, TILE = MODE >= 2, IMG = MODE == 3;
  constexpr int PK = DK * 2 + FLASH_PAD, PV = DV * 2 + FLASH_PAD;
  constexpr int KC = DK / 32, VC = DV / 32, KB = DK / 16, NKB = CK / 32;
  constexpr int OWN = 64 * NP;

  const int tid = threadIdx.x;
  const int lane = tid & 63, n = lane & 15, g = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  char* sK = smem;
  char* sV = smem + CK * PK;

  const int lin = xcd_remap(blockIdx.x, gridDim.x);
  int bh, r_own, x0;
  if constexpr (CAUSAL) flash_block_causal(lin, a.nblk_q, a.B * a.H, a.causal_group, OWN, true, bh, r_own, x0);
  else flash_block(lin, a.nblk_q, TILE ? a.g.TR : 1, OWN, bh, r_own, x0);
  const int wq0 = x0 + wave * 16 * NP;
  const int b = bh / a.H, h = bh - b * a.H;
  const TIO* qb = reinterpret_cast<const TIO*>(a.q) + b * a.qs[0] + h * a.qs[1];
  const TIO* dob = reinterpret_cast<const TIO*>(a.d_o) + b * a.dos[0] + h * a.dos[1];
  const char* kb_ = reinterpret_cast<const char*>(reinterpret_cast<const TIO*>(a.k) + b * a.ks[0] + h * a.ks[1]);
  const char* vb_ = reinterpret_cast<const char*>(reinterpret_cast<const TIO*>(a.v) + b * a.vs[0] + h * a.vs[1]);
  const FlashAddr<IMG> ak = flash_addr<IMG>(a.ks, a.tm), av = flash_addr<IMG>(a.vs, a.tm);
  RopeDev no_rope = RopeDev{};
  const int own_base = TILE ? r_own * a.Lq : 0;

  FlashWalk<MODE, CK> W;
  if (TILE) W.init_tile(a.g, r_own, x0, OWN, false);
  else W.init_seq(0, CAUSAL ? dlt_imin(a.Lk, x0 + OWN) : a.Lk);

  PairStage<DK, DV, CK> st;
  st.init(tid, a.dk_, a.dv_);
  if (W.nchunks > 0) st.issue(kb_, ak, vb_, av, W.at(0));

  u32x4 qf[NP][KC], dof[NP][VC];
  float nlse[NP], del_n[NP];
  int klim[NP], vlo[NP], vhi[NP];
#pragma unroll
  for (int p = 0; p < NP; p++) {
    const int xq = wq0 + 16 * p + n;
    const int64_t tq = xq < a.Lq ? (int64_t)(own_base + xq) : (int64_t)-1;
    klim[p] = CAUSAL ? dlt_imin(xq, a.Lk - 1) : a.Lk - 1;
    vlo[p] = vhi[p] = 0;
    if (TILE && wq0 + 16 * p < a.Lq) {
      int rl, rh;
      dlt_key_range(a.g, r_own, wq0 + 16 * p, rl, rh, vlo[p], vhi[p]);
    }
    swa1_load_own<TIO, CT, DK>(qf[p], qb, 1, a.dk_, flash_own_off<IMG>(a.qs, a.tm, tq), g, no_rope, false);
    swa1_load_own<TIO, CT, DV>(dof[p], dob, 1, a.dv_, flash_own_off<IMG>(a.dos, a.tm, tq), g, no_rope, false);
    const int64_t off = b * a.ls[0] + h * a.ls[1] + (tq >= 0 ? tq : 0) * a.ls[2];
    nlse[p] = tq >= 0 ? -a.lse[off] : 0.f;
    if (a.fuse_delta != 0) {
      // the reference's pre-pass (src/flash_attn.py:186-202) folded in: delta of the own queries
      const TIO* ob = reinterpret_cast<const TIO*>(a.o) + b * a.os[0] + h * a.os[1];
      u32x4 of[VC];
      swa1_load_own<TIO, CT, DV>(of, ob, 1, a.dv_, flash_own_off<IMG>(a.os, a.tm, tq), g, no_rope, false);
      float part = 0.f;
#pragma unroll
      for (int c_ = 0; c_ < VC; c_++) {
        float fo[8], fd[8];
        unpack8<CT>(of[c_], fo);
        unpack8<CT>(dof[p][c_], fd);
#pragma unroll
        for (int j = 0; j < 8; j++) part += fo[j] * fd[j];
      }
      del_n[p] = wave_sum4(part);
      if (g == 0 && tq >= 0) store_stream4(a.delta_out + off, del_n[p]);
    } else {
      del_n[p] = tq >= 0 ? a.delta[off] : 0.f;
    }
  }
  f32x4 dq_acc[NP][KB];
#pragma unroll
  for (int p = 0; p < NP; p++)
#pragma unroll
    for (int d = 0; d < KB; d++) dq_acc[p][d] = f32x4{0.f, 0.f, 0.f, 0.f};
  const float scale = a.scale_log2;

  if (W.nchunks > 0) st.commit(sK, PK, sV, PV);
  __syncthreads();
  pin_loaded(qf);
  pin_loaded(dof);
#pragma unroll
  for (int p = 0; p < NP; p++) { pin_loaded(nlse[p]); pin_loaded(del_n[p]); }
  // The dP products start from -delta of the lane's query (the C operand of the first product of a chain): the matrix
  // pipe delivers dP - delta.
  f32x4 dinit[NP];
#pragma unroll
  for (int p = 0; p < NP; p++) dinit[p] = f32x4{-del_n[p], -del_n[p], -del_n[p], -del_n[p]};

  // `tail`: some keys of the chunk lie past the end or (causal) above the wave's first query, and every pair is tested.
  // It is a compile-time tag: as a run-time flag the test was folded into a select per element of every chunk.
  auto chunk_tail = [&](const FlashChunk& c) {
    return !TILE && (c.nvalid < CK || (CAUSAL && c.x + CK - 1 > wq0));
  };
  auto consume_t = [&](const FlashChunk& c, auto tail_tag) __attribute__((always_inline)) {
    // the tag is true_type / false_type (dense: known per call site) or FlashTailDyn (causal: tested per chunk)
    bool tail;
    if constexpr (std::is_same<decltype(tail_tag), FlashTailDyn>::value) tail = chunk_tail(c);
    else tail = decltype(tail_tag)::value;
    const int k0 = c.x;
    const bool live = !CAUSAL || k0 <= wq0 + 16 * NP - 1;
#pragma unroll
    for (int kb = 0; kb < NKB; kb++) {
      if (!live) continue;
      bool bv[NP], need = false;
#pragma unroll
      for (int p = 0; p < NP; p++) {
        bv[p] = !TILE || (k0 + 32 * kb + 32 > vlo[p] && k0 + 32 * kb < vhi[p]);
        need = need || bv[p];
      }
      if (!need) continue;
      u32x4 ka[2][KC], va[2][VC];
#pragma unroll
      for (int mb = 0; mb < 2; mb++) {
#pragma unroll
        for (int c_ = 0; c_ < KC; c_++) ka[mb][c_] = lds_read16(sK + (32 * kb + 16 * mb + n) * PK + (32 * c_ + 8 * g) * 2);
#pragma unroll
        for (int c_ = 0; c_ < VC; c_++) va[mb][c_] = lds_read16(sV + (32 * kb + 16 * mb + n) * PV + (32 * c_ + 8 * g) * 2);
      }
      u32x4 dsb[NP];
#pragma unroll
      for (int p = 0; p < NP; p++) {
        if (!bv[p]) continue;
        f32x4 s[2], dp[2];
#pragma unroll
        for (int mb = 0; mb < 2; mb++) {
          s[mb] = f32x4{0.f, 0.f, 0.f, 0.f};
          dp[mb] = dinit[p];
#pragma unroll
          for (int c_ = 0; c_ < KC; c_++) s[mb] = Mma<CT>::mfma(ka[mb][c_], qf[p][c_], s[mb]);
#pragma unroll
          for (int c_ = 0; c_ < VC; c_++) dp[mb] = Mma<CT>::mfma(va[mb][c_], dof[p][c_], dp[mb]);
        }
        float ds[8];
#pragma unroll
        for (int mb = 0; mb < 2; mb++) {
          const bool hv = !TILE || (k0 + 32 * kb + 16 * mb >= vlo[p] && k0 + 32 * kb + 16 * mb < vhi[p]);
#pragma unroll
          for (int i = 0; i < 4; i++) {
            float pv = fast_exp2(fmaf(s[mb][i], scale, nlse[p]));
            if (tail) pv = (k0 + 32 * kb + 16 * mb + 4 * g + i) <= klim[p] ? pv : 0.f;
            if (TILE) pv = hv ? pv : 0.f;
            ds[4 * mb + i] = pv * dp[mb][i];
          }
        }
        dsb[p] = pack8<CT>(ds);
      }
#pragma unroll
      for (int d = 0; d < KB; d++) {
        const u32x4 kt = lds_read_tokens_as_k(sK, PK, 32 * kb, 16 * d, n, g);
#pragma unroll
        for (int p = 0; p < NP; p++)
          if (bv[p]) dq_acc[p][d] = Mma<CT>::mfma(kt, dsb[p], dq_acc[p][d]);
      }
    }
  };
  auto consume = [&](const FlashChunk& c) __attribute__((always_inline)) {
    if (CAUSAL) consume_t(c, FlashTailDyn{});
    else if (chunk_tail(c)) consume_t(c, std::true_type{});
    else consume_t(c, std::false_type{});
  };
  // last chunk peeled off: unconditional prefetch and commit inside the loop (see the forward kernel); without a causal
  // mask only the last chunk can be short
  FlashChunk cc = W.at(0);
  for (int ci = 0; ci + 1 < W.nchunks; ci++) {
    const FlashChunk cn = W.next(cc);
    st.issue(kb_, ak, vb_, av, cn);
    if (CAUSAL) consume(cc);
    else consume_t(cc, std::false_type{});
    __syncthreads();
    st.commit(sK, PK, sV, PV);
    __syncthreads();
    cc = cn;
  }
  if (W.nchunks > 0) consume(cc);
  __syncthreads();
  TIO* dqb = reinterpret_cast<TIO*>(a.dq) + b * a.dqs[0] + h * a.dqs[1];
  flash_write_grad<TIO, DK, NP>(smem, dq_acc, a.sm_scale, dqb, flash_tok<IMG>(a.dqs, a.tm), a.dqs[3], a.dk_, a.dq_vec != 0, own_base, x0, a.Lq, wave, n, g, tid);
}

// ---- dK / dV: own = keys, Q, dO, lse2 and delta stream
template <typename TIO, int DK, int DV, int NP, int CK, int MODE>
__global__ __launch_bounds__(256, flash_occ_kv(DK, DV, MODE)) void flash_bwd_kv_kernel(const FlashBwdArgs a) {
  typedef typename ComputeOf<TIO>::type CT;
  extern __shared__ __align__(16) char smem[];
  constexpr bool CAUSAL = MODE == 1, TILE = MODE >= 2, IMG = MODE == 3;
  constexpr int PQ = DK * 2 + FLASH_PAD, PD = DV * 2 + FLASH_PAD;
  constexpr int KC = DK / 32, VC = DV / 32, KB = DK / 16, VB = DV / 16, NQB = CK / 32;
  constexpr int OWN = 64 * NP;

  const int tid = threadIdx.x;
  const int lane = tid & 63, n = lane & 15, g = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  char* sQ = smem;
  char* sDO = smem + CK * PQ;
  float* sLse = reinterpret_cast<float*>(smem + CK * (PQ + PD));
  float* sDel = sLse + CK;

  const int lin = xcd_remap(blockIdx.x, gridDim.x);
  int bh, r_own, x0;
  if constexpr (CAUSAL) flash_block_causal(lin, a.nblk_k, a.B * a.H, a.causal_group, OWN, false, bh, r_own, x0);
  else flash_block(lin, a.nblk_k, TILE ? a.g.TR : 1, OWN, bh, r_own, x0);
  const int b = bh / a.H, h = bh - b * a.H;
  const TIO* kb_ = reinterpret_cast<const TIO*>(a.k) + b * a.ks[0] + h * a.ks[1];
  const TIO* vb_ = reinterpret_cast<const TIO*>(a.v) + b * a.vs[0] + h * a.vs[1];
  const char* qb = reinterpret_cast<const char*>(reinterpret_cast<const TIO*>(a.q) + b * a.qs[0] + h * a.qs[1]);
  const char* dob = reinterpret_cast<const char*>(reinterpret_cast<const TIO*>(a.d_o) + b * a.dos[0] + h * a.dos[1]);
  const float* lseb = a.lse + b * a.ls[0] + h * a.ls[1];
  const float* delb = a.delta + b * a.ls[0] + h * a.ls[1];
  const FlashAddr<IMG> aq = flash_addr<IMG>(a.qs, a.tm), ad = flash_addr<IMG>(a.dos, a.tm);
  RopeDev no_rope = RopeDev{};
  const int own_base = TILE ? r_own * a.Lk : 0;

  // causal: queries below the first own key see none of the own keys
  FlashWalk<MODE, CK> W;
  if (TILE) W.init_tile(a.g, r_own, x0, OWN, true);
  else W.init_seq(CAUSAL ? (x0 / CK) * CK : 0, a.Lq);
  const int wk0 = x0 + wave * 16 * NP;  // first own key of this wave

  PairStage<DK, DV, CK> st;
  st.init(tid, a.dk_, a.dv_);
  if (W.nchunks > 0) st.issue(qb, aq, dob, ad, W.at(0));
  float r_lse = 0.f, r_del = 0.f;
  auto issue_scalars = [&](const FlashChunk& c) {
    if (tid < CK) {
      const int64_t tok = c.tok0 + dlt_imin(tid, c.nvalid - 1);
      r_lse = lseb[tok * a.ls[2]];
      r_del = delb[tok * a.ls[2]];
    }
  };
  if (W.nchunks > 0) issue_scalars(W.at(0));

  u32x4 kf[NP][KC], vf[NP][VC];
  int qmin[NP];           // causal: first query that sees this lane's key
  int vlo[NP], vhi[NP];   // tile mode: x interval of the queries that see this key block
#pragma unroll
  for (int p = 0; p < NP; p++) {
    const int xk = wk0 + 16 * p + n;
    const int64_t tk = xk < a.Lk ? (int64_t)(own_base + xk) : (int64_t)-1;
    qmin[p] = CAUSAL ? xk : 0;
    vlo[p] = vhi[p] = 0;
    if (TILE && wk0 + 16 * p < a.Lk) {
      int rl, rh;
      dlt_query_range(a.g, r_own, wk0 + 16 * p, rl, rh, vlo[p], vhi[p]);
    }
    swa1_load_own<TIO, CT, DK>(kf[p], kb_, 1, a.dk_, flash_own_off<IMG>(a.ks, a.tm, tk), g, no_rope, false);
    swa1_load_own<TIO, CT, DV>(vf[p], vb_, 1, a.dv_, flash_own_off<IMG>(a.vs, a.tm, tk), g, no_rope, false);
  }
  f32x4 dk_acc[NP][KB], dv_acc[NP][VB];
#pragma unroll
  for (int p = 0; p < NP; p++) {
#pragma unroll
    for (int d = 0; d < KB; d++) dk_acc[p][d] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int d = 0; d < VB; d++) dv_acc[p][d] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  const float scale = a.scale_log2;

  if (W.nchunks > 0) {
    st.commit(sQ, PQ, sDO, PD);
    if (tid < CK) { sLse[tid] = r_lse; sDel[tid] = r_del; }
  }
  __syncthreads();
  pin_loaded(kf);
  pin_loaded(vf);
  // The own values are negated and the dP products start from the staged delta of the lane's four queries (the C operand
  // of the first product of a chain): the matrix pipe delivers -(dP - delta), and dS = -p (.) (the sign is an operand
  // modifier).
#pragma unroll
  for (int p = 0; p < NP; p++)
#pragma unroll
    for (int c_ = 0; c_ < VC; c_++) {
      vf[p][c_].x ^= 0x80008000u; vf[p][c_].y ^= 0x80008000u; vf[p][c_].z ^= 0x80008000u; vf[p][c_].w ^= 0x80008000u;
    }

  // `tail`: some queries of the chunk lie past the end or (causal) below the wave's last own key (a compile-time tag, as
  // in the dQ kernel)
  auto chunk_tail = [&](const FlashChunk& c) {
    return !TILE && (c.nvalid < CK || (CAUSAL && c.x < wk0 + 16 * NP - 1));
  };
  auto consume_t = [&](const FlashChunk& c, auto tail_tag) __attribute__((always_inline)) {
    // the tag is true_type / false_type (dense: known per call site) or FlashTailDyn (causal: tested per chunk)
    bool tail;
    if constexpr (std::is_same<decltype(tail_tag), FlashTailDyn>::value) tail = chunk_tail(c);
    else tail = decltype(tail_tag)::value;
    const int q0 = c.x;
    // causal: every query of the chunk lies below every own key of this wave
    const bool live = !CAUSAL || q0 + CK - 1 >= wk0;
#pragma unroll
    for (int qb_ = 0; qb_ < NQB; qb_++) {
      if (!live) continue;
      bool bv[NP], need = false;
#pragma unroll
      for (int p = 0; p < NP; p++) {
        bv[p] = !TILE || (q0 + 32 * qb_ + 32 > vlo[p] && q0 + 32 * qb_ < vhi[p]);
        need = need || bv[p];
      }
      if (!need) continue;
      // the first products run over one 16-query half at a time (operands of a half: KC + VC vectors), the second
      // products contract over the whole block
      float pr[NP][8], ds[NP][8];
#pragma unroll
      for (int mb = 0; mb < 2; mb++) {
        u32x4 qa[KC], da[VC];
#pragma unroll
        for (int c_ = 0; c_ < KC; c_++) qa[c_] = lds_read16(sQ + (32 * qb_ + 16 * mb + n) * PQ + (32 * c_ + 8 * g) * 2);
#pragma unroll
        for (int c_ = 0; c_ < VC; c_++) da[c_] = lds_read16(sDO + (32 * qb_ + 16 * mb + n) * PD + (32 * c_ + 8 * g) * 2);
        const f32x4 lq = *reinterpret_cast<const f32x4*>(sLse + 32 * qb_ + 16 * mb + 4 * g);
        const f32x4 dl = *reinterpret_cast<const f32x4*>(sDel + 32 * qb_ + 16 * mb + 4 * g);
#pragma unroll
        for (int p = 0; p < NP; p++) {
          if (!bv[p]) continue;
          f32x4 sv = {0.f, 0.f, 0.f, 0.f}, dp = dl;
#pragma unroll
          for (int c_ = 0; c_ < KC; c_++) sv = Mma<CT>::mfma(qa[c_], kf[p][c_], sv);
#pragma unroll
          for (int c_ = 0; c_ < VC; c_++) dp = Mma<CT>::mfma(da[c_], vf[p][c_], dp);
          const bool hv = !TILE || (q0 + 32 * qb_ + 16 * mb >= vlo[p] && q0 + 32 * qb_ + 16 * mb < vhi[p]);
#pragma unroll
          for (int i = 0; i < 4; i++) {
            float pv = fast_exp2(fmaf(sv[i], scale, -lq[i]));
            if (tail) {
              const int qi = q0 + 32 * qb_ + 16 * mb + 4 * g + i;
              pv = (qi >= qmin[p] && qi < a.Lq) ? pv : 0.f;
            }
            if (TILE) pv = hv ? pv : 0.f;
            pr[p][4 * mb + i] = pv;
            ds[p][4 * mb + i] = -pv * dp[i];
          }
        }
      }
      u32x4 pb[NP], dsb[NP];
#pragma unroll
      for (int p = 0; p < NP; p++) {
        pb[p] = pack8<CT>(pr[p]);
        dsb[p] = pack8<CT>(ds[p]);
      }
#pragma unroll
      for (int d = 0; d < VB; d++) {
        const u32x4 dt = lds_read_tokens_as_k(sDO, PD, 32 * qb_, 16 * d, n, g);
#pragma unroll
        for (int p = 0; p < NP; p++)
          if (bv[p]) dv_acc[p][d] = Mma<CT>::mfma(dt, pb[p], dv_acc[p][d]);
      }
#pragma unroll
      for (int d = 0; d < KB; d++) {
        const u32x4 qt = lds_read_tokens_as_k(sQ, PQ, 32 * qb_, 16 * d, n, g);
#pragma unroll
        for (int p = 0; p < NP; p++)
          if (bv[p]) dk_acc[p][d] = Mma<CT>::mfma(qt, dsb[p], dk_acc[p][d]);
      }
    }
  };
  auto consume = [&](const FlashChunk& c) __attribute__((always_inline)) {
    if (CAUSAL) consume_t(c, FlashTailDyn{});
    else if (chunk_tail(c)) consume_t(c, std::true_type{});
    else consume_t(c, std::false_type{});
  };
  FlashChunk cc = W.at(0);
  for (int ci = 0; ci + 1 < W.nchunks; ci++) {
    const FlashChunk cn = W.next(cc);
    st.issue(qb, aq, dob, ad, cn);
    issue_scalars(cn);
    if (CAUSAL) consume(cc);
    else consume_t(cc, std::false_type{});   // without a causal mask only the last chunk can be short
    __syncthreads();
    st.commit(sQ, PQ, sDO, PD);
    pin_loaded(r_lse);
    pin_loaded(r_del);
    if (tid < CK) { sLse[tid] = r_lse; sDel[tid] = r_del; }
    __syncthreads();
    cc = cn;
  }
  if (W.nchunks > 0) consume(cc);
  __syncthreads();
  TIO* dkb = reinterpret_cast<TIO*>(a.dk) + b * a.dks[0] + h * a.dks[1];
  TIO* dvb = reinterpret_cast<TIO*>(a.dv) + b * a.dvs[0] + h * a.dvs[1];
  flash_write_grad<TIO, DK, NP>(smem, dk_acc, a.sm_scale, dkb, flash_tok<IMG>(a.dks, a.tm), a.dks[3], a.dk_, a.dk_vec != 0, own_base, x0, a.Lk, wave, n, g, tid);
  flash_write_grad<TIO, DV, NP>(smem, dv_acc, 1.0f, dvb, flash_tok<IMG>(a.dvs, a.tm), a.dvs[3], a.dv_, a.dv_vec != 0, own_base, x0, a.Lk, wave, n, g, tid);
}
