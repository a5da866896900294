// Marching backward kernels for token grids (b_size == 1, head dim 64, windows up to 13 x 13): the decoupled dQ and
// dK/dV passes of tiled_swa_bwd_large_kernel_decoupled_q (src/tiled_swa.py:407-562) on the sliding LDS ring of
// swam_common.hpp.
//
//   dQ   : a wave owns a 4x4 patch of queries per step; the ring holds K and V.  It runs first and computes
//          delta = rowsum(o * dO) of its own queries on the way (the reference's pre-pass, src/tiled_swa.py:253-282),
//          which the dK/dV kernel reads back.
//   dK/dV: a wave owns a 4x4 patch of keys per step; the ring holds Q and dO of the queries that can see them (the
//          window is symmetric), plus their lse2 and delta.
// Both recompute P = exp2(s * scale - lse2) per 32-token block; tokens of the ring side are the MFMA rows, so P / dS
// leave the first products in the layout the second products take as B operand.
// ROPE 0: no rotation; 3: q and k arrive rotated (saved by the forward pass), dq / dk get the transposed rotation as
// they are stored.  TL: the rotary tables are copied into LDS in the prologue and read from there.
#pragma once
#include "swam_fwd_kernel.hpp"

struct SwamBwdArgs {
  AttnProblem p;
  SwamPlan plan;
  const void *q, *k, *v, *o, *d_o;
  const float* lse;
  float* delta;   // written by the dQ kernel, read by the dK/dV kernel
  void *dq, *dk, *dv;
  int64_t qs[4], ks[4], vs[4], os[4], dos[4], dqs[4], dks[4], dvs[4], ls[3];
  float scale_log2;
};

// a pair of own-token fragments (pieces g and 4 + g of token n)
struct SwamFrag { u32x4 f[2]; };

DLT_DEV void swam_frag_issue(SwamFrag& w, const char* base, int sn2, int tok, int g) {
  const char* p = base + ((uint32_t)((tok >= 0 ? tok : 0) * sn2) + 16 * g);
  w.f[0] = *reinterpret_cast<const u32x4*>(p);
  w.f[1] = *reinterpret_cast<const u32x4*>(p + 64);
}
DLT_DEV void swam_frag_pin(const SwamFrag& w) { pin_loaded(w.f[0]); pin_loaded(w.f[1]); }

// table rows for the two transposed tile rows a lane stores (piece lane & 7 of tokens tok[0], tok[1])
template <bool TL>
DLT_DEV void swam_store_tabs(SwamTab (&tb)[2], const int32_t (&id)[2], int lane, const RopeDev& rope, SwamLds tabs) {
  const int c = lane & 7;
#pragma unroll
  for (int it = 0; it < 2; it++) swam_tab_get<TL>(tb[it], id[it], (c >> 1) & 1, rope, tabs);
}

// =============================================================================================== dQ
template <typename TIO, int ROPE, bool TL>
__global__ __launch_bounds__(SWAM_THREADS) void swam_bwd_q_kernel(const SwamBwdArgs a) {
  typedef typename ComputeOf<TIO>::type CT;
  constexpr int D = 64;
  constexpr bool ROT = ROPE == 3;
  static_assert(!TL || ROT, "LDS tables only with rotation");
  constexpr int REGION = swam_region(D), SLOT = swam_slot(D);
  extern __shared__ __align__(16) char smem[];
  SwamLds tabs = (SwamLds)(smem + swam_ring(D));

  const int tid = threadIdx.x;
  const int lane = tid & 63, n = lane & 15, g = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int pc = wave & 3, rg = wave >> 2;
  const SwamGeom G = swam_geom(a.p, a.plan);

  const char* qb = reinterpret_cast<const char*>(a.q) + 2 * (G.b * a.qs[0] + G.h * a.qs[1]);
  const char* kb_ = reinterpret_cast<const char*>(a.k) + 2 * (G.b * a.ks[0] + G.h * a.ks[1]);
  const char* vb_ = reinterpret_cast<const char*>(a.v) + 2 * (G.b * a.vs[0] + G.h * a.vs[1]);
  const char* ob = reinterpret_cast<const char*>(a.o) + 2 * (G.b * a.os[0] + G.h * a.os[1]);
  const char* dob = reinterpret_cast<const char*>(a.d_o) + 2 * (G.b * a.dos[0] + G.h * a.dos[1]);
  TIO* dqb = reinterpret_cast<TIO*>(a.dq) + G.b * a.dqs[0] + G.h * a.dqs[1];
  const float* lseb = a.lse + G.b * a.ls[0] + G.h * a.ls[1];
  float* delb = a.delta + G.b * a.ls[0] + G.h * a.ls[1];
  const int sn2q = (int)a.qs[2] * 2, sn2o = (int)a.os[2] * 2, sn2do = (int)a.dos[2] * 2;
  const int64_t dqs2 = a.dqs[2], ls2 = a.ls[2];
  const RopeDev rope = a.p.rope;
  const int32_t* rope_idx = ROT ? rope.idx : nullptr;
  const float scale = a.scale_log2, sm_scale = a.p.sm_scale;

  SwamStage st;
  swam_stage_init(st, G, tid);
  const int kpar = wave >> 2;
  SwamSide side[2];
  {
    const SwamSide sk = swam_side(kb_, (int)a.ks[2] * 2, G, st), sv = swam_side(vb_, (int)a.vs[2] * 2, G, st);
    side[0] = kpar == 0 ? sk : sv;
    side[1] = kpar == 0 ? sv : sk;
  }
  SwamLane L;
  swam_lane_init(L, pc, n, g);
  const int c_p = G.c0 + 4 * pc;
  auto commit_chunk = [&](const SwamItem& it, int c) {
    swam_commit(it, st, smem + (c % SWAM_NSLOT) * SLOT + ((c & 1) == kpar ? 0 : REGION));
  };

  // own tokens of a step: q, dO, o fragments and lse2 in flight; `finish` turns o into delta
  struct Own { SwamFrag q, d_o, o; float lse; int tok; };
  auto own_issue = [&](Own& w, int r_p) {
    w.tok = swam_own_tok(G, r_p, c_p, n);
    swam_frag_issue(w.q, qb, sn2q, w.tok, g);
    swam_frag_issue(w.d_o, dob, sn2do, w.tok, g);
    swam_frag_issue(w.o, ob, sn2o, w.tok, g);
    w.lse = lseb[(int64_t)(w.tok >= 0 ? w.tok : 0) * ls2];
  };
  auto own_pin = [&](const Own& w) { swam_frag_pin(w.q); swam_frag_pin(w.d_o); swam_frag_pin(w.o); pin_loaded(w.lse); };
  // delta = rowsum(o * dO) of the own tokens, published for the dK/dV kernel
  auto own_delta = [&](const Own& w) {
    float part = 0.f;
#pragma unroll
    for (int c = 0; c < 2; c++) {
      float fo[8], fd[8];
      unpack8<CT>(w.o.f[c], fo);
      unpack8<CT>(w.d_o.f[c], fd);
#pragma unroll
      for (int j = 0; j < 8; j++) part += fo[j] * fd[j];
    }
    const float del = wave_sum4(part);
    if (g == 0 && w.tok >= 0) store_stream4(delb + (int64_t)w.tok * ls2, del);
    return del;
  };
  // rotary indices of the two tile rows a lane stores in step s
  auto store_ids = [&](int32_t (&id)[2], int s) {
    const int r_p = G.r0 + 8 * s + 4 * rg;
#pragma unroll
    for (int it = 0; it < 2; it++) {
      const int t = swam_own_tok(G, r_p, c_p, (lane >> 3) + 8 * it);
      id[it] = rope_idx[t >= 0 ? t : 0];
    }
  };

  // ---- prologue
  Own cur;
  float del_n;
  {
    f32x4 tab16;
    if (TL) tab16 = swam_tab_fetch(rope, tid);
    SwamItem it[SWAM_NSLOT];
#pragma unroll
    for (int c = 0; c < SWAM_NSLOT; c++) swam_issue(it[c], st, G, c, side[c & 1]);
    own_issue(cur, G.r0 + 4 * rg);
    if (TL) {
      pin_loaded(tab16);
      swam_tab_store(smem + swam_ring(D), tid, tab16);   // visible after the barrier that ends the prologue
    }
    // chunk by chunk (loads return in order): the LDS writes of a chunk overlap the arrival of the later ones
#pragma unroll
    for (int c = 0; c < SWAM_NSLOT; c++) {
      swam_pin(it[c]);
      commit_chunk(it[c], c);
    }
    own_pin(cur);
    del_n = own_delta(cur);
  }
  __syncthreads();

  const int qr_l = n >> 2, qc_l = n & 3;
  const int clo = dlt_imax(qc_l, G.WC - c_p), chi = dlt_imin(qc_l + 2 * G.WC, G.TC - 1 - c_p + G.WC);
  SwamLds lds = (SwamLds)smem;

  struct Out { f32x4 acc[4]; };
  auto step = [&](const int s) {
    const int r_p = G.r0 + 8 * s + 4 * rg;
    const u32x4 qf0 = cur.q.f[0], qf1 = cur.q.f[1], df0 = cur.d_o.f[0], df1 = cur.d_o.f[1];
    const bool q_ok = (r_p + qr_l < G.TR) && (c_p + qc_l < G.TC);
    const int rlo = dlt_imax(qr_l, G.WR - r_p), rhi = dlt_imin(qr_l + 2 * G.WR, G.TR - 1 - r_p + G.WR);
    const int cspan = q_ok ? chi - clo : -1;
    // the dP products start from -delta of the lane's query (the C operand): the matrix pipe delivers dP - delta
    const float neg_lse = -cur.lse, neg_del = -del_n;
    const f32x4 dinit = {neg_del, neg_del, neg_del, neg_del};
    int sb[4];
    {
      const int s5 = (2 * s + rg) % SWAM_NSLOT;
#pragma unroll
      for (int j = 0; j < 4; j++) sb[j] = __builtin_amdgcn_readfirstlane((s5 + j >= SWAM_NSLOT ? s5 + j - SWAM_NSLOT : s5 + j) * SLOT);
    }
    Out r;
#pragma unroll
    for (int d = 0; d < 4; d++) r.acc[d] = f32x4{0.f, 0.f, 0.f, 0.f};
    // first products half-block by half-block (16 keys: 4 halo rows x 4 columns), two operand buffers used alternately;
    // the dQ product contracts over the whole 32-key block
    u32x4 ka[2][2], va[2][2];
    auto read_half = [&](int hb, u32x4 (&kh)[2], u32x4 (&vh)[2]) {   // hb: half-block index 0..15 = 4 j + cg
      const int j = hb >> 2, cg = hb & 3;
      SwamLds pk = lds + sb[j] + 512 * cg, pv = pk + REGION;
      const int o0 = (cg & 1) ? L.a_odd : L.a_even, o1 = (cg & 1) ? L.a_even : L.a_odd;
      kh[0] = swam_lds16(pk + o0); kh[1] = swam_lds16(pk + o1);
      vh[0] = swam_lds16(pv + o0); vh[1] = swam_lds16(pv + o1);
    };
    read_half(0, ka[0], va[0]);
#pragma unroll
    for (int b = 0; b < 8; b++) {
      const int j = b >> 1, kb = b & 1;
      const int hrow = 4 * j + g;
      const bool row_vis = (j < G.nch) & (hrow >= rlo) & (hrow <= rhi);
      // K^T of this block (tokens along k) for the dQ product
      u32x4 kt[4];
      if (kb == 0) swam_read_tr_block<0>(lds + sb[j], L, kt); else swam_read_tr_block<1>(lds + sb[j], L, kt);
      float ds[8];
#pragma unroll
      for (int mb = 0; mb < 2; mb++) {
        const int hb = 2 * b + mb;
        if (hb < 15) read_half(hb + 1, ka[(hb + 1) & 1], va[(hb + 1) & 1]);
        __builtin_amdgcn_sched_barrier(0);
        const u32x4(&kc)[2] = ka[hb & 1];
        const u32x4(&vc)[2] = va[hb & 1];
        f32x4 sv = {0.f, 0.f, 0.f, 0.f}, pv;
        sv = Mma<CT>::mfma(kc[0], qf0, sv);
        pv = Mma<CT>::mfma(vc[0], df0, dinit);
        sv = Mma<CT>::mfma(kc[1], qf1, sv);
        pv = Mma<CT>::mfma(vc[1], df1, pv);
#pragma unroll
        for (int i = 0; i < 4; i++) {
          const bool vis = row_vis & ((unsigned)(8 * kb + 4 * mb + i - clo) <= (unsigned)cspan);
          const float e = fast_exp2(fmaf(sv[i], scale, vis ? neg_lse : -INFINITY));
          ds[4 * mb + i] = e * pv[i];
        }
      }
      const u32x4 dsb = pack8<CT>(ds);
#pragma unroll
      for (int d = 0; d < 4; d++) r.acc[d] = Mma<CT>::mfma(kt[d], dsb, r.acc[d]);
    }
    return r;
  };
  auto scratch_of = [&](int s) -> char* {
    const int c_new = 2 * s + 5;
    return smem + ((2 * s) % SWAM_NSLOT) * SLOT + ((c_new & 1) == kpar ? 0 : REGION) + 32 * (wave & 3) * 128;
  };
  // dq of step s: transposed to row pieces, rotated back when the inputs were rotated, stored
  auto store_dq = [&](const Out& r, int s, const int32_t (&id)[2]) {
    const int r_p = G.r0 + 8 * s + 4 * rg;
    int tok[2];
#pragma unroll
    for (int it = 0; it < 2; it++) tok[it] = swam_own_tok(G, r_p, c_p, (lane >> 3) + 8 * it);
    SwamTab tb[2];
    if (ROT) swam_store_tabs<TL>(tb, id, lane, rope, tabs);
    u32x4 v[2], pv[2];
    swam_tile_transpose<CT, ROT>(scratch_of(s), r.acc, sm_scale, lane, v, pv);
    if (ROT) {
#pragma unroll
      for (int it = 0; it < 2; it++) swam_rotate_piece<CT>(v[it], pv[it], tb[it], lane & 7, true);
    }
    swam_store_rows<TIO>(dqb, dqs2, tok, lane, v);
  };

  for (int s = 0; s + 1 < G.nstep; s++) {
    SwamItem ia, ib;
    swam_issue(ia, st, G, 2 * s + 5, side[1]);
    swam_issue(ib, st, G, 2 * s + 6, side[0]);
    Own nxt;
    own_issue(nxt, G.r0 + 8 * (s + 1) + 4 * rg);
    int32_t id[2] = {-1, -1};
    if (ROT) store_ids(id, s);
    const Out r = step(s);
    __syncthreads();
    swam_pin(ia);
    swam_pin(ib);
    own_pin(nxt);
    if (ROT) asm volatile("" ::"v"(id[0]), "v"(id[1]));
    store_dq(r, s, id);
    commit_chunk(ia, 2 * s + 5);
    commit_chunk(ib, 2 * s + 6);
    cur = nxt;
    del_n = own_delta(cur);
    __syncthreads();
  }
  {
    const int s = G.nstep - 1;
    int32_t id[2] = {-1, -1};
    if (ROT) store_ids(id, s);
    const Out r = step(s);
    __syncthreads();
    store_dq(r, s, id);
  }
}

// =============================================================================================== dK / dV
template <typename TIO, int ROPE, bool TL>
__global__ __launch_bounds__(SWAM_THREADS) void swam_bwd_kv_kernel(const SwamBwdArgs a) {
  typedef typename ComputeOf<TIO>::type CT;
  constexpr int D = 64;
  constexpr bool ROT = ROPE == 3;
  static_assert(!TL || ROT, "LDS tables only with rotation");
  constexpr int REGION = swam_region(D), SLOT = swam_slot(D);
  extern __shared__ __align__(16) char smem[];
  float* sLse = reinterpret_cast<float*>(smem + swam_ring(D));   // [slot][token of the chunk]
  float* sDel = sLse + SWAM_NSLOT * SWAM_TOK;
  constexpr int TAB_OFF = swam_ring(D) + 2 * SWAM_NSLOT * SWAM_TOK * 4;
  SwamLds tabs = (SwamLds)(smem + TAB_OFF);

  const int tid = threadIdx.x;
  const int lane = tid & 63, n = lane & 15, g = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int pc = wave & 3, rg = wave >> 2;
  const SwamGeom G = swam_geom(a.p, a.plan);

  const char* qb = reinterpret_cast<const char*>(a.q) + 2 * (G.b * a.qs[0] + G.h * a.qs[1]);
  const char* kb_ = reinterpret_cast<const char*>(a.k) + 2 * (G.b * a.ks[0] + G.h * a.ks[1]);
  const char* vb_ = reinterpret_cast<const char*>(a.v) + 2 * (G.b * a.vs[0] + G.h * a.vs[1]);
  const char* dob = reinterpret_cast<const char*>(a.d_o) + 2 * (G.b * a.dos[0] + G.h * a.dos[1]);
  TIO* dkb = reinterpret_cast<TIO*>(a.dk) + G.b * a.dks[0] + G.h * a.dks[1];
  TIO* dvb = reinterpret_cast<TIO*>(a.dv) + G.b * a.dvs[0] + G.h * a.dvs[1];
  const float* lseb = a.lse + G.b * a.ls[0] + G.h * a.ls[1];
  const float* delb = a.delta + G.b * a.ls[0] + G.h * a.ls[1];
  const int sn2k = (int)a.ks[2] * 2, sn2v = (int)a.vs[2] * 2;
  const int64_t dks2 = a.dks[2], dvs2 = a.dvs[2];
  const int ls2 = (int)a.ls[2];
  const RopeDev rope = a.p.rope;
  const int32_t* rope_idx = ROT ? rope.idx : nullptr;
  const float scale = a.scale_log2, sm_scale = a.p.sm_scale;

  SwamStage st;
  swam_stage_init(st, G, tid);
  const int kpar = wave >> 2;   // chunk parity for which this half stages Q (and the scalars); dO otherwise
  SwamSide side[2];
  {
    const SwamSide sq = swam_side(qb, (int)a.qs[2] * 2, G, st), sd = swam_side(dob, (int)a.dos[2] * 2, G, st);
    side[0] = kpar == 0 ? sq : sd;
    side[1] = kpar == 0 ? sd : sq;
  }
  SwamLane L;
  swam_lane_init(L, pc, n, g);
  const int c_p = G.c0 + 4 * pc;
  const int sc_lane = (g * SWAM_HCW + 4 * pc) * 4;   // byte offset of the lane's first scalar inside a chunk's array
  auto commit_chunk = [&](const SwamItem& it, int c) {
    swam_commit(it, st, smem + (c % SWAM_NSLOT) * SLOT + ((c & 1) == kpar ? 0 : REGION));
  };
  // per-token scalars of a Q chunk: the thread with piece 0 of a token fetches its lse2, the one with piece 1 its delta
  const float* sc_base = st.qd == 0 ? lseb : delb;
  float* sc_dst = (st.qd == 0 ? sLse : sDel) + (tid & 255) / 2;
  auto scalar_issue = [&](int c) -> float {
    const int r = dlt_imax(0, dlt_imin(swam_item_row(st, G, c), G.TR - 1));
    return sc_base[(uint32_t)((r * G.TC + st.cc) * ls2)];
  };
  auto scalar_commit = [&](float v, int c) {
    if (st.live) sc_dst[(c % SWAM_NSLOT) * SWAM_TOK] = v;
  };

  struct Own { SwamFrag k, v; int tok; };
  auto own_issue = [&](Own& w, int r_p) {
    w.tok = swam_own_tok(G, r_p, c_p, n);
    swam_frag_issue(w.k, kb_, sn2k, w.tok, g);
    swam_frag_issue(w.v, vb_, sn2v, w.tok, g);
  };
  auto own_pin = [&](const Own& w) { swam_frag_pin(w.k); swam_frag_pin(w.v); };
  // The own values are negated and the dP products start from the staged delta of the lane's four queries (read from LDS
  // straight into the C operand): the matrix pipe delivers -(dP - delta), and dS = -p (.) (the sign is an operand modifier).
  auto own_negate_v = [&](Own& w) {
#pragma unroll
    for (int c = 0; c < 2; c++) {
      w.v.f[c].x ^= 0x80008000u; w.v.f[c].y ^= 0x80008000u; w.v.f[c].z ^= 0x80008000u; w.v.f[c].w ^= 0x80008000u;
    }
  };
  auto store_ids = [&](int32_t (&id)[2], int s) {
    const int r_p = G.r0 + 8 * s + 4 * rg;
#pragma unroll
    for (int it = 0; it < 2; it++) {
      const int t = swam_own_tok(G, r_p, c_p, (lane >> 3) + 8 * it);
      id[it] = rope_idx[t >= 0 ? t : 0];
    }
  };

  // ---- prologue
  Own cur;
  {
    f32x4 tab16;
    if (TL) tab16 = swam_tab_fetch(rope, tid);
    SwamItem it[SWAM_NSLOT];
    float sc[3] = {0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < SWAM_NSLOT; c++) swam_issue(it[c], st, G, c, side[c & 1]);
#pragma unroll
    for (int i = 0; i < 3; i++)
      if (kpar + 2 * i < SWAM_NSLOT) sc[i] = scalar_issue(kpar + 2 * i);
    own_issue(cur, G.r0 + 4 * rg);
    if (TL) {
      pin_loaded(tab16);
      swam_tab_store(smem + TAB_OFF, tid, tab16);   // visible after the barrier that ends the prologue
    }
#pragma unroll
    for (int c = 0; c < SWAM_NSLOT; c++) {
      swam_pin(it[c]);
      commit_chunk(it[c], c);
    }
#pragma unroll
    for (int i = 0; i < 3; i++) pin_loaded(sc[i]);
    own_pin(cur);
    own_negate_v(cur);
#pragma unroll
    for (int i = 0; i < 3; i++)
      if (kpar + 2 * i < SWAM_NSLOT) scalar_commit(sc[i], kpar + 2 * i);
  }
  __syncthreads();

  const int qr_l = n >> 2, qc_l = n & 3;
  const int clo = dlt_imax(qc_l, G.WC - c_p), chi = dlt_imin(qc_l + 2 * G.WC, G.TC - 1 - c_p + G.WC);
  SwamLds lds = (SwamLds)smem;
  SwamLds ldsL = (SwamLds)sLse, ldsD = (SwamLds)sDel;

  struct Out { f32x4 dk[4], dv[4]; };
  auto step = [&](const int s) {
    const int r_p = G.r0 + 8 * s + 4 * rg;
    const u32x4 kf0 = cur.k.f[0], kf1 = cur.k.f[1], vf0 = cur.v.f[0], vf1 = cur.v.f[1];
    const bool k_ok = (r_p + qr_l < G.TR) && (c_p + qc_l < G.TC);
    const int rlo = dlt_imax(qr_l, G.WR - r_p), rhi = dlt_imin(qr_l + 2 * G.WR, G.TR - 1 - r_p + G.WR);
    const int cspan = k_ok ? chi - clo : -1;
    int sb[4], ss[4];
    {
      const int s5 = (2 * s + rg) % SWAM_NSLOT;
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const int sl = s5 + j >= SWAM_NSLOT ? s5 + j - SWAM_NSLOT : s5 + j;
        sb[j] = __builtin_amdgcn_readfirstlane(sl * SLOT);
        ss[j] = __builtin_amdgcn_readfirstlane(sl * SWAM_TOK * 4);
      }
    }
    Out r;
#pragma unroll
    for (int d = 0; d < 4; d++) { r.dk[d] = f32x4{0.f, 0.f, 0.f, 0.f}; r.dv[d] = f32x4{0.f, 0.f, 0.f, 0.f}; }
    // A block of 32 queries is two halves of 16 (4 halo rows x 4 columns at column groups cg and cg + 1): the first
    // products run half by half (two operand buffers of 16 registers per tensor, used alternately), the second
    // products contract over the whole block.
    u32x4 qa[2][2], da[2][2];
    auto read_half = [&](int hb, u32x4 (&qh)[2], u32x4 (&dh)[2]) {   // hb: half-block index 0..15 = 4 j + cg
      const int j = hb >> 2, cg = hb & 3;
      SwamLds pq = lds + sb[j] + 512 * cg, pd = pq + REGION;
      const int o0 = (cg & 1) ? L.a_odd : L.a_even, o1 = (cg & 1) ? L.a_even : L.a_odd;
      qh[0] = swam_lds16(pq + o0); qh[1] = swam_lds16(pq + o1);
      dh[0] = swam_lds16(pd + o0); dh[1] = swam_lds16(pd + o1);
    };
    read_half(0, qa[0], da[0]);
#pragma unroll
    for (int b = 0; b < 8; b++) {
      const int j = b >> 1, kb = b & 1;
      const int hrow = 4 * j + g;
      const bool row_vis = (j < G.nch) & (hrow >= rlo) & (hrow <= rhi);
      float pr[8], ds[8];
#pragma unroll
      for (int mb = 0; mb < 2; mb++) {
        const int hb = 2 * b + mb;
        if (hb < 15) read_half(hb + 1, qa[(hb + 1) & 1], da[(hb + 1) & 1]);
        // lse2 / delta of the half's queries (lane group g: halo row g, 4 columns)
        const f32x4 lq = *reinterpret_cast<DLT_LDS const f32x4*>(ldsL + ss[j] + sc_lane + 32 * kb + 16 * mb);
        const f32x4 dq_ = *reinterpret_cast<DLT_LDS const f32x4*>(ldsD + ss[j] + sc_lane + 32 * kb + 16 * mb);
        __builtin_amdgcn_sched_barrier(0);
        const u32x4(&qc)[2] = qa[hb & 1];
        const u32x4(&dc)[2] = da[hb & 1];
        f32x4 sv = {0.f, 0.f, 0.f, 0.f}, pv;
        sv = Mma<CT>::mfma(qc[0], kf0, sv);
        pv = Mma<CT>::mfma(dc[0], vf0, dq_);
        sv = Mma<CT>::mfma(qc[1], kf1, sv);
        pv = Mma<CT>::mfma(dc[1], vf1, pv);
#pragma unroll
        for (int i = 0; i < 4; i++) {
          const bool vis = row_vis & ((unsigned)(8 * kb + 4 * mb + i - clo) <= (unsigned)cspan);
          pr[4 * mb + i] = fast_exp2(fmaf(sv[i], scale, vis ? -lq[i] : -INFINITY));
          ds[4 * mb + i] = -pr[4 * mb + i] * pv[i];
        }
      }
      const u32x4 pb = pack8<CT>(pr), dsb = pack8<CT>(ds);
      // dO^T then Q^T of the block (tokens along k), one after the other in the same registers
      u32x4 dt[4];
      if (kb == 0) swam_read_tr_block<0>(lds + sb[j] + REGION, L, dt); else swam_read_tr_block<1>(lds + sb[j] + REGION, L, dt);
#pragma unroll
      for (int d = 0; d < 4; d++) r.dv[d] = Mma<CT>::mfma(dt[d], pb, r.dv[d]);
      u32x4 qt[4];
      if (kb == 0) swam_read_tr_block<0>(lds + sb[j], L, qt); else swam_read_tr_block<1>(lds + sb[j], L, qt);
#pragma unroll
      for (int d = 0; d < 4; d++) r.dk[d] = Mma<CT>::mfma(qt[d], dsb, r.dk[d]);
    }
    return r;
  };
  auto scratch_of = [&](int s) -> char* {
    const int c_new = 2 * s + 5;
    return smem + ((2 * s) % SWAM_NSLOT) * SLOT + ((c_new & 1) == kpar ? 0 : REGION) + 32 * (wave & 3) * 128;
  };
  auto store_grads = [&](const Out& r, int s, const int32_t (&id)[2]) {
    const int r_p = G.r0 + 8 * s + 4 * rg;
    int tok[2];
#pragma unroll
    for (int it = 0; it < 2; it++) tok[it] = swam_own_tok(G, r_p, c_p, (lane >> 3) + 8 * it);
    SwamTab tb[2];
    if (ROT) swam_store_tabs<TL>(tb, id, lane, rope, tabs);
    u32x4 v[2], pv[2], w[2], unused[2];
    swam_tile_transpose<CT, false>(scratch_of(s), r.dv, 1.0f, lane, w, unused);
    swam_tile_transpose<CT, ROT>(scratch_of(s), r.dk, sm_scale, lane, v, pv);
    if (ROT) {
#pragma unroll
      for (int it = 0; it < 2; it++) swam_rotate_piece<CT>(v[it], pv[it], tb[it], lane & 7, true);
    }
    swam_store_rows<TIO>(dvb, dvs2, tok, lane, w);
    swam_store_rows<TIO>(dkb, dks2, tok, lane, v);
  };

  for (int s = 0; s + 1 < G.nstep; s++) {
    SwamItem ia, ib;
    swam_issue(ia, st, G, 2 * s + 5, side[1]);
    swam_issue(ib, st, G, 2 * s + 6, side[0]);
    const float sc = scalar_issue(2 * s + 6 - kpar);   // the Q chunk among the two: 2 s + 5 (odd) or 2 s + 6 (even)
    Own nxt;
    own_issue(nxt, G.r0 + 8 * (s + 1) + 4 * rg);
    int32_t id[2] = {-1, -1};
    if (ROT) store_ids(id, s);
    const Out r = step(s);
    __syncthreads();
    swam_pin(ia);
    swam_pin(ib);
    pin_loaded(sc);
    own_pin(nxt);
    if (ROT) asm volatile("" ::"v"(id[0]), "v"(id[1]));
    store_grads(r, s, id);
    commit_chunk(ia, 2 * s + 5);
    commit_chunk(ib, 2 * s + 6);
    scalar_commit(sc, 2 * s + 6 - kpar);
    cur = nxt;
    own_negate_v(cur);
    __syncthreads();
  }
  {
    const int s = G.nstep - 1;
    int32_t id[2] = {-1, -1};
    if (ROT) store_ids(id, s);
    const Out r = step(s);
    __syncthreads();
    store_grads(r, s, id);
  }
}
