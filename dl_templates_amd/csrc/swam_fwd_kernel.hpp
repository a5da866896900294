// Marching forward kernel for token grids (b_size == 1, head dim 64, windows up to 13 x 13): the shape of the
// benchmark's headline configuration.  Replaces tiled_swa_fwd_kernel (src/tiled_swa.py:15-133): a 2D block of
// queries shares one K / V halo, here kept in an LDS ring that slides down the grid (swam_common.hpp).
//
// Per step a wave holds one 4x4 query patch and sees its whole window (up to 16 halo rows x 16 halo columns)
// in LDS at once, so the softmax is not an online one: all S^T = K Q^T blocks first, one row max, one
// exponential pass, then O^T += V^T P^T and the row sums through an MFMA against a row of ones.
#pragma once
#include "swam_common.hpp"

struct SwamFwdArgs {
  AttnProblem p;
  SwamPlan plan;
  const void *q, *k, *v;
  void* o;
  float* lse;
  int64_t qs[4], ks[4], vs[4], os[4], ls[3];
  void *q_rot, *k_rot;   // optional side outputs of the fused rotation (NULL: not stored)
  int64_t qrs[4], krs[4];
  float scale_log2;
};

struct SwamFwdOut { f32x4 acc[4]; float inv, lse2; };

// own-token B-operand fragments (head dim along k) in flight: lane (n, g) holds pieces g and 4 + g of token n
struct SwamOwn {
  u32x4 f[2];
  u32x4 partner;   // piece g ^ 1 (the rotary partner of piece g)
  int tok;         // token index inside the (batch, head) slab, -1: outside the grid
};

DLT_DEV int swam_own_tok(const SwamGeom& G, int r_p, int c_p, int n) {
  const int r = r_p + (n >> 2), c = c_p + (n & 3);
  return (r < G.TR && c < G.TC) ? r * G.TC + c : -1;
}

template <bool ROT>
DLT_DEV void swam_own_issue(SwamOwn& w, const char* base, int sn2, const SwamGeom& G, int r_p, int c_p, int n, int g) {
  w.tok = swam_own_tok(G, r_p, c_p, n);
  const int t = w.tok >= 0 ? w.tok : 0;
  const char* p = base + ((uint32_t)(t * sn2) + 16 * g);
  w.f[0] = *reinterpret_cast<const u32x4*>(p);
  w.f[1] = *reinterpret_cast<const u32x4*>(p + 64);
  if (ROT) w.partner = *reinterpret_cast<const u32x4*>(base + ((uint32_t)(t * sn2) + 16 * (g ^ 1)));
}

DLT_DEV void swam_own_pin(const SwamOwn& w, bool rot) {
  pin_loaded(w.f[0]);
  pin_loaded(w.f[1]);
  if (rot) pin_loaded(w.partner);
}

// rotate piece g of the own fragment (pieces 0, 1: row angle; 2, 3: column angle); `tb` = table row of axis g >> 1
template <typename CT>
DLT_DEV void swam_own_rotate(SwamOwn& w, const SwamTab& tb, int g, bool inverse) {
  if (!tb.rot) return;
  float self[8], partner[8];
  unpack8<CT>(w.f[0], self);
  unpack8<CT>(w.partner, partner);
  const unsigned sm = rope_sign_mask((g & 1) == 0, inverse);
#pragma unroll
  for (int j = 0; j < 8; j++)
    self[j] = rope_mix_signed(self[j], partner[j], tb.t[j >> 1][2 * (j & 1)], tb.t[j >> 1][2 * (j & 1) + 1], sm);
  w.f[0] = pack8<CT>(self);
}

// ROPE: 0 no rotation, 2 q and k rotated on their way in (k: between HBM and LDS, q: own fragments); TL: the rotary
// tables are copied into LDS (behind the ring) at kernel start and every table row is read from there
template <typename TIO, int ROPE, bool TL>
__global__ __launch_bounds__(SWAM_THREADS) void swam_fwd_kernel(const SwamFwdArgs a) {
  static_assert(!TL || ROPE != 0, "LDS tables only with rotation");
  typedef typename ComputeOf<TIO>::type CT;
  constexpr int D = 64;
  constexpr bool ROT = ROPE != 0;
  constexpr int REGION = swam_region(D), SLOT = swam_slot(D);
  extern __shared__ __align__(16) char smem[];
  SwamLds tabs = (SwamLds)(smem + swam_ring(D));

  const int tid = threadIdx.x;
  const int lane = tid & 63, n = lane & 15, g = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int pc = wave & 3, rg = wave >> 2;   // patch column, row group
  const SwamGeom G = swam_geom(a.p, a.plan);
  f32x4 tab16;
  if (TL) tab16 = swam_tab_fetch(a.p.rope, tid);   // first load of the kernel: the tables do not depend on any index

  const char* qb = reinterpret_cast<const char*>(a.q) + 2 * (G.b * a.qs[0] + G.h * a.qs[1]);
  const char* kb_ = reinterpret_cast<const char*>(a.k) + 2 * (G.b * a.ks[0] + G.h * a.ks[1]);
  const char* vb_ = reinterpret_cast<const char*>(a.v) + 2 * (G.b * a.vs[0] + G.h * a.vs[1]);
  TIO* ob = reinterpret_cast<TIO*>(a.o) + G.b * a.os[0] + G.h * a.os[1];
  float* lseb = a.lse + G.b * a.ls[0] + G.h * a.ls[1];
  const int sn2q = (int)a.qs[2] * 2;
  const int64_t os2 = a.os[2], ls2 = a.ls[2];
  const int32_t* rope_idx = ROT ? a.p.rope.idx : nullptr;
  const RopeDev rope = a.p.rope;
  const bool save_rot = ROT && a.k_rot != nullptr;
  TIO* qrb = save_rot ? reinterpret_cast<TIO*>(a.q_rot) + G.b * a.qrs[0] + G.h * a.qrs[1] : nullptr;
  char* krb = save_rot ? reinterpret_cast<char*>(a.k_rot) + 2 * (G.b * a.krs[0] + G.h * a.krs[1]) : nullptr;
  const int64_t qrs2 = a.qrs[2];
  const int sn2kr = (int)a.krs[2] * 2;
  const int band = a.plan.band;
  const float scale = a.scale_log2;

  SwamStage st;
  swam_stage_init(st, G, tid);
  // The lower half of the workgroup stages K of even chunks and V of odd ones, the upper half the reverse:
  // side[p] is the tensor this thread stages for chunks of parity p, kpar the parity for which that is K.
  const int hh = wave >> 2;
  const int kpar = hh;
  SwamSide side[2];
  {
    const SwamSide sk = swam_side(kb_, (int)a.ks[2] * 2, G, st), sv = swam_side(vb_, (int)a.vs[2] * 2, G, st);
    side[0] = kpar == 0 ? sk : sv;
    side[1] = kpar == 0 ? sv : sk;
  }
  SwamLane L;
  swam_lane_init(L, pc, n, g);
  const int c_p = G.c0 + 4 * pc;

  // fused rotation of a staged K item (table values in `tb`), and its store to k_rot when the token is the workgroup's own
  auto rotate_k = [&](SwamItem& it, const SwamTab& tb) {
    swam_rotate_pair<CT>(it.v[0], it.v[1], tb, false);
    if (save_rot && st.own_col && it.row >= G.r0 && it.row < G.r0 + band && it.row < G.TR) {
      char* p = krb + ((uint32_t)((it.row * G.TC + st.cc) * sn2kr) + 32 * st.qd);
      store_stream16(p, it.v[0]);
      store_stream16(p + 16, it.v[1]);
      store_stream16(p + 64, it.v[2]);
      store_stream16(p + 80, it.v[3]);
    }
  };
  auto rotate_q = [&](SwamOwn& w, const SwamTab& tb) {
    swam_own_rotate<CT>(w, tb, g, false);
    if (save_rot && w.tok >= 0) {
      TIO* qr = qrb + (int64_t)w.tok * qrs2;
      store_stream16(qr + 8 * g, w.f[0]);
      store_stream16(qr + 32 + 8 * g, w.f[1]);
    }
  };
  auto commit_chunk = [&](const SwamItem& it, int c) {
    swam_commit(it, st, smem + (c % SWAM_NSLOT) * SLOT + ((c & 1) == kpar ? 0 : REGION));
  };
  auto own_idx = [&](int r_p) -> int32_t {
    const int t = swam_own_tok(G, r_p, c_p, n);
    return rope_idx[t >= 0 ? t : 0];
  };

  // ---- prologue: the five chunks of step 0 and its own queries.  With rotation the token indices are requested first
  //      (also those of the next step's K chunk and queries, so that inside the loop the table rows can be requested
  //      together with the data), the table rows as soon as the indices are there.
  SwamOwn qo;
  int32_t idk_next = -1, idq_next = -1;   // rotary indices of the K item / own queries of the step after the current one
  {
    int32_t idk[3] = {-1, -1, -1}, idq = -1;
    if (ROT) {
#pragma unroll
      for (int i = 0; i < 3; i++)
        if (kpar + 2 * i < SWAM_NSLOT) idk[i] = swam_issue_idx(st, G, kpar + 2 * i, rope_idx);
      idq = own_idx(G.r0 + 4 * rg);
      idk_next = swam_issue_idx(st, G, 6 - kpar, rope_idx);   // chunk 5 (odd) or 6 (even)
      idq_next = own_idx(G.r0 + 8 + 4 * rg);
    }
    SwamItem it[SWAM_NSLOT];
#pragma unroll
    for (int c = 0; c < SWAM_NSLOT; c++) swam_issue(it[c], st, G, c, side[c & 1]);
    swam_own_issue<ROT>(qo, qb, sn2q, G, G.r0 + 4 * rg, c_p, n, g);
    SwamTab tb[3], tbq;
    if (TL) {
      // the tables into LDS (loads return in order: this one was requested first), visible to every wave after the barrier
      pin_loaded(tab16);
      swam_tab_store(smem + swam_ring(D), tid, tab16);
      __syncthreads();
    }
    if (ROT && !TL) {
#pragma unroll
      for (int i = 0; i < 3; i++)
        if (kpar + 2 * i < SWAM_NSLOT) swam_tab_issue(tb[i], idk[i], st.qd, rope);
      swam_tab_issue(tbq, idq, g >> 1, rope);
    }
    if (!ROT) {
      // chunk by chunk (loads return in order): the LDS writes of a chunk overlap the arrival of the later ones
#pragma unroll
      for (int c = 0; c < SWAM_NSLOT; c++) {
        swam_pin(it[c]);
        commit_chunk(it[c], c);
      }
    }
    if (ROT && TL) {
      // the tables are in LDS: chunk by chunk as the loads return, the K items rotated on their way
#pragma unroll
      for (int c = 0; c < SWAM_NSLOT; c++) {
        swam_pin(it[c]);
        if ((c & 1) == kpar) {
          swam_tab_get<true>(tb[0], idk[c >> 1], st.qd, rope, tabs);
          rotate_k(it[c], tb[0]);
        }
        commit_chunk(it[c], c);
      }
      swam_own_pin(qo, ROT);
      swam_tab_get<true>(tbq, idq, g >> 1, rope, tabs);
      rotate_q(qo, tbq);
    } else if (ROT) {
      // V chunks need no rotation and are written as they arrive; the K chunks wait for their table rows, which were
      // requested last (static register indexing: the K items of this half are chunks kpar, kpar + 2, kpar + 4)
      if (kpar == 0) {
        swam_pin(it[1]); commit_chunk(it[1], 1);
        swam_pin(it[3]); commit_chunk(it[3], 3);
      } else {
        swam_pin(it[0]); commit_chunk(it[0], 0);
        swam_pin(it[2]); commit_chunk(it[2], 2);
        swam_pin(it[4]); commit_chunk(it[4], 4);
      }
#pragma unroll
      for (int c = 0; c < SWAM_NSLOT; c++) swam_pin(it[c]);
      swam_own_pin(qo, ROT);
      if (kpar == 0) {
        rotate_k(it[0], tb[0]); commit_chunk(it[0], 0);
        rotate_k(it[2], tb[1]); commit_chunk(it[2], 2);
        rotate_k(it[4], tb[2]); commit_chunk(it[4], 4);
      } else {
        rotate_k(it[1], tb[0]); commit_chunk(it[1], 1);
        rotate_k(it[3], tb[1]); commit_chunk(it[3], 3);
      }
      rotate_q(qo, tbq);
    } else {
      swam_own_pin(qo, ROT);
    }
  }
  __syncthreads();

  const unsigned one2 = pack2<CT>(1.f, 1.f);
  const u32x4 ones = n == 0 ? u32x4{one2, one2, one2, one2} : u32x4{0u, 0u, 0u, 0u};
  const int qr_l = n >> 2, qc_l = n & 3;
  // column window of this lane's query in wave-window coordinates [clo, clo + cspan]; the same in every step
  const int clo = dlt_imax(qc_l, G.WC - c_p), chi = dlt_imin(qc_l + 2 * G.WC, G.TC - 1 - c_p + G.WC);

  // products and softmax of step s; `qo` holds the own queries (already rotated)
  SwamLds lds = (SwamLds)smem;
  auto step = [&](const int s) {
    const int r_p = G.r0 + 8 * s + 4 * rg;
    const u32x4 qf0 = qo.f[0], qf1 = qo.f[1];
    const bool q_ok = (r_p + qr_l < G.TR) && (c_p + qc_l < G.TC);
    const int rlo = dlt_imax(qr_l, G.WR - r_p), rhi = dlt_imin(qr_l + 2 * G.WR, G.TR - 1 - r_p + G.WR);
    const int cspan = q_ok ? chi - clo : -1;
    // LDS byte offsets of the window's chunks (wave-uniform)
    int sb[4];
    {
      const int s5 = (2 * s + rg) % SWAM_NSLOT;
#pragma unroll
      for (int j = 0; j < 4; j++) sb[j] = __builtin_amdgcn_readfirstlane((s5 + j >= SWAM_NSLOT ? s5 + j - SWAM_NSLOT : s5 + j) * SLOT);
    }
    // ---- S^T = K Q^T for the whole window, masked to -inf outside it; the A operands of the next chunk are
    //      requested before the products of the current one (two operand buffers, used alternately)
    float t[4][2][8];
    float mx[4] = {-INFINITY, -INFINITY, -INFINITY, -INFINITY};
    u32x4 ka[2][4];
    swam_read_a_half<0>(lds + sb[0], L, ka[0]);
#pragma unroll
    for (int b = 0; b < 8; b++) {
      const int j = b >> 1, kb = b & 1;
      if (b < 7) {
        if (kb == 0) swam_read_a_half<1>(lds + sb[j], L, ka[(b + 1) & 1]);
        else swam_read_a_half<0>(lds + sb[j < 3 ? j + 1 : 3], L, ka[(b + 1) & 1]);
      }
      __builtin_amdgcn_sched_barrier(0);
      const int hrow = 4 * j + g;
      const bool row_vis = (j < G.nch) & (hrow >= rlo) & (hrow <= rhi);
      const u32x4(&kc)[4] = ka[b & 1];
      f32x4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
      s0 = Mma<CT>::mfma(kc[0], qf0, s0);
      s1 = Mma<CT>::mfma(kc[2], qf0, s1);
      s0 = Mma<CT>::mfma(kc[1], qf1, s0);
      s1 = Mma<CT>::mfma(kc[3], qf1, s1);
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const bool v0 = row_vis & ((unsigned)(8 * kb + i - clo) <= (unsigned)cspan);
        const bool v1 = row_vis & ((unsigned)(8 * kb + 4 + i - clo) <= (unsigned)cspan);
        t[j][kb][i] = v0 ? s0[i] : -INFINITY;
        t[j][kb][4 + i] = v1 ? s1[i] : -INFINITY;
      }
      // four independent max chains, two new values per instruction
      mx[0] = fmaxf(fmaxf(mx[0], t[j][kb][0]), t[j][kb][1]);
      mx[1] = fmaxf(fmaxf(mx[1], t[j][kb][2]), t[j][kb][3]);
      mx[2] = fmaxf(fmaxf(mx[2], t[j][kb][4]), t[j][kb][5]);
      mx[3] = fmaxf(fmaxf(mx[3], t[j][kb][6]), t[j][kb][7]);
    }
    // exact row max of the raw scores (sm_scale > 0 keeps the order), p = exp2((s - m) * scale)
    const float mloc = wave_max4(fmaxf(fmaxf(mx[0], mx[1]), fmaxf(mx[2], mx[3])));
    const float m_use = mloc == -INFINITY ? 0.f : mloc;
    const float neg_m2 = -m_use * scale;
    f32x4 acc[4], acc_l = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int d = 0; d < 4; d++) acc[d] = f32x4{0.f, 0.f, 0.f, 0.f};
    // ---- O^T += V^T P^T, block by block; the V^T fragments of the next block are requested before the products
    u32x4 va[2][4];
    swam_read_tr_block<0>(lds + sb[0] + REGION, L, va[0]);
#pragma unroll
    for (int b = 0; b < 8; b++) {
      const int j = b >> 1, kb = b & 1;
      if (b < 7) {
        if (kb == 0) swam_read_tr_block<1>(lds + sb[j] + REGION, L, va[(b + 1) & 1]);
        else swam_read_tr_block<0>(lds + sb[j < 3 ? j + 1 : 3] + REGION, L, va[(b + 1) & 1]);
      }
#pragma unroll
      for (int i = 0; i < 8; i++) t[j][kb][i] = fast_exp2(fmaf(t[j][kb][i], scale, neg_m2));
      const u32x4 pb = pack8<CT>(t[j][kb]);
      __builtin_amdgcn_sched_barrier(0);
      const u32x4(&vc)[4] = va[b & 1];
#pragma unroll
      for (int d = 0; d < 4; d++) acc[d] = Mma<CT>::mfma(vc[d], pb, acc[d]);
      acc_l = Mma<CT>::mfma(ones, pb, acc_l);
    }
    // row 0 of the ones product (lane group 0) = sum over keys of P[key][query n]
    const float lt = wave_sum4(acc_l[0]);   // only row 0 of the ones operand is set: the other lane groups hold zeros
    SwamFwdOut r;
#pragma unroll
    for (int d = 0; d < 4; d++) r.acc[d] = acc[d];
    r.inv = lt > 0.f ? fast_rcp(lt) : 0.f;
    r.lse2 = m_use * scale + fast_log2(lt);
    return r;
  };
  // wave-private scratch for the store epilogue: the part of the oldest chunk's slot that this wave's own threads
  // overwrite at the next commit (LDS operations of one wave execute in order, so no barrier is needed between the two)
  auto scratch_of = [&](int s) -> char* {
    const int c_new = 2 * s + 5;   // the chunk that will replace chunk 2 s
    return smem + ((2 * s) % SWAM_NSLOT) * SLOT + ((c_new & 1) == kpar ? 0 : REGION) + 32 * (wave & 3) * 128;
  };
  // o of step s: accumulators -> 16-byte row pieces (through the wave's LDS scratch), then the stores
  struct OutRows { u32x4 v[2]; int tok[2]; };
  // The lane-derived addresses of the epilogue are computed from an opaque copy of the lane id: computed from `lane`
  // itself they are hoisted out of the step loop and then live (spilled to scratch) across the products.
  auto transpose_o = [&](const SwamFwdOut& r, int s) {
    OutRows w;
    const int r_p = G.r0 + 8 * s + 4 * rg;
    int ln = lane;
    asm volatile("" : "+v"(ln));
#pragma unroll
    for (int it = 0; it < 2; it++) w.tok[it] = swam_own_tok(G, r_p, c_p, (ln >> 3) + 8 * it);
    u32x4 unused[2];
    swam_tile_transpose<CT, false>(scratch_of(s), r.acc, r.inv, ln, w.v, unused);
    return w;
  };
  auto store_o = [&](const OutRows& w, const SwamFwdOut& r) {
    if (g == 0 && qo.tok >= 0) store_stream4(lseb + (int64_t)qo.tok * ls2, r.lse2);
    int ln = lane;
    asm volatile("" : "+v"(ln));
    swam_store_rows<TIO>(ob, os2, w.tok, ln, w.v);
  };

  // The last step is peeled off so that inside the loop prefetch and commit are unconditional (a conditional
  // prefetch leaves a path with loads pending across the back edge: every later wait becomes a full one).
  for (int s = 0; s + 1 < G.nstep; s++) {
    // chunks 2 s + 5 (odd) and 2 s + 6 (even) and the own queries of the next step; with rotation also the token
    // indices for the step after (the table rows are requested once the step's products are done: holding them in
    // registers across the products would not fit)
    SwamItem ia, ib;
    swam_issue(ia, st, G, 2 * s + 5, side[1]);
    swam_issue(ib, st, G, 2 * s + 6, side[0]);
    SwamOwn qn;
    swam_own_issue<ROT>(qn, qb, sn2q, G, G.r0 + 8 * (s + 1) + 4 * rg, c_p, n, g);
    int32_t idk_nn = -1, idq_nn = -1;
    if (ROT) {
      idk_nn = swam_issue_idx(st, G, 2 * s + 8 - kpar, rope_idx);
      idq_nn = own_idx(G.r0 + 8 * (s + 2) + 4 * rg);
    }
    const SwamFwdOut r = step(s);
    __syncthreads();   // every wave is done with the chunks of this step
    swam_pin(ia);
    swam_pin(ib);
    swam_own_pin(qn, ROT);
    SwamTab tbk, tbq;
    if (ROT) {
      asm volatile("" ::"v"(idk_nn), "v"(idq_nn));
      swam_tab_get<TL>(tbk, idk_next, st.qd, rope, tabs);
      swam_tab_get<TL>(tbq, idq_next, g >> 1, rope, tabs);
    }
    const OutRows w = transpose_o(r, s);   // LDS only: overlaps the table loads
    if (ROT) {
      if (kpar) rotate_k(ia, tbk); else rotate_k(ib, tbk);
      rotate_q(qn, tbq);
      idk_next = idk_nn;
      idq_next = idq_nn;
    }
    store_o(w, r);
    commit_chunk(ia, 2 * s + 5);
    commit_chunk(ib, 2 * s + 6);
    qo = qn;
    __syncthreads();
  }
  {
    const int s = G.nstep - 1;
    const SwamFwdOut r = step(s);
    __syncthreads();
    const OutRows w = transpose_o(r, s);
    store_o(w, r);
  }
}
