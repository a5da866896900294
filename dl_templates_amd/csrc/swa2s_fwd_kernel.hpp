// Forward kernel for token grids at head dim 128 (b_size == 1, no rotation), two stacked patches per wave: the work of
// tiled_swa_fwd_kernel (src/tiled_swa.py:15-133) on the streaming structure of swa2_common.hpp with a band of 16 grid
// rows per workgroup.  Wave w owns the 4x4 patches at rows 8 (w >> 2) and 8 (w >> 2) + 4, columns 4 (w & 3): both see the
// same window columns, so every K fragment read from LDS feeds the score products of both patches and every V^T
// fragment both output products (two matrix instructions per operand read instead of one), and the two independent
// product chains fill each other's latencies.  A halo row is staged once per 16 own rows.  Scores, maxima and output
// products are those of swa2_fwd_kernel in the same order; the row sums are taken with two-element dot products on the
// vector pipe (fp32 accumulation of the rounded probabilities, summed in another order than the matrix instruction of
// swa2_fwd_kernel does), which frees the registers of that instruction's operands and accumulators: 253 registers at
// 6 column groups, none spilled.
#pragma once
#include "swa2_fwd_kernel.hpp"

template <typename TIO, int D, int NCG>
__global__ __launch_bounds__(SWA2_THREADS, 2) void swa2s_fwd_kernel(const Swa2FwdArgs a) {
  typedef typename ComputeOf<TIO>::type CT;
  typedef Swa2Cfg<D, NCG> C;
  constexpr int KC = C::KC, VB = C::VB, NKB = C::NKB;
  constexpr int NG = VB / 4;   // groups of four 16-dim blocks of the output
  extern __shared__ __align__(16) char smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63, n = lane & 15, g = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int pc = wave & 3, rp = wave >> 2;
  const Swa2Geom G0 = swa2_geom(a.p, a.plan);

  const char* qb = reinterpret_cast<const char*>(a.q) + 2 * (G0.b * a.qs[0] + G0.h * a.qs[1]);
  const char* kb_ = reinterpret_cast<const char*>(a.k) + 2 * (G0.b * a.ks[0] + G0.h * a.ks[1]);
  const char* vb_ = reinterpret_cast<const char*>(a.v) + 2 * (G0.b * a.vs[0] + G0.h * a.vs[1]);
  TIO* ob = reinterpret_cast<TIO*>(a.o) + G0.b * a.os[0] + G0.h * a.os[1];
  float* lseb = a.lse + G0.b * a.ls[0] + G0.h * a.ls[1];
  const int64_t os2 = a.os[2], ls2 = a.ls[2];
  const float scale = a.scale_log2;

  // staging: waves 0-3 copy the four halo rows of K, waves 4-7 those of V
  const bool stage_k = wave < 4;
  const char* sbase = stage_k ? kb_ : vb_;
  const int ssn2 = (int)(stage_k ? a.ks[2] : a.vs[2]) * 2;
  const uint32_t srow = (uint32_t)(G0.TC * ssn2);
  Swa2Geom G = G0;   // column pass 0
  Swa2Stage<C> st;
  swa2_stage_init(st, G, wave, lane, ssn2);
  swa2_issue(st, G, G.ch_first, sbase, srow, smem + (G.ch_first & 1) * C::BUF, wave);

  // own queries of both patches straight into B-operand fragments
  const int c_p = G.c0 + 4 * pc;
  int r_p[2], tq[2];
  u32x4 qf[2][KC];
  Swa2Win W0[2], W[2];
#pragma unroll
  for (int p = 0; p < 2; p++) {
    r_p[p] = G.r0 + 4 * (2 * rp + p);
    tq[p] = (r_p[p] + (n >> 2) < G.TR && c_p + (n & 3) < G.TC) ? (r_p[p] + (n >> 2)) * G.TC + c_p + (n & 3) : -1;
    swa2_own_frags<KC>(qf[p], qb, (int)a.qs[2] * 2, tq[p], g);
    W0[p] = swa2_window(G0, 2 * rp + p, pc, n);
    W[p] = W0[p];
  }
  Swa2Lane<C> L;
  swa2_lane_init(L, pc, n, g);

  float m_run[2] = {-INFINITY, -INFINITY};
  f32x4 acc[2][VB];
  float lsum[2] = {0.f, 0.f};   // per lane: sum of the probabilities of its own token over the halo rows g of every chunk
#pragma unroll
  for (int p = 0; p < 2; p++) {
#pragma unroll
    for (int d = 0; d < VB; d++) acc[p][d] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  const unsigned one2 = pack2<CT>(1.f, 1.f);
  int ncg = swa2_pass_ncg(G0.WC, NCG, 0);

  swa2_wait_copies();   // also: the own fragments have arrived
  pin_loaded(qf);
  __syncthreads();

  // PM: the patches that see rows of the chunk (bit 0: the upper patch, bit 1: the lower one).  The chunks of a wave come
  // in the order "upper only" (at most one), "both", "lower only" (at most one); the one-patch bodies issue no product,
  // mask, exponential or reduction for the other patch.
  auto consume = [&](const int ch, Swa2Lds __restrict__ cur, char* __restrict__ nxt, auto more_tag, auto pm_tag) {
    constexpr bool more = decltype(more_tag)::value;   // a later chunk exists: its copies are issued between the products
    constexpr int PM = decltype(pm_tag)::value;
    constexpr bool P0 = (PM & 1) != 0, P1 = (PM & 2) != 0;
    Swa2Lds sK = cur;
    Swa2Lds sV = sK + C::REGION;
    const char* nrow = swa2_issue_row(G, ch + 1, sbase, srow, wave);
    char* ndst = swa2_issue_dst<C>(nxt, wave);
    const int hrow = 4 * ch + g;
    // both patches see the same window columns (the test of patch 0 serves both: its rows lie above those of patch 1, so
    // wherever the own token of patch 1 is inside the grid that of patch 0 is too); a patch row outside the grid is
    // folded into the row test
    const bool row_vis[2] = {(hrow >= W[0].rlo) && (hrow <= W[0].rhi), (hrow >= W[1].rlo) && (hrow <= W[1].rhi) && W[1].cspan >= 0};
    // ---- scores of the chunk, one column group (16 keys) at a time
    float t[2][NKB][8];
    float mx[2][4];
#pragma unroll
    for (int p = 0; p < 2; p++)
#pragma unroll
      for (int i = 0; i < 4; i++) mx[p][i] = -INFINITY;
    u32x4 ka[KC];
    f32x4 sc[2][2];
    auto mask_max = [&](const int p, const int cg, const f32x4& sv) {
      const int kb = cg >> 1, h4 = 4 * (cg & 1);
#pragma unroll
      for (int i = 0; i < 4; i++) t[p][kb][h4 + i] = swa2_visible(W[0], row_vis[p], cg, i, ncg) ? sv[i] : -INFINITY;
      mx[p][cg & 3] = fmaxf(fmaxf(mx[p][cg & 3], t[p][kb][h4]), t[p][kb][h4 + 1]);
      mx[p][(cg + 2) & 3] = fmaxf(fmaxf(mx[p][(cg + 2) & 3], t[p][kb][h4 + 2]), t[p][kb][h4 + 3]);
    };
    // K fragments live in ONE set of registers: piece c of the next group is requested as soon as the products of piece c
    // of this group are issued (with two patches every fragment feeds two products, so one group of read-ahead covers
    // the LDS latency)
    swa2_read_a<C, 0>(sK, L, ka);
    swa2_for<0, NCG>([&](auto cgc) {
      constexpr int cg = decltype(cgc)::value;
      if constexpr (more) swa2_issue_one<C, cg>(st, nrow, ndst);
      __builtin_amdgcn_sched_barrier(0);
      f32x4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int c = 0; c < KC; c++) {
        if constexpr (P0) s0 = Mma<CT>::mfma(ka[c], qf[0][c], s0);
        if constexpr (P1) s1 = Mma<CT>::mfma(ka[c], qf[1][c], s1);
        if constexpr (cg > 0) {
          if (P0 && c == 1) mask_max(0, cg - 1, sc[0][(cg - 1) & 1]);
          if (P1 && c == KC - 1) mask_max(1, cg - 1, sc[1][(cg - 1) & 1]);
        }
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (cg + 1 < NCG) ka[c] = swa2_lds16(sK + swa2_read_a_off<C, cg + 1>(L, c));
        __builtin_amdgcn_sched_barrier(0);
      }
      if constexpr (P0) sc[0][cg & 1] = s0;
      if constexpr (P1) sc[1][cg & 1] = s1;
    });
    if constexpr (P0) mask_max(0, NCG - 1, sc[0][(NCG - 1) & 1]);
    if constexpr (P1) mask_max(1, NCG - 1, sc[1][(NCG - 1) & 1]);
    // reference maxima move only when some score exceeds them by more than 2^8 after scaling (see swa2_fwd_kernel)
    float mloc[2] = {-INFINITY, -INFINITY};
    if constexpr (P0) mloc[0] = wave_max4(fmaxf(fmaxf(mx[0][0], mx[0][1]), fmaxf(mx[0][2], mx[0][3])));
    if constexpr (P1) mloc[1] = wave_max4(fmaxf(fmaxf(mx[1][0], mx[1][1]), fmaxf(mx[1][2], mx[1][3])));
    swa2_for<0, 2>([&](auto pc_) {
      constexpr int p = decltype(pc_)::value;
      if constexpr ((PM >> p) & 1) {
        if (__builtin_amdgcn_ballot_w64((mloc[p] - m_run[p]) * scale > 8.f)) {
          keep_branch();
          const float m_new = fmaxf(m_run[p], mloc[p]);
          // a lane that has not seen a key yet keeps its (zero) accumulators as they are
          const float alpha = m_new == -INFINITY ? 1.f : fast_exp2((m_run[p] - m_new) * scale);
          m_run[p] = m_new;
#pragma unroll
          for (int d = 0; d < VB; d++) acc[p][d] *= alpha;
          lsum[p] *= alpha;
        }
      }
    });
    const float neg_m2[2] = {m_run[0] == -INFINITY ? 0.f : -m_run[0] * scale, m_run[1] == -INFINITY ? 0.f : -m_run[1] * scale};
    // ---- O^T += V^T P^T, 32 keys at a time: with two patches every V^T fragment feeds two products
    u32x4 va[4];
    u32x4 pb[2][2];
    // V^T fragments live in one set of registers too: fragment d of the next step is requested behind the products of
    // fragment d of this step
    auto read_v = [&](auto ic, const int d) {
      constexpr int i = decltype(ic)::value, kb = i / NG, grp = i % NG;
      const u32x2 lo = swa2_lds_tr(sV + swa2_read_tr_off<C, kb>(L, 4 * grp + d, 0));
      const u32x2 hi = swa2_lds_tr(sV + swa2_read_tr_off<C, kb>(L, 4 * grp + d, 1));
      va[d].x = lo.x; va[d].y = lo.y; va[d].z = hi.x; va[d].w = hi.y;
    };
    // probability of element e (0 .. 7) of block kb for the active patches; the pair (e - 1, e) is packed behind odd e
    auto prob = [&](const int kb, const int e) {
#pragma unroll
      for (int p = 0; p < 2; p++)
        if ((PM >> p) & 1) {
          t[p][kb][e] = fast_exp2(fmaf(t[p][kb][e], scale, neg_m2[p]));
          if (e & 1) pb[p][kb & 1][e >> 1] = pack2<CT>(t[p][kb][e - 1], t[p][kb][e]);
        }
    };
#pragma unroll
    for (int d = 0; d < 4; d++) read_v(std::integral_constant<int, 0>{}, d);
#pragma unroll
    for (int e = 0; e < 8; e++) prob(0, e);
    swa2_for<0, NKB * NG>([&](auto ic) {
      constexpr int i = decltype(ic)::value, kb = i / NG, grp = i % NG;
      if constexpr (more) swa2_issue_one<C, NCG + i>(st, nrow, ndst);
      __builtin_amdgcn_sched_barrier(0);
      const u32x4 pk0 = pb[0][kb & 1], pk1 = pb[1][kb & 1];
#pragma unroll
      for (int d = 0; d < 4; d++) {
        if constexpr (P0) acc[0][4 * grp + d] = Mma<CT>::mfma(va[d], pk0, acc[0][4 * grp + d]);
        if constexpr (P1) acc[1][4 * grp + d] = Mma<CT>::mfma(va[d], pk1, acc[1][4 * grp + d]);
        if constexpr (kb + 1 < NKB) {
          // the exponentials of the next 32 keys, EPS elements per patch behind every fragment's products
          constexpr int EPS = 2 / NG;
#pragma unroll
          for (int e = (4 * grp + d) * EPS; e < (4 * grp + d + 1) * EPS; e++) prob(kb + 1, e);
        }
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (i + 1 < NKB * NG) read_v(std::integral_constant<int, i + 1>{}, d);
        __builtin_amdgcn_sched_barrier(0);
      }
      if constexpr (grp == NG - 1) {
        // row sums of the rounded probabilities (the values the products above use)
#pragma unroll
        for (int j = 0; j < 4; j++) {
          if constexpr (P0) lsum[0] = dot2_acc<CT>(pk0[j], one2, lsum[0]);
          if constexpr (P1) lsum[1] = dot2_acc<CT>(pk1[j], one2, lsum[1]);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    });
  };

  // Chunk ranges of the two patches (a patch outside the grid has an empty range; the lower patch starts and ends at or
  // after the upper one, and their ranges touch or overlap): upper only, both, lower only.  One loop per kind, in that
  // order, and copy-only rounds before and after, keep the accumulators in place (see swa2_fwd_kernel).
  const bool ok1 = W[1].ch_lo <= W[1].ch_hi;
  const int a_lo = W[0].ch_lo, a_hi = W[0].ch_hi;
  const int b_lo = ok1 ? W[1].ch_lo : a_hi + 1, b_hi = ok1 ? W[1].ch_hi : a_hi;
  const int w_lo = a_lo;
  const int both_lo = dlt_imax(a_lo, b_lo), both_hi = dlt_imin(a_hi, b_hi);
  auto copy_only = [&](int ch) {
    swa2_issue(st, G, ch + 1, sbase, srow, smem + ((ch + 1) & 1) * C::BUF, wave);
    swa2_wait_copies();
    __syncthreads();
  };
  auto round = [&](int ch, auto pm_tag) {
    consume(ch, (Swa2Lds)smem + (ch & 1) * C::BUF, smem + ((ch + 1) & 1) * C::BUF, std::true_type{}, pm_tag);
    swa2_wait_copies();
    __syncthreads();
  };
  typedef std::integral_constant<int, 1> PmUpper;
  typedef std::integral_constant<int, 2> PmLower;
  typedef std::integral_constant<int, 3> PmBoth;
  for (int pass = 0;;) {
    int ch = G.ch_first;
    for (; ch < G.ch_last && ch < w_lo; ch++) copy_only(ch);
    for (; ch < G.ch_last && ch <= a_hi && ch < both_lo; ch++) round(ch, PmUpper{});
    for (; ch < G.ch_last && ch <= both_hi; ch++) round(ch, PmBoth{});
    for (; ch < G.ch_last && ch <= b_hi; ch++) round(ch, PmLower{});
    for (; ch < G.ch_last; ch++) copy_only(ch);
    {
      const int cl = G.ch_last;
      const bool in0 = cl >= a_lo && cl <= a_hi, in1 = ok1 && cl >= b_lo && cl <= b_hi;
      Swa2Lds cur = (Swa2Lds)smem + (cl & 1) * C::BUF;
      char* nxt = smem + ((cl + 1) & 1) * C::BUF;
      if (in0 && in1) consume(cl, cur, nxt, std::false_type{}, PmBoth{});
      else if (in0) consume(cl, cur, nxt, std::false_type{}, PmUpper{});
      else if (in1) consume(cl, cur, nxt, std::false_type{}, PmLower{});
    }
    __syncthreads();   // every wave is done with both chunk buffers
    if (++pass >= a.plan.npass) break;
    G = swa2_pass_geom(G0, NCG, pass);
    W[0] = swa2_pass_window(W0[0], NCG, pass);
    W[1] = swa2_pass_window(W0[1], NCG, pass);
    ncg = swa2_pass_ncg(G0.WC, NCG, pass);
    swa2_stage_init(st, G, wave, lane, ssn2);
    swa2_issue(st, G, G.ch_first, sbase, srow, smem + (G.ch_first & 1) * C::BUF, wave);
    swa2_wait_copies();
    __syncthreads();
  }

  // ---- epilogue (the loop ended with a barrier: the chunk buffers are free), one patch after the other
#pragma unroll
  for (int p = 0; p < 2; p++) {
    const float lt = wave_sum4(lsum[p]);
    const float inv = lt > 0.f ? fast_rcp(lt) : 0.f;
    if (g == 0 && tq[p] >= 0) store_stream4(lseb + (int64_t)tq[p] * ls2, m_run[p] * scale + fast_log2(lt));
    swa2_store_own<C, TIO, CT>(smem + wave * C::TILE, acc[p], inv, ob, os2, G, r_p[p], c_p, lane);
  }
}
