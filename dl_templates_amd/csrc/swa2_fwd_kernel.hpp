// Forward kernel for token grids at head dim 64 / 128 (b_size == 1, no rotation): replaces tiled_swa_fwd_kernel
// (src/tiled_swa.py:15-133).  Structure in swa2_common.hpp; per chunk a wave
//   1. computes S^T = K Q^T for its NCG column groups of 4 x 4 keys, masked to -inf outside the window,
//   2. runs one online-softmax update on the raw scores (p = exp2((s - m) scale)),
//   3. accumulates O^T += V^T P^T; the row sums come from one extra MFMA against a row of ones.
#pragma once
#include "swa2_common.hpp"

struct Swa2FwdArgs {
  AttnProblem p;
  Swa2Plan plan;
  const void *q, *k, *v;
  void* o;
  float* lse;
  int64_t qs[4], ks[4], vs[4], os[4], ls[3];
  float scale_log2;
};

// waves per SIMD the register budget is sized for: at head dim 64 two workgroups share a CU
constexpr int swa2_occ_fwd(int D) { return D == 64 ? 4 : 2; }

template <typename TIO, int D, int NCG>
__global__ __launch_bounds__(SWA2_THREADS, swa2_occ_fwd(D)) void swa2_fwd_kernel(const Swa2FwdArgs a) {
  typedef typename ComputeOf<TIO>::type CT;
  typedef Swa2Cfg<D, NCG> C;
  constexpr int KC = C::KC, VB = C::VB, NKB = C::NKB;
  constexpr int NG = VB / 4;   // groups of four 16-dim blocks of the output
  extern __shared__ __align__(16) char smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63, n = lane & 15, g = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int pc = wave & 3, rg = wave >> 2;
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
  // column pass 0 (the only one unless the window is wider than the class: swa2_pass_geom)
  Swa2Geom G = G0;
  Swa2Stage<C> st;
  swa2_stage_init(st, G, wave, lane, ssn2);
  swa2_issue(st, G, G.ch_first, sbase, srow, smem + (G.ch_first & 1) * C::BUF, wave);

  // own queries straight into B-operand fragments: lane (n, g) holds head dims 32 c + 8 g .. + 7 of query n
  const int r_p = G.r0 + 4 * rg, c_p = G.c0 + 4 * pc;
  const int tq = (r_p + (n >> 2) < G.TR && c_p + (n & 3) < G.TC) ? (r_p + (n >> 2)) * G.TC + c_p + (n & 3) : -1;
  u32x4 qf[KC];
  swa2_own_frags<KC>(qf, qb, (int)a.qs[2] * 2, tq, g);
  const Swa2Win W0 = swa2_window(G0, rg, pc, n);
  Swa2Win W = W0;
  Swa2Lane<C> L;
  swa2_lane_init(L, pc, n, g);

  float m_run = -INFINITY;
  f32x4 acc[VB], acc_l = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int d = 0; d < VB; d++) acc[d] = f32x4{0.f, 0.f, 0.f, 0.f};
  const unsigned one2 = pack2<CT>(1.f, 1.f);
  const u32x4 ones = n == 0 ? u32x4{one2, one2, one2, one2} : u32x4{0u, 0u, 0u, 0u};
  int ncg = swa2_pass_ncg(G0.WC, NCG, 0);   // column groups of the wave window that can hold a visible token

  swa2_wait_copies();   // also: the own fragments have arrived
  // the compiler does not see that wait: tell it that the own fragments are loaded, or it waits for them (and with them
  // for every copy in flight) at their first use inside every round of the chunk loop
  pin_loaded(qf);
  __syncthreads();

  // `cur` (the chunk being read) and `nxt` (the buffer the next chunk is copied into) are distinct buffers: the restrict
  // qualifiers let the compiler see that the operand reads do not depend on the copies in flight, so that it does not
  // wait for those in front of every LDS read
  auto consume = [&](const int ch, Swa2Lds __restrict__ cur, char* __restrict__ nxt, auto more_tag) {
    constexpr bool more = decltype(more_tag)::value;   // a later chunk exists: its copies are issued between the products
    Swa2Lds sK = cur;
    Swa2Lds sV = sK + C::REGION;
    const char* nrow = swa2_issue_row(G, ch + 1, sbase, srow, wave);
    char* ndst = swa2_issue_dst<C>(nxt, wave);
    const int hrow = 4 * ch + g;
    const bool row_vis = (hrow >= W.rlo) & (hrow <= W.rhi);
    // ---- scores of the chunk, one column group (16 keys) at a time.  Per group: the operands of the next group are
    //      requested, one copy instruction of the next chunk is issued, and the products of this group are issued
    //      with the masking and the running maxima of the previous group between them.
    float t[NKB][8];
    float mx[4] = {-INFINITY, -INFINITY, -INFINITY, -INFINITY};
    u32x4 ka[2][KC];
    f32x4 sc[2];
    auto mask_max = [&](const int cg, const f32x4& sv) {
      const int kb = cg >> 1, h4 = 4 * (cg & 1);
#pragma unroll
      for (int i = 0; i < 4; i++) t[kb][h4 + i] = swa2_visible(W, row_vis, cg, i, ncg) ? sv[i] : -INFINITY;
      mx[cg & 3] = fmaxf(fmaxf(mx[cg & 3], t[kb][h4]), t[kb][h4 + 1]);
      mx[(cg + 2) & 3] = fmaxf(fmaxf(mx[(cg + 2) & 3], t[kb][h4 + 2]), t[kb][h4 + 3]);
    };
    swa2_read_a<C, 0>(sK, L, ka[0]);
    swa2_for<0, NCG>([&](auto cgc) {
      constexpr int cg = decltype(cgc)::value;
      if constexpr (more) swa2_issue_one<C, cg>(st, nrow, ndst);
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (cg + 1 < NCG) swa2_read_a<C, cg + 1>(sK, L, ka[(cg + 1) & 1]);
      __builtin_amdgcn_sched_barrier(0);
      f32x4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int c = 0; c < KC; c++) s = Mma<CT>::mfma(ka[cg & 1][c], qf[c], s);
      sc[cg & 1] = s;
      if constexpr (cg > 0) mask_max(cg - 1, sc[(cg - 1) & 1]);
      SWA2_MIX(KC, 8 / KC)
      __builtin_amdgcn_sched_barrier(0);
    });
    mask_max(NCG - 1, sc[(NCG - 1) & 1]);
    // The reference maximum m_run only moves when some score exceeds it by more than 2^8 after scaling: p then stays
    // below 2^8, well inside the range of the 16-bit operand and of the fp32 sums, and the rescaling of the
    // accumulators is skipped for most chunks.  o and lse do not depend on which reference was used.
    const float mloc = wave_max4(fmaxf(fmaxf(mx[0], mx[1]), fmaxf(mx[2], mx[3])));
    if (__builtin_amdgcn_ballot_w64((mloc - m_run) * scale > 8.f)) {
      keep_branch();
      const float m_new = fmaxf(m_run, mloc);
      // a lane that has not seen a key yet keeps its (zero) accumulators as they are: with column passes, or with tiles of
      // several tokens, a query's first keys may lie in a later pass than those of the lane that triggers the update
      const float alpha = m_new == -INFINITY ? 1.f : fast_exp2((m_run - m_new) * scale);
      m_run = m_new;
#pragma unroll
      for (int d = 0; d < VB; d++) acc[d] *= alpha;
      acc_l *= alpha;
    }
    const float neg_m2 = m_run == -INFINITY ? 0.f : -m_run * scale;
    // ---- O^T += V^T P^T, 32 keys (two column groups) at a time: V^T fragments are requested four at a time, one
    //      group ahead of their products, and the exponentials of the next 32 keys are issued between the products
    u32x4 va[2][4];
    u32x4 pb[2];
    auto probs = [&](const int kb, const int half, u32x4& out) {   // half 0: elements 0-3 -> out.x, out.y; half 1: 4-7
#pragma unroll
      for (int i = 4 * half; i < 4 * half + 4; i++) t[kb][i] = fast_exp2(fmaf(t[kb][i], scale, neg_m2));
      if (half == 0) { out.x = pack2<CT>(t[kb][0], t[kb][1]); out.y = pack2<CT>(t[kb][2], t[kb][3]); }
      else { out.z = pack2<CT>(t[kb][4], t[kb][5]); out.w = pack2<CT>(t[kb][6], t[kb][7]); }
    };
    swa2_read_tr<C, 0, 0, 4>(sV, L, va[0]);
    probs(0, 0, pb[0]);
    probs(0, 1, pb[0]);
    swa2_for<0, NKB * NG>([&](auto ic) {
      constexpr int i = decltype(ic)::value, kb = i / NG, grp = i % NG;
      if constexpr (more) swa2_issue_one<C, NCG + i>(st, nrow, ndst);
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (i + 1 < NKB * NG) swa2_read_tr<C, (i + 1) / NG, 4 * ((i + 1) % NG), 4>(sV, L, va[(i + 1) & 1]);
      __builtin_amdgcn_sched_barrier(0);
      const u32x4 pk = pb[kb & 1];
#pragma unroll
      for (int d = 0; d < 4; d++) acc[4 * grp + d] = Mma<CT>::mfma(va[i & 1][d], pk, acc[4 * grp + d]);
      if constexpr (grp == NG - 1) acc_l = Mma<CT>::mfma(ones, pk, acc_l);
      if constexpr (kb + 1 < NKB) {
        if constexpr (NG == 2) probs(kb + 1, grp, pb[(kb + 1) & 1]);
        else { probs(kb + 1, 0, pb[(kb + 1) & 1]); probs(kb + 1, 1, pb[(kb + 1) & 1]); }
      }
      SWA2_MIX(grp == NG - 1 ? 5 : 4, NG == 2 ? (grp == 0 ? 3 : 2) : 5)
      __builtin_amdgcn_sched_barrier(0);
    });
  };

  // Every wave runs ch_last - ch_first rounds of (work, wait for its copies, workgroup barrier).  The chunks that hold
  // visible rows of its patch are contiguous; the rounds before and after them only copy.  Three loops instead of one
  // with a branch keep the accumulators in place (a branch inside the loop had them copied on every round).
  const int act_lo = dlt_imax(G.ch_first, W.ch_lo), act_hi = dlt_imin(G.ch_last - 1, W.ch_hi);
  auto copy_only = [&](int ch) {
    swa2_issue(st, G, ch + 1, sbase, srow, smem + ((ch + 1) & 1) * C::BUF, wave);
    swa2_wait_copies();
    __syncthreads();
  };
  for (int pass = 0;;) {
    int ch = G.ch_first;
    for (; ch < G.ch_last && ch < act_lo; ch++) copy_only(ch);
    for (; ch <= act_hi; ch++) {
      consume(ch, (Swa2Lds)smem + (ch & 1) * C::BUF, smem + ((ch + 1) & 1) * C::BUF, std::true_type{});
      swa2_wait_copies();
      __syncthreads();
    }
    for (; ch < G.ch_last; ch++) copy_only(ch);
    if (G.ch_last >= W.ch_lo && G.ch_last <= W.ch_hi)
      consume(G.ch_last, (Swa2Lds)smem + (G.ch_last & 1) * C::BUF, smem + ((G.ch_last + 1) & 1) * C::BUF, std::false_type{});
    __syncthreads();   // every wave is done with both chunk buffers
    if (++pass >= a.plan.npass) break;
    // next column pass: the same rows again, 4 NCG columns further to the right
    G = swa2_pass_geom(G0, NCG, pass);
    W = swa2_pass_window(W0, NCG, pass);
    ncg = swa2_pass_ncg(G0.WC, NCG, pass);
    swa2_stage_init(st, G, wave, lane, ssn2);
    swa2_issue(st, G, G.ch_first, sbase, srow, smem + (G.ch_first & 1) * C::BUF, wave);
    swa2_wait_copies();
    __syncthreads();
  }

  // ---- epilogue (the loop ended with a barrier: the chunk buffers are free)
  const float lt = wave_sum4(acc_l[0]);   // only row 0 of the ones operand is set: the other lane groups hold zeros
  const float inv = lt > 0.f ? fast_rcp(lt) : 0.f;
  if (g == 0 && tq >= 0) store_stream4(lseb + (int64_t)tq * ls2, m_run * scale + fast_log2(lt));
  swa2_store_own<C, TIO, CT>(smem + wave * C::TILE, acc, inv, ob, os2, G, r_p, c_p, lane);
}
