// Backward kernels for token grids at head dim 64 / 128 (b_size == 1, no rotation): the decoupled dQ and dK/dV passes
// of tiled_swa_bwd_large_kernel_decoupled_q (src/tiled_swa.py:407-562) on the streaming structure of swa2_common.hpp.
//
//   dQ   : a wave owns a 4x4 patch of queries; K and V stream through LDS.  It runs first and computes
//          delta = rowsum(o * dO) of its own queries on the way (the reference's pre-pass, src/tiled_swa.py:253-282),
//          which the dK/dV kernel reads back.
//   dK/dV: a wave owns a 4x4 patch of keys; Q and dO of the queries that can see them stream through LDS (the window
//          is symmetric), with their lse2 and delta in a small table behind each chunk.
// Both recompute P = exp2(s * scale - lse2) per 32 streamed tokens; streamed tokens are the MFMA rows of the first
// products, so P / dS leave them in the layout the second products take as B operand.
#pragma once
#include "swa2_fwd_kernel.hpp"

struct Swa2BwdArgs {
  AttnProblem p;
  Swa2Plan plan;
  const void *q, *k, *v, *o, *d_o;
  const float* lse;
  float* delta;   // written by the dQ kernel, read by the dK/dV kernel (strides of lse)
  void *dq, *dk, *dv;
  int64_t qs[4], ks[4], vs[4], os[4], dos[4], dqs[4], dks[4], dvs[4], ls[3];
  float scale_log2;
};

// waves per SIMD the register budget is sized for
constexpr int swa2_occ_bwd_q(int D) { return D == 64 ? 4 : 2; }
constexpr int swa2_occ_bwd_kv(int D) { return 2; }

// =============================================================================================== dQ
template <typename TIO, int D, int NCG>
__global__ __launch_bounds__(SWA2_THREADS, swa2_occ_bwd_q(D)) void swa2_bwd_q_kernel(const Swa2BwdArgs a) {
  typedef typename ComputeOf<TIO>::type CT;
  typedef Swa2Cfg<D, NCG> C;
  constexpr int KC = C::KC, VB = C::VB, NKB = C::NKB;
  constexpr int NG = VB / 4;   // groups of four 16-dim blocks of dQ
  extern __shared__ __align__(16) char smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63, n = lane & 15, g = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int pc = wave & 3, rg = wave >> 2;
  const Swa2Geom G0 = swa2_geom(a.p, a.plan);

  const char* qb = reinterpret_cast<const char*>(a.q) + 2 * (G0.b * a.qs[0] + G0.h * a.qs[1]);
  const char* kb_ = reinterpret_cast<const char*>(a.k) + 2 * (G0.b * a.ks[0] + G0.h * a.ks[1]);
  const char* vb_ = reinterpret_cast<const char*>(a.v) + 2 * (G0.b * a.vs[0] + G0.h * a.vs[1]);
  const char* ob = reinterpret_cast<const char*>(a.o) + 2 * (G0.b * a.os[0] + G0.h * a.os[1]);
  const char* dob = reinterpret_cast<const char*>(a.d_o) + 2 * (G0.b * a.dos[0] + G0.h * a.dos[1]);
  TIO* dqb = reinterpret_cast<TIO*>(a.dq) + G0.b * a.dqs[0] + G0.h * a.dqs[1];
  const float* lseb = a.lse + G0.b * a.ls[0] + G0.h * a.ls[1];
  float* delb = a.delta + G0.b * a.ls[0] + G0.h * a.ls[1];
  const float scale = a.scale_log2;

  // staging: waves 0-3 copy the four halo rows of K, waves 4-7 those of V
  const bool stage_k = wave < 4;
  const char* sbase = stage_k ? kb_ : vb_;
  const int ssn2 = (int)(stage_k ? a.ks[2] : a.vs[2]) * 2;
  const uint32_t srow = (uint32_t)(G0.TC * ssn2);
  Swa2Geom G = G0;   // column pass 0 (see the forward kernel)
  Swa2Stage<C> st;
  swa2_stage_init(st, G, wave, lane, ssn2);
  swa2_issue(st, G, G.ch_first, sbase, srow, smem + (G.ch_first & 1) * C::BUF, wave);

  const int r_p = G.r0 + 4 * rg, c_p = G.c0 + 4 * pc;
  const int tq = (r_p + (n >> 2) < G.TR && c_p + (n & 3) < G.TC) ? (r_p + (n >> 2)) * G.TC + c_p + (n & 3) : -1;
  u32x4 qf[KC], dof[KC];
  float neg_lse, del_n;
  {
    u32x4 of[KC];
    swa2_own_frags<KC>(qf, qb, (int)a.qs[2] * 2, tq, g);
    swa2_own_frags<KC>(dof, dob, (int)a.dos[2] * 2, tq, g);
    swa2_own_frags<KC>(of, ob, (int)a.os[2] * 2, tq, g);
    neg_lse = tq >= 0 ? -lseb[(int64_t)tq * a.ls[2]] : -INFINITY;
    // delta = rowsum(o * dO) of the own token: D / 4 head dims per lane, summed over the four lanes of the token
    float part = 0.f;
#pragma unroll
    for (int c = 0; c < KC; c++)
#pragma unroll
      for (int j = 0; j < 4; j++) {
        part = fmaf(unpack_lo<CT>(of[c][j]), unpack_lo<CT>(dof[c][j]), part);
        part = fmaf(unpack_hi<CT>(of[c][j]), unpack_hi<CT>(dof[c][j]), part);
      }
    del_n = wave_sum4(part);
    if (g == 0 && tq >= 0) store_stream4(delb + (int64_t)tq * a.ls[2], del_n);
  }
  const Swa2Win W0 = swa2_window(G0, rg, pc, n);
  Swa2Win W = W0;
  Swa2Lane<C> L;
  swa2_lane_init(L, pc, n, g);

  f32x4 acc[VB];
#pragma unroll
  for (int d = 0; d < VB; d++) acc[d] = f32x4{0.f, 0.f, 0.f, 0.f};
  int ncg = swa2_pass_ncg(G0.WC, NCG, 0);

  swa2_wait_copies();   // also: the own fragments have arrived
  // the compiler does not see that wait: tell it that the own fragments are loaded, or it waits for them (and with them
  // for every copy in flight) at their first use inside every round of the chunk loop
  pin_loaded(qf);
  pin_loaded(dof);
  pin_loaded(neg_lse);
  // the dP products start from -delta of the lane's query (the C operand): the matrix pipe delivers dP - delta
  const f32x4 dinit = {-del_n, -del_n, -del_n, -del_n};
  __syncthreads();

  // `cur` and `nxt` are distinct chunk buffers (see the forward kernel)
  auto consume = [&](const int ch, Swa2Lds __restrict__ cur, char* __restrict__ nxt, auto more_tag) {
    constexpr bool more = decltype(more_tag)::value;
    Swa2Lds sK = cur;
    Swa2Lds sV = sK + C::REGION;
    const char* nrow = swa2_issue_row(G, ch + 1, sbase, srow, wave);
    char* ndst = swa2_issue_dst<C>(nxt, wave);
    const int hrow = 4 * ch + g;
    const bool row_vis = (hrow >= W.rlo) & (hrow <= W.rhi);
    u32x4 xk[2][KC], xv[2][KC], kt[2][4];
    swa2_read_a<C, 0>(sK, L, xk[0]);
    swa2_for<0, NKB>([&](auto kbc) {
      constexpr int kb = decltype(kbc)::value;
      f32x4 s[2], dp[2];
      float t[8];
      // dS^T of one column group: p = exp2(s scale - lse2) where visible, dS = p (dP - delta)
      auto elementwise = [&](const int half) {
        const int cg = 2 * kb + half;
#pragma unroll
        for (int i = 0; i < 4; i++) {
          const float p = fast_exp2(fmaf(s[half][i], scale, neg_lse));
          const float ds = p * dp[half][i];
          t[4 * half + i] = swa2_visible(W, row_vis, cg, i, ncg) ? ds : 0.f;
        }
      };
      // ---- stage 1: S of the even column group
      if constexpr (more) swa2_issue_one<C, 4 * kb>(st, nrow, ndst);
      swa2_read_a<C, 2 * kb>(sV, L, xv[0]);
      __builtin_amdgcn_sched_barrier(0);
      s[0] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int c = 0; c < KC; c++) s[0] = Mma<CT>::mfma(xk[0][c], qf[c], s[0]);
      __builtin_amdgcn_sched_barrier(0);
      // ---- stage 2: dP of the even column group
      if constexpr (more) swa2_issue_one<C, 4 * kb + 1>(st, nrow, ndst);
      swa2_read_a<C, 2 * kb + 1>(sK, L, xk[1]);
      __builtin_amdgcn_sched_barrier(0);
      dp[0] = dinit;
#pragma unroll
      for (int c = 0; c < KC; c++) dp[0] = Mma<CT>::mfma(xv[0][c], dof[c], dp[0]);
      __builtin_amdgcn_sched_barrier(0);
      // ---- stage 3: S of the odd column group
      if constexpr (more) swa2_issue_one<C, 4 * kb + 2>(st, nrow, ndst);
      swa2_read_a<C, 2 * kb + 1>(sV, L, xv[1]);
      __builtin_amdgcn_sched_barrier(0);
      s[1] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int c = 0; c < KC; c++) s[1] = Mma<CT>::mfma(xk[1][c], qf[c], s[1]);
      __builtin_amdgcn_sched_barrier(0);
      // ---- stage 4: dP of the odd column group, with the elementwise work of the even one between the products
      swa2_read_tr<C, kb, 0, 4>(sK, L, kt[0]);
      __builtin_amdgcn_sched_barrier(0);
      dp[1] = dinit;
#pragma unroll
      for (int c = 0; c < KC; c++) dp[1] = Mma<CT>::mfma(xv[1][c], dof[c], dp[1]);
      elementwise(0);
      SWA2_MIX(KC, 16 / KC)
      __builtin_amdgcn_sched_barrier(0);
      // ---- stage 5: elementwise work of the odd column group
      if constexpr (more) swa2_issue_one<C, 4 * kb + 3>(st, nrow, ndst);
      if constexpr (NG == 2) swa2_read_tr<C, kb, 4, 4>(sK, L, kt[1]);
      elementwise(1);
      const u32x4 pk = pack8<CT>(t);
      __builtin_amdgcn_sched_barrier(0);
      // ---- stages 6, 7: dQ^T += K^T dS^T
      if constexpr (kb + 1 < NKB) swa2_read_a<C, 2 * kb + 2>(sK, L, xk[0]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int d = 0; d < 4; d++) acc[d] = Mma<CT>::mfma(kt[0][d], pk, acc[d]);
      if constexpr (NG == 2) {
#pragma unroll
        for (int d = 0; d < 4; d++) acc[4 + d] = Mma<CT>::mfma(kt[1][d], pk, acc[4 + d]);
      }
      __builtin_amdgcn_sched_barrier(0);
    });
  };

  // three loops: copy-only rounds before and after the rounds with visible rows (see the forward kernel)
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

  swa2_store_own<C, TIO, CT>(smem + wave * C::TILE, acc, a.p.sm_scale, dqb, a.dqs[2], G, r_p, c_p, lane);
}

// =============================================================================================== dK / dV
// A chunk buffer holds Q, dO and a table of per-token scalars: lse2 then delta, [4 halo rows][HCW halo columns] each.
template <typename TIO, int D, int NCG>
__global__ __launch_bounds__(SWA2_THREADS, swa2_occ_bwd_kv(D)) void swa2_bwd_kv_kernel(const Swa2BwdArgs a) {
  typedef typename ComputeOf<TIO>::type CT;
  typedef Swa2Cfg<D, NCG> C;
  constexpr int KC = C::KC, VB = C::VB, NKB = C::NKB;
  constexpr int NP2 = VB / 2;   // pairs of 16-dim blocks per gradient
  extern __shared__ __align__(16) char smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63, n = lane & 15, g = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int pc = wave & 3, rg = wave >> 2;
  const Swa2Geom G0 = swa2_geom(a.p, a.plan);

  const char* qb = reinterpret_cast<const char*>(a.q) + 2 * (G0.b * a.qs[0] + G0.h * a.qs[1]);
  const char* kb_ = reinterpret_cast<const char*>(a.k) + 2 * (G0.b * a.ks[0] + G0.h * a.ks[1]);
  const char* vb_ = reinterpret_cast<const char*>(a.v) + 2 * (G0.b * a.vs[0] + G0.h * a.vs[1]);
  const char* dob = reinterpret_cast<const char*>(a.d_o) + 2 * (G0.b * a.dos[0] + G0.h * a.dos[1]);
  TIO* dkb = reinterpret_cast<TIO*>(a.dk) + G0.b * a.dks[0] + G0.h * a.dks[1];
  TIO* dvb = reinterpret_cast<TIO*>(a.dv) + G0.b * a.dvs[0] + G0.h * a.dvs[1];
  const float* lseb = a.lse + G0.b * a.ls[0] + G0.h * a.ls[1];
  const float* delb = a.delta + G0.b * a.ls[0] + G0.h * a.ls[1];
  const float scale = a.scale_log2;

  // staging: waves 0-3 copy the four halo rows of Q and of lse2, waves 4-7 those of dO and of delta
  const bool stage_q = wave < 4;
  const char* sbase = stage_q ? qb : dob;
  const int ssn2 = (int)(stage_q ? a.qs[2] : a.dos[2]) * 2;
  const uint32_t srow = (uint32_t)(G0.TC * ssn2);
  Swa2Geom G = G0;   // column pass 0 (see the forward kernel)
  Swa2Stage<C> st;
  swa2_stage_init(st, G, wave, lane, ssn2);
  const float* scal_base = stage_q ? lseb : delb;
  const int ls2 = (int)a.ls[2];
  // lane l < HCW copies the scalar of halo column l (clamped like the rows: positions outside the grid are masked)
  uint32_t scal_off = (uint32_t)(swa2_scal_col(G, lane) * ls2) * 4u;
  auto issue_scalars = [&](int ch, char* buf) {
    const int r = swa2_issue_grid_row(G, ch, wave);
    const char* row = reinterpret_cast<const char*>(scal_base) + (uint32_t)(r * G.TC * ls2) * 4u;   // wave-uniform
    char* dst = buf + swa2_scal_dst_off<C>(wave);
    if (lane < C::HCW)
      dlt_copy4_to_lds(row, scal_off, dst);
  };
  swa2_issue(st, G, G.ch_first, sbase, srow, smem + (G.ch_first & 1) * C::BUF_KV, wave);
  issue_scalars(G.ch_first, smem + (G.ch_first & 1) * C::BUF_KV);

  const int r_p = G.r0 + 4 * rg, c_p = G.c0 + 4 * pc;
  const int tk = (r_p + (n >> 2) < G.TR && c_p + (n & 3) < G.TC) ? (r_p + (n >> 2)) * G.TC + c_p + (n & 3) : -1;
  u32x4 kf[KC], vf[KC];
  swa2_own_frags<KC>(kf, kb_, (int)a.ks[2] * 2, tk, g);
  swa2_own_frags<KC>(vf, vb_, (int)a.vs[2] * 2, tk, g);
  const Swa2Win W0 = swa2_window(G0, rg, pc, n);
  Swa2Win W = W0;
  Swa2Lane<C> L;
  swa2_lane_init(L, pc, n, g);
  // scalars of the queries (halo row g, window columns 4 cg .. 4 cg + 3) of a chunk
  const int scal_lane = swa2_scal_lane_off<C>(g, pc);

  f32x4 acck[VB], accv[VB];
#pragma unroll
  for (int d = 0; d < VB; d++) { acck[d] = f32x4{0.f, 0.f, 0.f, 0.f}; accv[d] = f32x4{0.f, 0.f, 0.f, 0.f}; }
  int ncg = swa2_pass_ncg(G0.WC, NCG, 0);

  swa2_wait_copies();
  // the compiler does not see that wait: tell it that the own fragments are loaded, or it waits for them (and with them
  // for every copy in flight) at their first use inside every round of the chunk loop
  pin_loaded(kf);
  pin_loaded(vf);
  // The own values are negated and the dP products start from the staged delta of the lane's four queries (read from LDS
  // straight into the C operand, a stage or more ahead): the matrix pipe delivers -(dP - delta), and dS = -p (.) (the sign
  // is an operand modifier).
#pragma unroll
  for (int c = 0; c < KC; c++) {
    vf[c].x ^= 0x80008000u; vf[c].y ^= 0x80008000u; vf[c].z ^= 0x80008000u; vf[c].w ^= 0x80008000u;
  }
  __syncthreads();

  auto consume = [&](const int ch, Swa2Lds __restrict__ cur, char* __restrict__ nxt, auto more_tag) {
    constexpr bool more = decltype(more_tag)::value;
    Swa2Lds sQ = cur;
    Swa2Lds sD = sQ + C::REGION;
    Swa2Lds sLse = cur + C::BUF + scal_lane;
    Swa2Lds sDel = sLse + C::TOK * 4;
    const char* nrow = swa2_issue_row(G, ch + 1, sbase, srow, wave);
    char* ndst = swa2_issue_dst<C>(nxt, wave);
    if constexpr (more) issue_scalars(ch + 1, nxt);
    const int hrow = 4 * ch + g;
    const bool row_vis = (hrow >= W.rlo) & (hrow <= W.rhi);
    // two A-operand buffers: a buffer is free again once the products that read it have been issued, one stage before
    // the next read into it returns.  Transposed operands come in pairs of 16-dim blocks, one pair ahead of its products.
    u32x4 x[2][KC], tr[2][2];
    swa2_read_a<C, 0>(sQ, L, x[0]);
    f32x4 lse_e = __builtin_bit_cast(f32x4, swa2_lds16(sLse)), del_e = __builtin_bit_cast(f32x4, swa2_lds16(sDel));
    swa2_for<0, NKB>([&](auto kbc) {
      constexpr int kb = decltype(kbc)::value;
      u32x4 pp, pd;
      // P and dS of one column group, packed: p = exp2(s scale - lse2) where visible, dS = p (dP - delta)
      auto elementwise = [&](const int half, const f32x4& sv, const f32x4& dpv, const f32x4& lse4) {
        const int cg = 2 * kb + half;
        float tp[4], td[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
          const float p = fast_exp2(fmaf(sv[i], scale, -lse4[i]));
          const bool vis = swa2_visible(W, row_vis, cg, i, ncg);
          tp[i] = vis ? p : 0.f;
          td[i] = vis ? -p * dpv[i] : 0.f;
        }
        if (half == 0) {
          pp.x = pack2<CT>(tp[0], tp[1]); pp.y = pack2<CT>(tp[2], tp[3]);
          pd.x = pack2<CT>(td[0], td[1]); pd.y = pack2<CT>(td[2], td[3]);
        } else {
          pp.z = pack2<CT>(tp[0], tp[1]); pp.w = pack2<CT>(tp[2], tp[3]);
          pd.z = pack2<CT>(td[0], td[1]); pd.w = pack2<CT>(td[2], td[3]);
        }
      };
      // ---- stage 1: S of the even column group (rows: queries, columns: own keys)
      if constexpr (more) swa2_issue_one<C, 4 * kb>(st, nrow, ndst);
      swa2_read_a<C, 2 * kb>(sD, L, x[1]);
      const f32x4 lse_o = __builtin_bit_cast(f32x4, swa2_lds16(sLse + 32 * kb + 16));
      const f32x4 del_o = __builtin_bit_cast(f32x4, swa2_lds16(sDel + 32 * kb + 16));
      __builtin_amdgcn_sched_barrier(0);
      f32x4 s0 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int c = 0; c < KC; c++) s0 = Mma<CT>::mfma(x[0][c], kf[c], s0);
      __builtin_amdgcn_sched_barrier(0);
      // ---- stage 2: dP of the even column group
      if constexpr (more) swa2_issue_one<C, 4 * kb + 1>(st, nrow, ndst);
      swa2_read_a<C, 2 * kb + 1>(sQ, L, x[0]);
      __builtin_amdgcn_sched_barrier(0);
      f32x4 dp0 = del_e;
#pragma unroll
      for (int c = 0; c < KC; c++) dp0 = Mma<CT>::mfma(x[1][c], vf[c], dp0);
      __builtin_amdgcn_sched_barrier(0);
      // ---- stage 3: S of the odd column group, with the elementwise work of the even one between the products
      if constexpr (more) swa2_issue_one<C, 4 * kb + 2>(st, nrow, ndst);
      swa2_read_a<C, 2 * kb + 1>(sD, L, x[1]);
      __builtin_amdgcn_sched_barrier(0);
      f32x4 s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int c = 0; c < KC; c++) s1 = Mma<CT>::mfma(x[0][c], kf[c], s1);
      elementwise(0, s0, dp0, lse_e);
      SWA2_MIX(KC, 20 / KC)
      __builtin_amdgcn_sched_barrier(0);
      // ---- stage 4: dP of the odd column group
      swa2_read_tr<C, kb, 0, 2>(sD, L, tr[0]);
      __builtin_amdgcn_sched_barrier(0);
      f32x4 dp1 = del_o;
#pragma unroll
      for (int c = 0; c < KC; c++) dp1 = Mma<CT>::mfma(x[1][c], vf[c], dp1);
      __builtin_amdgcn_sched_barrier(0);
      // ---- stage 5: elementwise work of the odd column group
      if constexpr (more) swa2_issue_one<C, 4 * kb + 3>(st, nrow, ndst);
      swa2_read_tr<C, kb, 2, 2>(sD, L, tr[1]);
      elementwise(1, s1, dp1, lse_o);
      __builtin_amdgcn_sched_barrier(0);
      // ---- stage 6: dV^T += dO^T P over NP2 pairs of 16-dim blocks, then dK^T += Q^T dS over NP2 pairs.  Pair j of the
      //      sequence sits in tr[j & 1]; pair j + 2 is requested once the products of pair j are issued, and the first
      //      operands of the next 32 queries before the last pair.
      swa2_for<0, 2 * NP2>([&](auto jc) {
        constexpr int j = decltype(jc)::value;
        constexpr int d0 = 2 * (j % NP2);
        if constexpr (j == 2 * NP2 - 1 && kb + 1 < NKB) {
          swa2_read_a<C, 2 * kb + 2>(sQ, L, x[0]);
          lse_e = __builtin_bit_cast(f32x4, swa2_lds16(sLse + 32 * (kb + 1)));
          del_e = __builtin_bit_cast(f32x4, swa2_lds16(sDel + 32 * (kb + 1)));
          __builtin_amdgcn_sched_barrier(0);
        }
        if constexpr (j < NP2) {
#pragma unroll
          for (int d = 0; d < 2; d++) accv[d0 + d] = Mma<CT>::mfma(tr[j & 1][d], pp, accv[d0 + d]);
        } else {
#pragma unroll
          for (int d = 0; d < 2; d++) acck[d0 + d] = Mma<CT>::mfma(tr[j & 1][d], pd, acck[d0 + d]);
        }
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (j + 2 < 2 * NP2) {
          constexpr int j2 = j + 2;
          if constexpr (j2 < NP2) swa2_read_tr<C, kb, 2 * j2, 2>(sD, L, tr[j & 1]);
          else swa2_read_tr<C, kb, 2 * (j2 - NP2), 2>(sQ, L, tr[j & 1]);
          __builtin_amdgcn_sched_barrier(0);
        }
      });
    });
  };

  // three loops, as in the dQ kernel
  const int act_lo = dlt_imax(G.ch_first, W.ch_lo), act_hi = dlt_imin(G.ch_last - 1, W.ch_hi);
  auto copy_only = [&](int ch) {
    char* nxt = smem + ((ch + 1) & 1) * C::BUF_KV;
    swa2_issue(st, G, ch + 1, sbase, srow, nxt, wave);
    issue_scalars(ch + 1, nxt);
    swa2_wait_copies();
    __syncthreads();
  };
  for (int pass = 0;;) {
    int ch = G.ch_first;
    for (; ch < G.ch_last && ch < act_lo; ch++) copy_only(ch);
    for (; ch <= act_hi; ch++) {
      consume(ch, (Swa2Lds)smem + (ch & 1) * C::BUF_KV, smem + ((ch + 1) & 1) * C::BUF_KV, std::true_type{});
      swa2_wait_copies();
      __syncthreads();
    }
    for (; ch < G.ch_last; ch++) copy_only(ch);
    if (G.ch_last >= W.ch_lo && G.ch_last <= W.ch_hi)
      consume(G.ch_last, (Swa2Lds)smem + (G.ch_last & 1) * C::BUF_KV, smem + ((G.ch_last + 1) & 1) * C::BUF_KV, std::false_type{});
    __syncthreads();   // every wave is done with both chunk buffers
    if (++pass >= a.plan.npass) break;
    // next column pass: the same rows again, 4 NCG columns further to the right
    G = swa2_pass_geom(G0, NCG, pass);
    W = swa2_pass_window(W0, NCG, pass);
    ncg = swa2_pass_ncg(G0.WC, NCG, pass);
    swa2_stage_init(st, G, wave, lane, ssn2);
    scal_off = (uint32_t)(swa2_scal_col(G, lane) * ls2) * 4u;
    swa2_issue(st, G, G.ch_first, sbase, srow, smem + (G.ch_first & 1) * C::BUF_KV, wave);
    issue_scalars(G.ch_first, smem + (G.ch_first & 1) * C::BUF_KV);
    swa2_wait_copies();
    __syncthreads();
  }

  swa2_store_own<C, TIO, CT>(smem + wave * C::TILE, accv, 1.f, dvb, a.dvs[2], G, r_p, c_p, lane);
  swa2_store_own<C, TIO, CT>(smem + wave * C::TILE, acck, a.p.sm_scale, dkb, a.dks[2], G, r_p, c_p, lane);
}
