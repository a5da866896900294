// Backward kernels for token grids (b_size == 1): the decoupled dK/dV and dQ passes of
// tiled_swa_bwd_large_kernel_decoupled_q (src/tiled_swa.py:407-562) on the 2D-patch / shared
// halo structure of the token-grid forward kernel.  The reference has no backward for tiles of
// fewer than 16 tokens (src/tiled_swa.py:660-661).
//
//   dK/dV: a wave owns a 4x4 patch of keys; the queries that can see them (their halo, by the
//          symmetry of the window) stream through LDS in chunks of CR rows: Q (rotated when
//          the rotary encoding is fused), dO, lse2 and delta.
//   dQ   : a wave owns a 4x4 patch of queries; K (rotated) and V stream through LDS.  It runs
//          first and can compute delta = rowsum(o * dO) of its own queries on the way (the
//          reference's separate pre-pass, src/tiled_swa.py:253-282), which the dK/dV kernel
//          launched after it reads back.
// Both recompute P = exp2(s * scale - lse2) per block; tokens of the streamed side are the MFMA
// rows, so P / dS leave the first products in the layout the second products take as B operand.
#pragma once
#include "swa1_common.hpp"

struct Swa1BwdArgs {
  AttnProblem p;
  Swa1Plan plan;
  const void *q, *k, *v, *o, *d_o;
  const float *lse, *delta;
  float* delta_out;   // fuse_delta: the dQ kernel computes delta = rowsum(o * dO) of its own tokens and stores it here
  void *dq, *dk, *dv;
  int64_t qs[4], ks[4], vs[4], os[4], dos[4], dqs[4], dks[4], dvs[4], ls[3];
  int32_t fuse_delta;
  int32_t rope_mode;  // 0 none, 1 rotation with the plain staging map, 2 balanced staging map
  int32_t q_vec, k_vec, v_vec, do_vec, dq_vec, dk_vec, dv_vec;
  int32_t rope_pbit;
  float scale_log2;
};

// per-token fp32 values (lse2 / delta) of halo rows [cr0, cr0 + CR): CR * HCW values over 256 threads
template <int HCW, int CR>
struct ScalarRegs { float v[(CR * HCW + 255) / 256]; };

// lse2 and delta share their indexing: the offsets are computed once and BEFORE the first load (an
// address computation placed between two loads can end up waiting for the first one: the compiler
// forms 32-bit multiply-adds with a 64-bit instruction whose unused upper addend half may be the
// register the pending load writes).
template <int HCW, int CR>
DLT_DEV void swa1_issue_scalar2(ScalarRegs<HCW, CR>& sa, ScalarRegs<HCW, CR>& sb, const float* base_a, const float* base_b,
                                int64_t stride, const Swa1Geom& G, int cr0, int tid) {
  constexpr int NS = (CR * HCW + 255) / 256;
  uint32_t off[NS];
#pragma unroll
  for (int it = 0; it < NS; it++) {
    // clamped like the tile staging: out-of-grid halo positions are masked by the window bias;
    // threads past the end of the chunk re-read its first token (the value is not stored)
    const int idx = dlt_imin(tid + 256 * it, CR * HCW - 1);
    const int hr = idx / HCW, hc = idx - hr * HCW;
    const int r = dlt_imax(0, dlt_imin(G.r0 - G.WR + cr0 + hr, G.TR - 1));
    const int c = dlt_imax(0, dlt_imin(G.c0 - G.WC + hc, G.TC - 1));
    off[it] = (uint32_t)((r * G.TC + c) * (int)stride);
  }
#pragma unroll
  for (int it = 0; it < NS; it++) {
    sa.v[it] = base_a[off[it]];
    sb.v[it] = base_b[off[it]];
  }
}

template <int HCW, int CR>
DLT_DEV void swa1_commit_scalar(const ScalarRegs<HCW, CR>& sr, float* s, int tid) {
#pragma unroll
  for (int it = 0; it < (CR * HCW + 255) / 256; it++) pin_loaded(sr.v[it]);  // the wait, on every path
#pragma unroll
  for (int it = 0; it < (CR * HCW + 255) / 256; it++) {
    const int idx = tid + 256 * it;
    if (idx < CR * HCW) s[idx] = sr.v[it];
  }
}

// shared prologue: workgroup -> band, lane -> window biases
template <int NCGMAX>
struct Swa1Lane {
  Swa1Geom G;
  int b, h;
  int rlo, rhi;
  int clo, cspan;  // column window [clo, clo + cspan] of this lane's own token (cspan < 0: none)
  bool cg_edge[NCGMAX];
  int wcol_lo, wcol_hi;
  bool wave_ok;
  int ch_first, ch_last;

  DLT_DEV void init(const AttnProblem& p, const Swa1Plan& P, int wave, int n, int cr = 8) {
    const int lin = xcd_remap(blockIdx.x, gridDim.x);
    const int per_bh = P.nblk_r * P.nblk_c;
    const int bh = lin / per_bh;
    const int rem = lin - bh * per_bh;
    const int br = rem / P.nblk_c;
    b = bh / p.H;
    h = bh - b * p.H;
    G.r0 = 4 * br; G.c0 = 16 * (rem - br * P.nblk_c);
    G.TR = p.g.TR; G.TC = p.g.TC; G.WR = p.g.WR; G.WC = p.g.WC;
    const int qr_l = n >> 2, qc_l = n & 3;
    const int cw = G.c0 + 4 * wave;
    const bool q_ok = (G.r0 + qr_l < G.TR) && (cw + qc_l < G.TC);
    rlo = dlt_imax(qr_l, G.WR - G.r0);
    rhi = dlt_imin(qr_l + 2 * G.WR, G.TR - 1 - G.r0 + G.WR);
    clo = dlt_imax(qc_l, G.WC - cw);
    const int chi = dlt_imin(qc_l + 2 * G.WC, G.TC - 1 - cw + G.WC);
    cspan = q_ok ? chi - clo : -1;
    // column groups whose 4 columns lie inside every lane's window need no test (wave-uniform flag)
#pragma unroll
    for (int cg = 0; cg < NCGMAX; cg++)
      cg_edge[cg] = __builtin_amdgcn_ballot_w64(!((unsigned)(4 * cg - clo) <= (unsigned)cspan &&
                                                  (unsigned)(4 * cg + 3 - clo) <= (unsigned)cspan)) != 0;
    wcol_lo = dlt_imax(0, G.WC - cw);
    wcol_hi = G.TC - 1 - cw + G.WC;
    wave_ok = cw < G.TC;
    const int wrow_lo = dlt_imax(0, G.WR - G.r0), wrow_hi = dlt_imin(3 + 2 * G.WR, G.TR - 1 - G.r0 + G.WR);
    ch_first = wrow_lo / cr;
    ch_last = wrow_hi / cr;
  }
  DLT_DEV int64_t own_token(int row) const {
    const int r = G.r0 + ((row & 15) >> 2), c = G.c0 + 4 * (row >> 4) + (row & 3);
    return (r < G.TR && c < G.TC) ? (int64_t)r * G.TC + c : (int64_t)-1;
  }
  // window column 4 * cg + i visible from this lane's own token
  DLT_DEV bool col_ok(int cg, int i) const { return (unsigned)(4 * cg + i - clo) <= (unsigned)cspan; }
  DLT_DEV bool block_on(const Swa1Plan& P, int cg) const {
    return wave_ok && cg < P.ncg && 4 * cg <= wcol_hi && 4 * cg + 3 >= wcol_lo;
  }
};

// accumulators (C layout, [dim][own token]) -> LDS tile [own token][dim] -> HBM rows
template <typename TIO, int D, typename LaneT>
DLT_DEV void swa1_write_grad(char* sT, f32x4 (&acc)[D / 16], float mul, TIO* base, int64_t sn, int64_t sd, int dact, bool vec,
                             const LaneT& L, const RopeDev& rope, int wave, int n, int g, int tid) {
  typedef typename TileOf<TIO>::type TL;
  constexpr int PT = D * (int)sizeof(TL) + 16;
  TL* row = reinterpret_cast<TL*>(sT + (16 * wave + n) * PT);
#pragma unroll
  for (int d = 0; d < D / 16; d++)
#pragma unroll
    for (int i = 0; i < 4; i++) row[16 * d + 4 * g + i] = (TL)(acc[d][i] * mul);
  __syncthreads();
  store_tile<TIO, TL, D>(sT, PT, base, sn, sd, dact, vec, 64, [&](int r) { return L.own_token(r); }, rope, tid);
  __syncthreads();
}

// =============================================================================================
template <typename TIO, int D, int NCGMAX, int CR, int ROPE>
// Occupancy target of the variants with rotation: one below what the kernel reaches (its register count
// still admits three workgroups per CU).  With a target of three the compiler, a few registers over its
// budget, reschedules the whole kernel for minimum register pressure and the product loop loses its
// read-ahead (LDS reads issued one or two ahead of their MFMA instead of a dozen).
__global__ __launch_bounds__(256, (D <= 64 ? (CR == 4 && NCGMAX <= 4 && ROPE == 0 ? 3 : 2) : (CR == 4 ? 2 : 1))) void swa1_bwd_kv_kernel(const Swa1BwdArgs a) {
  typedef typename ComputeOf<TIO>::type CT;
  extern __shared__ __align__(16) char smem[];
  // ROPE 3: q and k arrive rotated (saved by the forward pass); only the gradients are rotated back on store
  constexpr int LROT = ROPE == 3 ? 0 : ROPE;  // rotation applied to the tile loads
  constexpr bool WIDE = LROT == 0;
  constexpr int PA = swa1_pitch(D, NCGMAX, 0, WIDE, true), PB = swa1_pitch(D, NCGMAX, 1, WIDE, true);  // Q rows, dO rows
  constexpr int KC = D / 32, DB = D / 16;
  constexpr int HCW = swa1_hcw(NCGMAX);
  constexpr int REGION = CR * HCW * PA;
  constexpr int NKB = CR == 8 ? NCGMAX : NCGMAX / 2;
  constexpr int MB_STEP = CR == 8 ? 4 * HCW : 4;

  const int tid = threadIdx.x;
  const int lane = tid & 63, n = lane & 15, g = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const Swa1Plan& P = a.plan;
  char* sQ = smem;
  char* sDO = smem + REGION;
  float* sLse = reinterpret_cast<float*>(smem + REGION + CR * HCW * PB);
  float* sDel = sLse + CR * HCW;

  Swa1Lane<NCGMAX> L;
  L.init(a.p, P, wave, n, CR);
  const Swa1Geom& G = L.G;
  const int b = L.b, h = L.h;

  const TIO* qb = reinterpret_cast<const TIO*>(a.q) + b * a.qs[0] + h * a.qs[1];
  const TIO* kb_ = reinterpret_cast<const TIO*>(a.k) + b * a.ks[0] + h * a.ks[1];
  const TIO* vb_ = reinterpret_cast<const TIO*>(a.v) + b * a.vs[0] + h * a.vs[1];
  const TIO* dob = reinterpret_cast<const TIO*>(a.d_o) + b * a.dos[0] + h * a.dos[1];
  const float* lseb = a.lse + b * a.ls[0] + h * a.ls[1];
  const float* delb = a.delta + b * a.ls[0] + h * a.ls[1];
  RopeDev fwd_rope = a.p.rope;  fwd_rope.inverse = 0;
  RopeDev inv_rope = a.p.rope;  inv_rope.inverse = 1;
  RopeDev no_rope = a.p.rope;   no_rope.enabled = 0;
  constexpr bool use_rope = LROT != 0, store_rope = ROPE != 0;
  constexpr bool BAL = LROT == 2;
  const int32_t* rope_idx = use_rope ? a.p.rope.idx : nullptr;
  auto own_token = [&](int row) { return L.own_token(row); };

  constexpr bool TAIL = LROT == 0 && swa1_use_tail(D, HCW, CR);
  constexpr int NI = swa1_items_t(D, HCW, CR, TAIL);
  StagePlan<NI> sp;
  swa1_plan_init<D, HCW, CR, BAL, TAIL, WIDE, PA, PB>(sp, G, tid, a.rope_pbit);
  const bool on_k = (sp.coff[0] >> 1) < a.p.dk, on_v = (sp.coff[0] >> 1) < a.p.dv;
  const int sn2q = (int)a.qs[2] * 2, sn2d = (int)a.dos[2] * 2;
  StageRegs<NI> srq, srd;
  swa1_regs_zero(srq);
  TabRegs<NI> tr_srq;
  swa1_regs_zero(srd);
  swa1_issue<NI, BAL, TAIL, 0>(srq, sp, on_k, qb, sn2q, G, CR * L.ch_first, rope_idx, (sp.t_off >> 1) < a.p.dk);
  swa1_issue<NI, BAL, TAIL, 1>(srd, sp, on_v, dob, sn2d, G, CR * L.ch_first, nullptr, (sp.t_off >> 1) < a.p.dv);
  ScalarRegs<HCW, CR> r_lse, r_del;
  swa1_issue_scalar2<HCW, CR>(r_lse, r_del, lseb, delb, a.ls[2], G, CR * L.ch_first, tid);

  // own keys / values straight into B-operand fragments
  u32x4 kf[KC], vf[KC];
  {
    const int64_t tk = L.own_token(16 * wave + n);
    swa1_load_own<TIO, CT, D>(vf, vb_, a.vs[2], a.p.dv, tk, g, no_rope, false);
    swa1_load_own<TIO, CT, D>(kf, kb_, a.ks[2], a.p.dk, tk, g, fwd_rope, use_rope);
  }

  f32x4 dk_acc[DB], dv_acc[DB];
#pragma unroll
  for (int d = 0; d < DB; d++) { dk_acc[d] = f32x4{0.f, 0.f, 0.f, 0.f}; dv_acc[d] = f32x4{0.f, 0.f, 0.f, 0.f}; }
  const float scale = a.scale_log2;

  if (LROT == 2) swa1_tab_issue(tr_srq, srq, sp, fwd_rope);
  swa1_commit<CT, NI, BAL, LROT, TAIL, 0, PA>(srq, sp, sQ, a.rope_pbit, fwd_rope, on_k, &tr_srq, (sp.t_off >> 1) < a.p.dk);
  swa1_commit<CT, NI, BAL, 0, TAIL, 1, PB>(srd, sp, sDO, 1, no_rope, false, nullptr, (sp.t_off >> 1) < a.p.dv);
  swa1_commit_scalar<HCW, CR>(r_lse, sLse, tid);
  swa1_commit_scalar<HCW, CR>(r_del, sDel, tid);
  __syncthreads();
  pin_loaded(kf);
  pin_loaded(vf);

  // products of the chunk resident in LDS
  auto consume = [&](const int ch) {
    const int cr0 = CR * ch;
    float rbias[2];
#pragma unroll
    for (int mb = 0; mb < 2; mb++) {
      const int hrow = cr0 + (CR == 8 ? 4 * mb : 0) + g;
      rbias[mb] = (hrow >= L.rlo && hrow <= L.rhi) ? 0.f : -INFINITY;
    }
#pragma unroll
    for (int kb = 0; kb < NKB; kb++) {
      const int cg0 = CR == 8 ? kb : 2 * kb, cg1 = CR == 8 ? kb : 2 * kb + 1;
      if (!(L.wave_ok && cg0 < P.ncg && 4 * cg0 <= L.wcol_hi && 4 * cg1 + 3 >= L.wcol_lo)) continue;
      const int key0 = (n >> 2) * HCW + 4 * wave + 4 * cg0 + (n & 3);  // A-operand row of this lane
      const int tok0 = g * HCW + 4 * wave + 4 * cg0;                    // first of the 4 result columns
      f32x4 s[2], dp[2];
#pragma unroll
      for (int mb = 0; mb < 2; mb++) {
        s[mb] = f32x4{0.f, 0.f, 0.f, 0.f};
        dp[mb] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < KC; c++) {
          s[mb] = Mma<CT>::mfma(lds_read16(sQ + (key0 + mb * MB_STEP) * PA + (32 * c + 8 * g) * 2), kf[c], s[mb]);
          dp[mb] = Mma<CT>::mfma(lds_read16(sDO + (key0 + mb * MB_STEP) * PB + (32 * c + 8 * g) * 2), vf[c], dp[mb]);
        }
      }
      float pr[8], ds[8];
#pragma unroll
      for (int mb = 0; mb < 2; mb++) {
        const f32x4 lq = *reinterpret_cast<const f32x4*>(sLse + tok0 + mb * MB_STEP);
        const f32x4 dq_ = *reinterpret_cast<const f32x4*>(sDel + tok0 + mb * MB_STEP);
        const int cg = mb == 0 ? cg0 : cg1;
#pragma unroll
        for (int i = 0; i < 4; i++) {
          float nl = rbias[mb] - lq[i];
          if (L.cg_edge[cg]) nl = L.col_ok(cg, i) ? nl : -INFINITY;
          const float pv = fast_exp2(fmaf(s[mb][i], scale, nl));
          pr[4 * mb + i] = pv;
          ds[4 * mb + i] = pv * (dp[mb][i] - dq_[i]);
        }
      }
      const u32x4 pb = pack8<CT>(pr), dsb = pack8<CT>(ds);
      const int kt0 = 4 * wave + 4 * cg0;
#pragma unroll
      for (int d = 0; d < DB; d++) {
        dv_acc[d] = Mma<CT>::mfma(swa1_read_tokens_as_k(sDO, PB, HCW, kt0, 16 * d, n, g, MB_STEP), pb, dv_acc[d]);
        dk_acc[d] = Mma<CT>::mfma(swa1_read_tokens_as_k(sQ, PA, HCW, kt0, 16 * d, n, g, MB_STEP), dsb, dk_acc[d]);
      }
    }
  };
  // the last chunk is peeled off: prefetch and commit are unconditional inside the loop (see the
  // forward kernel)
  for (int ch = L.ch_first; ch < L.ch_last; ch++) {
    swa1_issue_scalar2<HCW, CR>(r_lse, r_del, lseb, delb, a.ls[2], G, CR * ch + CR, tid);
    swa1_issue<NI, BAL, TAIL, 0>(srq, sp, on_k, qb, sn2q, G, CR * ch + CR, rope_idx, (sp.t_off >> 1) < a.p.dk);
    swa1_issue<NI, BAL, TAIL, 1>(srd, sp, on_v, dob, sn2d, G, CR * ch + CR, nullptr, (sp.t_off >> 1) < a.p.dv);
    consume(ch);
    if (LROT == 2) swa1_tab_issue(tr_srq, srq, sp, fwd_rope);
    __syncthreads();
    swa1_commit<CT, NI, BAL, LROT, TAIL, 0, PA>(srq, sp, sQ, a.rope_pbit, fwd_rope, on_k, &tr_srq, (sp.t_off >> 1) < a.p.dk);
    swa1_commit<CT, NI, BAL, 0, TAIL, 1, PB>(srd, sp, sDO, 1, no_rope, false, nullptr, (sp.t_off >> 1) < a.p.dv);
    swa1_commit_scalar<HCW, CR>(r_lse, sLse, tid);
    swa1_commit_scalar<HCW, CR>(r_del, sDel, tid);
    __syncthreads();
  }
  consume(L.ch_last);
  __syncthreads();

  TIO* dkb = reinterpret_cast<TIO*>(a.dk) + b * a.dks[0] + h * a.dks[1];
  TIO* dvb = reinterpret_cast<TIO*>(a.dv) + b * a.dvs[0] + h * a.dvs[1];
  if (a.dk_vec != 0 && a.dv_vec != 0) {  // the loop ended with a workgroup barrier: the chunk buffers are free
    char* sW = smem + wave * 16 * (D * 2 + 16);
    swa1_store_own<TIO, CT, D>(sW, dk_acc, a.p.sm_scale, dkb, a.dks[2], a.p.dk, G, wave, lane, inv_rope, store_rope);
    swa1_store_own<TIO, CT, D>(sW, dv_acc, 1.0f, dvb, a.dvs[2], a.p.dv, G, wave, lane, no_rope, false);
    return;
  }
  swa1_write_grad<TIO, D>(smem, dk_acc, a.p.sm_scale, dkb, a.dks[2], a.dks[3], a.p.dk, a.dk_vec != 0, L, store_rope ? inv_rope : no_rope, wave, n, g, tid);
  swa1_write_grad<TIO, D>(smem, dv_acc, 1.0f, dvb, a.dvs[2], a.dvs[3], a.p.dv, a.dv_vec != 0, L, no_rope, wave, n, g, tid);
}

// =============================================================================================
template <typename TIO, int D, int NCGMAX, int CR, int ROPE>
__global__ __launch_bounds__(256, (D <= 64 ? (CR == 4 && NCGMAX <= 4 ? 4 : 2) : (CR == 4 ? 2 : 1))) void swa1_bwd_q_kernel(const Swa1BwdArgs a) {
  typedef typename ComputeOf<TIO>::type CT;
  extern __shared__ __align__(16) char smem[];
  // ROPE 3: q and k arrive rotated (saved by the forward pass); only the gradients are rotated back on store
  constexpr int LROT = ROPE == 3 ? 0 : ROPE;  // rotation applied to the tile loads
  constexpr bool WIDE = LROT == 0;
  constexpr int PA = swa1_pitch(D, NCGMAX, 0, WIDE), PB = swa1_pitch(D, NCGMAX, 1, WIDE);  // K rows, V rows
  constexpr int KC = D / 32, DB = D / 16;
  constexpr int HCW = swa1_hcw(NCGMAX);
  constexpr int REGION = CR * HCW * PA;
  constexpr int NKB = CR == 8 ? NCGMAX : NCGMAX / 2;
  constexpr int MB_STEP = CR == 8 ? 4 * HCW : 4;

  const int tid = threadIdx.x;
  const int lane = tid & 63, n = lane & 15, g = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const Swa1Plan& P = a.plan;
  char* sK = smem;
  char* sV = smem + REGION;

  Swa1Lane<NCGMAX> L;
  L.init(a.p, P, wave, n, CR);
  const Swa1Geom& G = L.G;
  const int b = L.b, h = L.h;

  const TIO* qb = reinterpret_cast<const TIO*>(a.q) + b * a.qs[0] + h * a.qs[1];
  const TIO* kb_ = reinterpret_cast<const TIO*>(a.k) + b * a.ks[0] + h * a.ks[1];
  const TIO* vb_ = reinterpret_cast<const TIO*>(a.v) + b * a.vs[0] + h * a.vs[1];
  const TIO* dob = reinterpret_cast<const TIO*>(a.d_o) + b * a.dos[0] + h * a.dos[1];
  RopeDev fwd_rope = a.p.rope;  fwd_rope.inverse = 0;
  RopeDev inv_rope = a.p.rope;  inv_rope.inverse = 1;
  RopeDev no_rope = a.p.rope;   no_rope.enabled = 0;
  constexpr bool use_rope = LROT != 0, store_rope = ROPE != 0;
  constexpr bool BAL = LROT == 2;
  const int32_t* rope_idx = use_rope ? a.p.rope.idx : nullptr;
  auto own_token = [&](int row) { return L.own_token(row); };

  constexpr bool TAIL = LROT == 0 && swa1_use_tail(D, HCW, CR);
  constexpr int NI = swa1_items_t(D, HCW, CR, TAIL);
  StagePlan<NI> sp;
  swa1_plan_init<D, HCW, CR, BAL, TAIL, WIDE, PA, PB>(sp, G, tid, a.rope_pbit);
  const bool on_k = (sp.coff[0] >> 1) < a.p.dk, on_v = (sp.coff[0] >> 1) < a.p.dv;
  const int sn2k = (int)a.ks[2] * 2, sn2v = (int)a.vs[2] * 2;
  StageRegs<NI> srk, srv;
  swa1_regs_zero(srk);
  TabRegs<NI> tr_srk;
  swa1_regs_zero(srv);
  swa1_issue<NI, BAL, TAIL, 0>(srk, sp, on_k, kb_, sn2k, G, CR * L.ch_first, rope_idx, (sp.t_off >> 1) < a.p.dk);
  swa1_issue<NI, BAL, TAIL, 1>(srv, sp, on_v, vb_, sn2v, G, CR * L.ch_first, nullptr, (sp.t_off >> 1) < a.p.dv);

  // own output gradients, outputs and queries straight into B-operand fragments.  Everything that
  // needs no rotation is requested first; the rotated query fragments wait for their table rows last.
  u32x4 qf[KC], dof[KC], of[KC];
  const int64_t tq = L.own_token(16 * wave + n);
  const int64_t loff = b * a.ls[0] + h * a.ls[1] + (tq >= 0 ? tq : 0) * a.ls[2];
  const float lse_ld = a.lse[loff];
  const float del_ld = a.fuse_delta != 0 ? 0.f : a.delta[loff];
  swa1_load_own<TIO, CT, D>(dof, dob, a.dos[2], a.p.dv, tq, g, no_rope, false);
  {
    // o is only needed when delta is computed here; otherwise dO is re-read (a valid address, unused)
    const TIO* ob = a.fuse_delta != 0 ? reinterpret_cast<const TIO*>(a.o) + b * a.os[0] + h * a.os[1] : dob;
    swa1_load_own<TIO, CT, D>(of, ob, a.fuse_delta != 0 ? a.os[2] : a.dos[2], a.p.dv, tq, g, no_rope, false);
  }
  swa1_load_own<TIO, CT, D>(qf, qb, a.qs[2], a.p.dk, tq, g, fwd_rope, use_rope);
  const float lse_n = tq >= 0 ? lse_ld : 0.f;
  float del_n;
  if (a.fuse_delta != 0) {
    // delta of the own tokens, computed here and published for the dK/dV kernel that runs next
    float part = 0.f;
#pragma unroll
    for (int c = 0; c < KC; c++) {
      float fo[8], fd[8];
      unpack8<CT>(of[c], fo);
      unpack8<CT>(dof[c], fd);
#pragma unroll
      for (int j = 0; j < 8; j++) part += fo[j] * fd[j];
    }
    del_n = wave_sum4(part);
    if (g == 0 && tq >= 0) a.delta_out[loff] = del_n;
  } else {
    del_n = tq >= 0 ? del_ld : 0.f;
  }

  f32x4 dq_acc[DB];
#pragma unroll
  for (int d = 0; d < DB; d++) dq_acc[d] = f32x4{0.f, 0.f, 0.f, 0.f};
  const float scale = a.scale_log2;

  if (LROT == 2) swa1_tab_issue(tr_srk, srk, sp, fwd_rope);
  swa1_commit<CT, NI, BAL, LROT, TAIL, 0, PA>(srk, sp, sK, a.rope_pbit, fwd_rope, on_k, &tr_srk, (sp.t_off >> 1) < a.p.dk);
  swa1_commit<CT, NI, BAL, 0, TAIL, 1, PB>(srv, sp, sV, 1, no_rope, false, nullptr, (sp.t_off >> 1) < a.p.dv);
  __syncthreads();
  pin_loaded(qf);
  pin_loaded(dof);
  pin_loaded(lse_n);
  pin_loaded(del_n);

  // products of the chunk resident in LDS
  auto consume = [&](const int ch) {
    const int cr0 = CR * ch;
    float rbias[2];
#pragma unroll
    for (int mb = 0; mb < 2; mb++) {
      const int hrow = cr0 + (CR == 8 ? 4 * mb : 0) + g;
      rbias[mb] = ((hrow >= L.rlo && hrow <= L.rhi) ? 0.f : -INFINITY) - lse_n;
    }
#pragma unroll
    for (int kb = 0; kb < NKB; kb++) {
      const int cg0 = CR == 8 ? kb : 2 * kb, cg1 = CR == 8 ? kb : 2 * kb + 1;
      if (!(L.wave_ok && cg0 < P.ncg && 4 * cg0 <= L.wcol_hi && 4 * cg1 + 3 >= L.wcol_lo)) continue;
      const int key0 = (n >> 2) * HCW + 4 * wave + 4 * cg0 + (n & 3);
      f32x4 s[2], dp[2];
#pragma unroll
      for (int mb = 0; mb < 2; mb++) {
        s[mb] = f32x4{0.f, 0.f, 0.f, 0.f};
        dp[mb] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < KC; c++) {
          s[mb] = Mma<CT>::mfma(lds_read16(sK + (key0 + mb * MB_STEP) * PA + (32 * c + 8 * g) * 2), qf[c], s[mb]);
          dp[mb] = Mma<CT>::mfma(lds_read16(sV + (key0 + mb * MB_STEP) * PB + (32 * c + 8 * g) * 2), dof[c], dp[mb]);
        }
      }
      float ds[8];
#pragma unroll
      for (int mb = 0; mb < 2; mb++)
#pragma unroll
        for (int i = 0; i < 4; i++) {
          const int cg = mb == 0 ? cg0 : cg1;
          float nl = rbias[mb];
          if (L.cg_edge[cg]) nl = L.col_ok(cg, i) ? nl : -INFINITY;
          const float pv = fast_exp2(fmaf(s[mb][i], scale, nl));
          ds[4 * mb + i] = pv * (dp[mb][i] - del_n);
        }
      const u32x4 dsb = pack8<CT>(ds);
      const int kt0 = 4 * wave + 4 * cg0;
#pragma unroll
      for (int d = 0; d < DB; d++)
        dq_acc[d] = Mma<CT>::mfma(swa1_read_tokens_as_k(sK, PA, HCW, kt0, 16 * d, n, g, MB_STEP), dsb, dq_acc[d]);
    }
  };
  for (int ch = L.ch_first; ch < L.ch_last; ch++) {
    swa1_issue<NI, BAL, TAIL, 0>(srk, sp, on_k, kb_, sn2k, G, CR * ch + CR, rope_idx, (sp.t_off >> 1) < a.p.dk);
    swa1_issue<NI, BAL, TAIL, 1>(srv, sp, on_v, vb_, sn2v, G, CR * ch + CR, nullptr, (sp.t_off >> 1) < a.p.dv);
    consume(ch);
    if (LROT == 2) swa1_tab_issue(tr_srk, srk, sp, fwd_rope);
    __syncthreads();
    swa1_commit<CT, NI, BAL, LROT, TAIL, 0, PA>(srk, sp, sK, a.rope_pbit, fwd_rope, on_k, &tr_srk, (sp.t_off >> 1) < a.p.dk);
    swa1_commit<CT, NI, BAL, 0, TAIL, 1, PB>(srv, sp, sV, 1, no_rope, false, nullptr, (sp.t_off >> 1) < a.p.dv);
    __syncthreads();
  }
  consume(L.ch_last);
  __syncthreads();

  TIO* dqb = reinterpret_cast<TIO*>(a.dq) + b * a.dqs[0] + h * a.dqs[1];
  if (a.dq_vec != 0) {
    swa1_store_own<TIO, CT, D>(smem + wave * 16 * (D * 2 + 16), dq_acc, a.p.sm_scale, dqb, a.dqs[2], a.p.dk, G, wave, lane,
                               inv_rope, store_rope);
    return;
  }
  swa1_write_grad<TIO, D>(smem, dq_acc, a.p.sm_scale, dqb, a.dqs[2], a.dqs[3], a.p.dk, a.dq_vec != 0, L, store_rope ? inv_rope : no_rope, wave, n, g, tid);
}
