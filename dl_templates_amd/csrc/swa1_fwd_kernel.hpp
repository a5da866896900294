// Forward kernel for token grids (b_size == 1, the shape of every SWA config of the benchmark).
//
// Replaces tiled_swa_fwd_kernel (src/tiled_swa.py:15-133), whose idea it generalises: a 2D
// block of queries shares one K/V halo.  The halo is streamed through LDS in chunks of 8 rows
// (K and V side by side); while a chunk is being consumed the next one is already in flight
// from HBM into registers.  Per chunk a wave (one 4x4 query patch)
//   1. computes S^T = K Q^T for its NCG blocks of 8x4 keys,
//   2. scales and masks with additive per-column / per-row biases (the window test costs no
//      compare in the inner loop) and runs ONE online-softmax update for the whole chunk,
//   3. accumulates O^T += V^T P^T.
#pragma once
#include "swa1_common.hpp"

#ifndef SWA1_FWD_CR
#define SWA1_FWD_CR 4  // halo rows per chunk in the forward and dQ kernels
#endif
#ifndef SWA1_KV_CR
#define SWA1_KV_CR 4   // halo rows per chunk in the dK/dV kernel
#endif

struct Swa1FwdArgs {
  AttnProblem p;
  Swa1Plan plan;
  const void *q, *k, *v;
  void* o;
  float* lse;
  int64_t qs[4], ks[4], vs[4], os[4], ls[3];
  // optional side outputs of the fused rotation: the rotated q and k (NULL: not stored); rows of
  // element stride 1, 16-byte aligned
  void *q_rot, *k_rot;
  int64_t qrs[4], krs[4];
  int32_t q_vec, o_vec;
  int32_t rope_pbit;  // chunk distance between rotary partners (R / 8), 1 without rotation
  int32_t rope_mode;  // 0 none, 1 rotation with the plain staging map, 2 balanced staging map
  float scale_log2;
};

// CR: halo rows per chunk.  8: a 32-token block is 8 rows x 4 columns; 4: 4 rows x 8 columns
// (half the LDS and staging registers per workgroup, hence more resident workgroups per CU).
template <typename TIO, int D, int NCGMAX, int CR, int ROPE>
__global__ __launch_bounds__(256, (D <= 64 ? (CR == 4 ? (NCGMAX <= 4 ? 4 : 3) : 2) : (CR == 4 ? 2 : 1))) void swa1_fwd_kernel(const Swa1FwdArgs a) {
  typedef typename ComputeOf<TIO>::type CT;
  extern __shared__ __align__(16) char smem[];
  constexpr bool WIDE = ROPE == 0;  // padded-by-32 layout: kernels without rotation
  constexpr int PA = swa1_pitch(D, NCGMAX, 0, WIDE), PB = swa1_pitch(D, NCGMAX, 1, WIDE);  // K rows, V rows
  constexpr int KC = D / 32, VB = D / 16;
  constexpr int HCW = swa1_hcw(NCGMAX);
  constexpr int REGION = CR * HCW * PA;
  constexpr int NKB = CR == 8 ? NCGMAX : NCGMAX / 2;      // 32-token blocks per wave and chunk
  constexpr int MB_STEP = CR == 8 ? 4 * HCW : 4;          // token distance between the halves of a block
  static_assert(CR == 8 || NCGMAX % 2 == 0, "4-row chunks pair column groups");
  // Row sums: one extra MFMA against a row of ones per block (ONES); the VALU alternative is kept
  // for experiments.
  constexpr bool ONES = true;

  const int tid = threadIdx.x;
  const int lane = tid & 63, n = lane & 15, g = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const Swa1Plan& P = a.plan;
  char* sK = smem;
  char* sV = smem + REGION;

  const int lin = xcd_remap(blockIdx.x, gridDim.x);
  const int per_bh = P.nblk_r * P.nblk_c;
  const int bh = lin / per_bh;
  const int rem = lin - bh * per_bh;
  const int br = rem / P.nblk_c;
  const int b = bh / a.p.H, h = bh - b * a.p.H;
  Swa1Geom G;
  G.r0 = 4 * br; G.c0 = 16 * (rem - br * P.nblk_c);
  G.TR = a.p.g.TR; G.TC = a.p.g.TC; G.WR = a.p.g.WR; G.WC = a.p.g.WC;

  const TIO* qb = reinterpret_cast<const TIO*>(a.q) + b * a.qs[0] + h * a.qs[1];
  const TIO* kb_ = reinterpret_cast<const TIO*>(a.k) + b * a.ks[0] + h * a.ks[1];
  const TIO* vb_ = reinterpret_cast<const TIO*>(a.v) + b * a.vs[0] + h * a.vs[1];
  TIO* ob = reinterpret_cast<TIO*>(a.o) + b * a.os[0] + h * a.os[1];
  RopeDev no_rope = a.p.rope;
  no_rope.enabled = 0;
  constexpr bool use_rope = ROPE != 0;
  constexpr bool BAL = ROPE == 2;
  const int32_t* rope_idx = use_rope ? a.p.rope.idx : nullptr;

  // own queries: LDS row 16 w + n <-> grid (r0 + (n >> 2), c0 + 4 w + (n & 3))
  auto own_token = [&](int row) -> int64_t {
    const int r = G.r0 + ((row & 15) >> 2), c = G.c0 + 4 * (row >> 4) + (row & 3);
    return (r < G.TR && c < G.TC) ? (int64_t)r * G.TC + c : (int64_t)-1;
  };

  // halo rows that hold at least one grid row; chunks outside are skipped by the whole workgroup
  const int wrow_lo = dlt_imax(0, G.WR - G.r0), wrow_hi = dlt_imin(3 + 2 * G.WR, G.TR - 1 - G.r0 + G.WR);
  const int ch_first = wrow_lo / CR, ch_last = wrow_hi / CR;

  constexpr bool TAIL = ROPE == 0 && swa1_use_tail(D, HCW, CR);
  constexpr int NI = swa1_items_t(D, HCW, CR, TAIL);
  StagePlan<NI> sp;
  swa1_plan_init<D, HCW, CR, BAL, TAIL, WIDE, PA, PB>(sp, G, tid, a.rope_pbit);
  const bool on_k = (sp.coff[0] >> 1) < a.p.dk, on_v = (sp.coff[0] >> 1) < a.p.dv;
  const int sn2k = (int)a.ks[2] * 2, sn2v = (int)a.vs[2] * 2;
  const int64_t tq_own = own_token(16 * wave + n);
  StageRegs<NI> srk, srv;
  swa1_regs_zero(srk);
  TabRegs<NI> tr_srk;
  swa1_regs_zero(srv);
  swa1_issue<NI, BAL, TAIL, 0>(srk, sp, on_k, kb_, sn2k, G, CR * ch_first, rope_idx, (sp.t_off >> 1) < a.p.dk);
  swa1_issue<NI, BAL, TAIL, 1>(srv, sp, on_v, vb_, sn2v, G, CR * ch_first, nullptr, (sp.t_off >> 1) < a.p.dv);

  // own queries straight into B-operand fragments (rotated on the way when fused)
  u32x4 qf[KC];
  swa1_load_own<TIO, CT, D>(qf, qb, a.qs[2], a.p.dk, tq_own, g, a.p.rope, use_rope);
  // side outputs of the fused rotation (optional): this workgroup's own queries and keys, rotated
  const bool save_rot = use_rope && a.k_rot != nullptr;
  u32x4 kf_own[KC];
  if (save_rot) swa1_load_own<TIO, CT, D>(kf_own, kb_, a.ks[2], a.p.dk, tq_own, g, a.p.rope, true);

  // ---- window of this lane's query in halo coordinates -> additive biases
  const int qr_l = n >> 2, qc_l = n & 3;
  const int cw = G.c0 + 4 * wave;
  const bool q_ok = (G.r0 + qr_l < G.TR) && (cw + qc_l < G.TC);
  const int rlo = dlt_imax(qr_l, G.WR - G.r0), rhi = dlt_imin(qr_l + 2 * G.WR, G.TR - 1 - G.r0 + G.WR);
  const int clo = dlt_imax(qc_l, G.WC - cw), chi = dlt_imin(qc_l + 2 * G.WC, G.TC - 1 - cw + G.WC);
  // window columns of this wave that hold at least one grid column
  const int wcol_lo = dlt_imax(0, G.WC - cw), wcol_hi = G.TC - 1 - cw + G.WC;
  const bool wave_ok = cw < G.TC;
  // per-lane column window [clo, clo + cspan] in window coordinates (empty for a query outside the
  // grid); column groups whose 4 columns are inside every lane's window need no test (wave-uniform)
  const int cspan = q_ok ? chi - clo : -1;
  bool cg_edge[NCGMAX];
#pragma unroll
  for (int cg = 0; cg < NCGMAX; cg++)
    cg_edge[cg] = __builtin_amdgcn_ballot_w64(!((unsigned)(4 * cg - clo) <= (unsigned)cspan &&
                                                (unsigned)(4 * cg + 3 - clo) <= (unsigned)cspan)) != 0;

  // running max of the RAW scores (sm_scale > 0 keeps the order), sum in acc_l through an
  // extra MFMA whose A operand is a row of ones: row 0 of the result is sum_k P[k][query]
  float m_run = -INFINITY;
  f32x4 acc[VB], acc_l = {0.f, 0.f, 0.f, 0.f};
  float l_run = 0.f;  // per-lane partial row sum (only without the ones trick)
#pragma unroll
  for (int d = 0; d < VB; d++) acc[d] = f32x4{0.f, 0.f, 0.f, 0.f};
  const float scale = a.scale_log2;
  const unsigned one2 = pack2<CT>(1.f, 1.f);
  const u32x4 ones = n == 0 ? u32x4{one2, one2, one2, one2} : u32x4{0u, 0u, 0u, 0u};

  if (ROPE == 2) swa1_tab_issue(tr_srk, srk, sp, a.p.rope);
  swa1_commit<CT, NI, BAL, ROPE, TAIL, 0, PA>(srk, sp, sK, a.rope_pbit, a.p.rope, on_k, &tr_srk, (sp.t_off >> 1) < a.p.dk);
  swa1_commit<CT, NI, BAL, 0, TAIL, 1, PB>(srv, sp, sV, 1, a.p.rope, false, nullptr, (sp.t_off >> 1) < a.p.dv);
  __syncthreads();
  pin_loaded(qf);
  if (save_rot && tq_own >= 0) {
    TIO* qr = reinterpret_cast<TIO*>(a.q_rot) + b * a.qrs[0] + h * a.qrs[1] + tq_own * a.qrs[2];
    TIO* kr = reinterpret_cast<TIO*>(a.k_rot) + b * a.krs[0] + h * a.krs[1] + tq_own * a.krs[2];
#pragma unroll
    for (int c = 0; c < KC; c++) {
      const int ch = 4 * c + g;
      if (8 * ch < a.p.dk) {
        store_stream16(qr + 8 * ch, qf[c]);
        store_stream16(kr + 8 * ch, kf_own[c]);
      }
    }
  }

  // products and softmax update of the chunk resident in LDS
  auto consume = [&](const int ch) {
    const int cr0 = CR * ch;

    // block kb, half mb -> (row offset inside the chunk, column group)
    float t[NKB][8];
    float mloc = -INFINITY;
    float rbias[2];
#pragma unroll
    for (int mb = 0; mb < 2; mb++) {
      const int hrow = cr0 + (CR == 8 ? 4 * mb : 0) + g;
      rbias[mb] = (hrow >= rlo && hrow <= rhi) ? 0.f : -INFINITY;
    }
    const bool row_edge = __builtin_amdgcn_ballot_w64(rbias[0] != 0.f || rbias[1] != 0.f) != 0;
    bool on[NKB];
#pragma unroll
    for (int kb = 0; kb < NKB; kb++) {
      const int cg0 = CR == 8 ? kb : 2 * kb, cg1 = CR == 8 ? kb : 2 * kb + 1;
      on[kb] = wave_ok && cg0 < P.ncg && 4 * cg0 <= wcol_hi && 4 * cg1 + 3 >= wcol_lo;
      if (on[kb]) {
        const int key0 = (n >> 2) * HCW + 4 * wave + 4 * cg0 + (n & 3);
        f32x4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < KC; c++) {
          const u32x4 k0 = lds_read16(sK + key0 * PA + (32 * c + 8 * g) * 2);
          const u32x4 k1 = lds_read16(sK + (key0 + MB_STEP) * PA + (32 * c + 8 * g) * 2);
          s0 = Mma<CT>::mfma(k0, qf[c], s0);
          s1 = Mma<CT>::mfma(k1, qf[c], s1);
        }
#pragma unroll
        for (int i = 0; i < 4; i++) { t[kb][i] = s0[i]; t[kb][4 + i] = s1[i]; }
        if (cg_edge[cg0] || cg_edge[cg1]) {
#pragma unroll
          for (int i = 0; i < 4; i++) {
            t[kb][i] = (unsigned)(4 * cg0 + i - clo) <= (unsigned)cspan ? t[kb][i] : -INFINITY;
            t[kb][4 + i] = (unsigned)(4 * cg1 + i - clo) <= (unsigned)cspan ? t[kb][4 + i] : -INFINITY;
          }
        }
        if (row_edge) {
#pragma unroll
          for (int i = 0; i < 4; i++) { t[kb][i] += rbias[0]; t[kb][4 + i] += rbias[1]; }
        }
        mloc = fmaxf(mloc, fmaxf(fmaxf(fmaxf(t[kb][0], t[kb][1]), fmaxf(t[kb][2], t[kb][3])),
                                 fmaxf(fmaxf(t[kb][4], t[kb][5]), fmaxf(t[kb][6], t[kb][7]))));
      } else {
#pragma unroll
        for (int i = 0; i < 8; i++) t[kb][i] = -INFINITY;
      }
    }
    // one online-softmax update per chunk: p = exp2(s * scale - m * scale)
    mloc = wave_max4(mloc);
    const float m_new = fmaxf(m_run, mloc);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = fast_exp2((m_run - m_use) * scale);
    const float neg_m2 = -m_use * scale;
    m_run = m_new;
    u32x4 pb[NKB];
    float psum = 0.f;
#pragma unroll
    for (int kb = 0; kb < NKB; kb++) {
#pragma unroll
      for (int i = 0; i < 8; i++) {
        t[kb][i] = fast_exp2(fmaf(t[kb][i], scale, neg_m2));
        if (!ONES) psum += t[kb][i];
      }
      pb[kb] = pack8<CT>(t[kb]);
    }
    if (!ONES) l_run = l_run * alpha + psum;
    if (__builtin_amdgcn_ballot_w64(alpha != 1.f)) {
#pragma unroll
      for (int d = 0; d < VB; d++) acc[d] *= alpha;
      if (ONES) acc_l *= alpha;
    }
#pragma unroll
    for (int kb = 0; kb < NKB; kb++) {
      if (on[kb]) {
        const int key0 = 4 * wave + 4 * (CR == 8 ? kb : 2 * kb);
        if (D > 64) {
          // two waves per SIMD: V^T fragments are requested four at a time ahead of their products, so that
          // one LDS latency is paid per group instead of one per product
#pragma unroll
          for (int d0 = 0; d0 < VB; d0 += 4) {
            u32x4 vfr[4];
#pragma unroll
            for (int d = 0; d < 4; d++) vfr[d] = swa1_read_tokens_as_k(sV, PB, HCW, key0, 16 * (d0 + d), n, g, MB_STEP);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int d = 0; d < 4; d++) acc[d0 + d] = Mma<CT>::mfma(vfr[d], pb[kb], acc[d0 + d]);
          }
        } else {
#pragma unroll
          for (int d = 0; d < VB; d++)
            acc[d] = Mma<CT>::mfma(swa1_read_tokens_as_k(sV, PB, HCW, key0, 16 * d, n, g, MB_STEP), pb[kb], acc[d]);
        }
        if (ONES) acc_l = Mma<CT>::mfma(ones, pb[kb], acc_l);
      }
    }
  };
  // The last chunk is peeled off so that inside the loop the prefetch and the commit are
  // unconditional: with `if (has_next)` around each, the compiler sees a path on which loads stay
  // pending across the back edge and guards every later load with a full vmcnt(0) wait.
  for (int ch = ch_first; ch < ch_last; ch++) {
    // next chunk: HBM -> registers while this one is consumed
    swa1_issue<NI, BAL, TAIL, 0>(srk, sp, on_k, kb_, sn2k, G, CR * ch + CR, rope_idx, (sp.t_off >> 1) < a.p.dk);
    swa1_issue<NI, BAL, TAIL, 1>(srv, sp, on_v, vb_, sn2v, G, CR * ch + CR, nullptr, (sp.t_off >> 1) < a.p.dv);
    consume(ch);
    if (ROPE == 2) swa1_tab_issue(tr_srk, srk, sp, a.p.rope);  // table rows of the next chunk's tokens, ahead of the barrier
    __syncthreads();  // every wave is done with this chunk
    swa1_commit<CT, NI, BAL, ROPE, TAIL, 0, PA>(srk, sp, sK, a.rope_pbit, a.p.rope, on_k, &tr_srk, (sp.t_off >> 1) < a.p.dk);
    swa1_commit<CT, NI, BAL, 0, TAIL, 1, PB>(srv, sp, sV, 1, a.p.rope, false, nullptr, (sp.t_off >> 1) < a.p.dv);
    __syncthreads();
  }
  consume(ch_last);
  __syncthreads();

  // ---- epilogue
  typedef typename TileOf<TIO>::type TL;
  constexpr int PO = D * (int)sizeof(TL) + 16;
  // row 0 of the ones product lives in lane group 0; per-lane partial sums are added over the 4 groups
  const float lt = wave_sum4(ONES ? acc_l[0] : l_run);   // ones product: only lane group 0 is non-zero
  const float inv = lt > 0.f ? fast_rcp(lt) : 0.f;
  const int64_t tq = own_token(16 * wave + n);
  if (g == 0 && tq >= 0) store_stream4(a.lse + (b * a.ls[0] + h * a.ls[1] + tq * a.ls[2]), m_run * scale + fast_log2(lt));
  if (a.o_vec != 0) {  // the loop ended with a workgroup barrier: the chunk buffers are free
    swa1_store_own<TIO, CT, D>(smem + wave * 16 * PO, acc, inv, ob, a.os[2], a.p.dv, G, wave, lane, no_rope, false);
    return;
  }
  TL* orow = reinterpret_cast<TL*>(smem + (16 * wave + n) * PO);
#pragma unroll
  for (int d = 0; d < VB; d++)
#pragma unroll
    for (int i = 0; i < 4; i++) orow[16 * d + 4 * g + i] = (TL)(acc[d][i] * inv);
  __syncthreads();
  store_tile<TIO, TL, D>(smem, PO, ob, a.os[2], a.os[3], a.p.dv, a.o_vec != 0, 64, own_token, no_rope, tid);
}
