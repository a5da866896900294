// Backward attention kernels (windowed 2D and dense) for gfx950.
//
// Replaces tiled_swa_bwd_preprocess_kernel and tiled_swa_bwd_large_kernel_decoupled_q
// (src/tiled_swa.py:253-282, :407-562) and _attn_bwd_preprocess / _attn_bwd
// (src/flash_attn.py:186-449).  Same decoupled structure as the reference, hence no atomics
// and bit-reproducible gradients:
//   delta kernel : delta = rowsum(o * do)
//   dK/dV kernel : a workgroup owns 64*NP keys and streams the queries whose window holds
//                  them (Q, dO, lse2, delta) through LDS;  P = exp2(S2 - lse2) is recomputed,
//                  dV^T += dO^T P, dP = dO V^T, dS = P (dP - delta), dK^T += Q^T dS
//   dQ kernel    : a workgroup owns 64*NP queries and streams their keys / values;
//                  dQ^T += K^T dS^T
// Tokens of the streamed side are always the MFMA rows, so P / dS come out of the first
// product in the layout the second product wants as its B operand; the [token][dim] LDS tiles
// are read a second time through the transposing LDS read for the token-contracted products.
#pragma once
#include "attn_common.hpp"

struct BwdArgs {
  AttnProblem p;
  AttnPlan plan;
  const void *q, *k, *v, *o, *d_o;
  const float* lse;
  float* delta;
  void *dq, *dk, *dv;
  int64_t qs[5], ks[5], vs[5], os[5], dos[5], dqs[5], dks[5], dvs[5], ls[3];
  int32_t q_vec, k_vec, v_vec, o_vec, do_vec, dq_vec, dk_vec, dv_vec;
  float scale_log2;
  int64_t n_tokens_q;  // tokens per (batch, head) on the query side
};

// ---- delta = rowsum(o * do), one 8-dim chunk per thread, reduced over the DV/8 lanes of a token
template <typename TIO, int DV>
__global__ __launch_bounds__(256) void attn_delta_kernel(const BwdArgs a) {
  typedef typename ComputeOf<TIO>::type CT;
  constexpr int CH = DV / 8;
  const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int c = (int)(gid % CH);
  const int64_t tok = gid / CH;
  const int64_t total = (int64_t)a.p.B * a.p.H * a.n_tokens_q;
  float part = 0.f;
  int64_t bh = 0, nn = 0;
  if (tok < total) {
    bh = tok / a.n_tokens_q;
    nn = tok - bh * a.n_tokens_q;
    const int b = (int)(bh / a.p.H), h = (int)(bh - (int64_t)b * a.p.H);
    const int nvalid = dlt_imin(8, a.p.dv - 8 * c);
    if (nvalid > 0) {
      const TIO* po = reinterpret_cast<const TIO*>(a.o) + b * a.os[0] + h * a.os[1] + tok_addr(a.os, a.p.tm)(nn) + (int64_t)8 * c * a.os[3];
      const TIO* pd = reinterpret_cast<const TIO*>(a.d_o) + b * a.dos[0] + h * a.dos[1] + tok_addr(a.dos, a.p.tm)(nn) + (int64_t)8 * c * a.dos[3];
      if (sizeof(TIO) == 4) {
        // dO rounded as the products of the main kernel see it (o is what the forward pass stored): delta then equals
        // sum_k P dP of those products, and gradients that cancel (a query that sees one key) cancel here too
#pragma unroll
        for (int j = 0; j < 8; j++)
          if (j < nvalid) part += (float)po[j * a.os[3]] * unpack_lo<CT>(pack2<CT>((float)pd[j * a.dos[3]], 0.f));
      } else {
        float fo[8], fd[8];
        unpack8<CT>(Io<TIO, CT>::load8(po, a.o_vec != 0, a.os[3], nvalid), fo);
        unpack8<CT>(Io<TIO, CT>::load8(pd, a.do_vec != 0, a.dos[3], nvalid), fd);
#pragma unroll
        for (int j = 0; j < 8; j++) part += fo[j] * fd[j];
      }
    }
  }
#pragma unroll
  for (int off = 1; off < CH; off <<= 1) part += __shfl_xor(part, off);
  if (tok < total && c == 0) {
    const int b = (int)(bh / a.p.H), h = (int)(bh - (int64_t)b * a.p.H);
    store_stream4(a.delta + (b * a.ls[0] + h * a.ls[1] + nn * a.ls[2]), part);
  }
}

// per-token fp32 vector (lse2 / delta) -> LDS, zero for tokens outside the grid
template <typename TokFn>
DLT_DEV void stage_scalars(float* s, const float* base, int64_t stride, int n, TokFn tok, int tid) {
  for (int i = tid; i < n; i += 256) {
    const int64_t t = tok(i);
    s[i] = t >= 0 ? base[t * stride] : 0.f;
  }
}

// accumulators (C layout, [dim][own token]) -> LDS tile [own token][dim] -> HBM rows
template <typename TIO, int D, int NP, typename Ctx, typename SN>
DLT_DEV void write_grad_tile(char* sT, f32x4 (&acc)[NP][D / 16], float mul, TIO* base, const SN& sn, int64_t sd, int dact,
                             bool vec, const Ctx& T, const RopeDev& rope, int wave, int n, int g, int tid) {
  typedef typename TileOf<TIO>::type TL;
  constexpr int PT = D * (int)sizeof(TL) + 16;
#pragma unroll
  for (int p = 0; p < NP; p++) {
    TL* row = reinterpret_cast<TL*>(sT + (wave * 16 * NP + 16 * p + n) * PT);
#pragma unroll
    for (int d = 0; d < D / 16; d++)
#pragma unroll
      for (int i = 0; i < 4; i++) row[16 * d + 4 * g + i] = (TL)(acc[p][d][i] * mul);
  }
  __syncthreads();
  store_tile<TIO, TL, D>(sT, PT, base, sn, sd, dact, vec, 64 * NP, [&](int r) { return T.own_token(r); }, rope, tid);
  __syncthreads();
}

// =============================================================================================
// dK / dV
template <typename TIO, int DK, int DV, int NP>
__global__ __launch_bounds__(256) void attn_bwd_kv_kernel(const BwdArgs a) {
  typedef typename ComputeOf<TIO>::type CT;
  extern __shared__ __align__(16) char smem[];
  // fp32 tensors: q and k are staged as hi + lo bf16 pairs (stage_tile_split) and a score is three products, as in the
  // forward kernel whose log-sum-exp the probabilities are recomputed against; dK / dQ contract over the hi parts
  constexpr bool SPLIT = sizeof(TIO) == 4;
  constexpr int PQ = DK * (SPLIT ? 4 : 2) + 16, PV = DV * 2 + 16;
  constexpr int OWN = 64 * NP;
  constexpr int KC = DK / 32, VC = DV / 32, KB = DK / 16, VB = DV / 16;

  const int tid = threadIdx.x;
  const int lane = tid & 63, n = lane & 15, g = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const DltGeom& G = a.p.g;

  TileCtx<NP, true> T;
  T.init(G, a.plan, a.p.H, wave, n);
  const int b = T.b, h = T.h;
  const int rlo = T.rlo, rhi = T.rhi, X0 = T.X0, X1 = T.X1, wxlo = T.wxlo, wxhi = T.wxhi;

  char* sOwnK = smem;                 // own K tile, then the gradient tiles of the epilogue
  char* sOwnV = smem + OWN * PQ;      // own V tile
  char* sQ = smem + a.plan.off_a;     // halo: Q  [tok][PQ]
  char* sDO = smem + a.plan.off_b;    // halo: dO [tok][PV]
  float* sLse = reinterpret_cast<float*>(smem + a.plan.off_c);
  float* sDel = reinterpret_cast<float*>(smem + a.plan.off_d);

  const TIO* qb = reinterpret_cast<const TIO*>(a.q) + b * a.qs[0] + h * a.qs[1];
  const TIO* kb_ = reinterpret_cast<const TIO*>(a.k) + b * a.ks[0] + h * a.ks[1];
  const TIO* vb_ = reinterpret_cast<const TIO*>(a.v) + b * a.vs[0] + h * a.vs[1];
  const TIO* dob = reinterpret_cast<const TIO*>(a.d_o) + b * a.dos[0] + h * a.dos[1];
  const float* lseb = a.lse + b * a.ls[0] + h * a.ls[1];
  const float* delb = a.delta + b * a.ls[0] + h * a.ls[1];
  RopeDev fwd_rope = a.p.rope;  fwd_rope.inverse = 0;
  if (a.p.rope_prerot) fwd_rope.enabled = 0;  // q and k arrive rotated
  RopeDev inv_rope = a.p.rope;  inv_rope.inverse = 1;
  RopeDev no_rope = a.p.rope;   no_rope.enabled = 0;

  // ---- own keys / values -> B-operand fragments (head dim along k)
  stage_tile_qk<TIO, CT, DK>(sOwnK, PQ, kb_, tok_addr(a.ks, a.p.tm), a.ks[3], a.p.dk, a.k_vec != 0, OWN,
                          [&](int row) { return T.own_token(row); }, fwd_rope, tid);
  stage_tile<TIO, CT, DV>(sOwnV, PV, vb_, tok_addr(a.vs, a.p.tm), a.vs[3], a.p.dv, a.v_vec != 0, OWN,
                          [&](int row) { return T.own_token(row); }, no_rope, tid);
  __syncthreads();
  u32x4 kf[NP][KC], klo[SPLIT ? NP : 1][KC], vf[NP][VC];
#pragma unroll
  for (int p = 0; p < NP; p++) {
    const int row = wave * 16 * NP + 16 * p + n;
#pragma unroll
    for (int c = 0; c < KC; c++) {
      kf[p][c] = lds_read16(sOwnK + row * PQ + (32 * c + 8 * g) * 2);
      if constexpr (SPLIT) klo[p][c] = lds_read16(sOwnK + row * PQ + DK * 2 + (32 * c + 8 * g) * 2);
    }
#pragma unroll
    for (int c = 0; c < VC; c++) vf[p][c] = lds_read16(sOwnV + row * PV + (32 * c + 8 * g) * 2);
  }

  f32x4 dk_acc[NP][KB], dv_acc[NP][VB];
#pragma unroll
  for (int p = 0; p < NP; p++) {
#pragma unroll
    for (int d = 0; d < KB; d++) dk_acc[p][d] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int d = 0; d < VB; d++) dv_acc[p][d] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  const int CX = a.plan.chunk_x;
  const bool rowfit = a.plan.rowfit != 0;
  const float scale = a.scale_log2;
  bool first_chunk = true;

  for (int kr0 = rlo; kr0 <= rhi; kr0 += a.plan.chunk_rows) {
    const int nr = dlt_imin(a.plan.chunk_rows, rhi - kr0 + 1);
    for (int cx0 = X0; cx0 < X1; cx0 += rowfit ? 0x40000000 : CX) {
      const int stage_w = rowfit ? dlt_imin(CX, X1 - cx0 + 32) : CX;
      if (!first_chunk) __syncthreads();
      first_chunk = false;
      for (int ri = 0; ri < nr; ri++) {
        const int64_t row_tok0 = (int64_t)(kr0 + ri) * G.XLq + cx0;
        auto tok = [&](int xi) { return cx0 + xi < G.XLq ? row_tok0 + xi : (int64_t)-1; };
        stage_tile_qk<TIO, CT, DK>(sQ + ri * CX * PQ, PQ, qb, tok_addr(a.qs, a.p.tm), a.qs[3], a.p.dk, a.q_vec != 0, stage_w, tok, fwd_rope, tid);
        stage_tile<TIO, CT, DV>(sDO + ri * CX * PV, PV, dob, tok_addr(a.dos, a.p.tm), a.dos[3], a.p.dv, a.do_vec != 0, stage_w, tok, no_rope, tid);
        stage_scalars(sLse + ri * CX, lseb, a.ls[2], stage_w, tok, tid);
        stage_scalars(sDel + ri * CX, delb, a.ls[2], stage_w, tok, tid);
      }
      __syncthreads();

      const int kstart = rowfit ? wxlo : cx0;
      const int kend = rowfit ? wxhi : dlt_imin(wxhi, cx0 + CX);
      for (int ri = 0; ri < nr; ri++) {
        for (int kx0 = kstart; kx0 < kend; kx0 += 32) {
          if (kx0 + 32 <= wxlo) continue;
          const int kb = ri * CX + (kx0 - cx0);
          u32x4 qa[2][KC], ql[SPLIT ? 2 : 1][KC], da[2][VC];
          float lq[8], dq_[8];
#pragma unroll
          for (int mb = 0; mb < 2; mb++) {
#pragma unroll
            for (int c = 0; c < KC; c++) {
              qa[mb][c] = lds_read16(sQ + (kb + 16 * mb + n) * PQ + (32 * c + 8 * g) * 2);
              if constexpr (SPLIT) ql[mb][c] = lds_read16(sQ + (kb + 16 * mb + n) * PQ + DK * 2 + (32 * c + 8 * g) * 2);
            }
#pragma unroll
            for (int c = 0; c < VC; c++) da[mb][c] = lds_read16(sDO + (kb + 16 * mb + n) * PV + (32 * c + 8 * g) * 2);
#pragma unroll
            for (int i = 0; i < 4; i++) {
              lq[4 * mb + i] = sLse[kb + 16 * mb + 4 * g + i];
              dq_[4 * mb + i] = sDel[kb + 16 * mb + 4 * g + i];
            }
          }
#pragma unroll
          for (int p = 0; p < NP; p++) {
            if (T.patch_skips(p, kx0)) continue;
            f32x4 s[2], dp[2];
#pragma unroll
            for (int mb = 0; mb < 2; mb++) {
              s[mb] = f32x4{0.f, 0.f, 0.f, 0.f};
              dp[mb] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
              for (int c = 0; c < KC; c++) {
                if constexpr (SPLIT) {   // same order as the forward kernel: lo * hi, hi * lo, hi * hi
                  s[mb] = Mma<CT>::mfma(qa[mb][c], klo[p][c], s[mb]);
                  s[mb] = Mma<CT>::mfma(ql[mb][c], kf[p][c], s[mb]);
                }
                s[mb] = Mma<CT>::mfma(qa[mb][c], kf[p][c], s[mb]);
              }
#pragma unroll
              for (int c = 0; c < VC; c++) dp[mb] = Mma<CT>::mfma(da[mb][c], vf[p][c], dp[mb]);
            }
            float pr[8], ds[8];
            const bool need_mask = T.patch_needs_mask(p, kx0);
#pragma unroll
            for (int mb = 0; mb < 2; mb++)
#pragma unroll
              for (int i = 0; i < 4; i++) {
                const int e = 4 * mb + i;
                float pv = fast_exp2(s[mb][i] * scale - lq[e]);
                if (need_mask) pv = T.valid(p, kx0, g, mb, i) ? pv : 0.f;
                pr[e] = pv;
                ds[e] = pv * (dp[mb][i] - dq_[e]);
              }
            const u32x4 pb = pack8<CT>(pr), dsb = pack8<CT>(ds);
#pragma unroll
            for (int d = 0; d < VB; d++)
              dv_acc[p][d] = Mma<CT>::mfma(lds_read_tokens_as_k(sDO, PV, kb, 16 * d, n, g), pb, dv_acc[p][d]);
#pragma unroll
            for (int d = 0; d < KB; d++)
              dk_acc[p][d] = Mma<CT>::mfma(lds_read_tokens_as_k(sQ, PQ, kb, 16 * d, n, g), dsb, dk_acc[p][d]);
          }
        }
      }
    }
  }

  __syncthreads();
  TIO* dkb = reinterpret_cast<TIO*>(a.dk) + b * a.dks[0] + h * a.dks[1];
  TIO* dvb = reinterpret_cast<TIO*>(a.dv) + b * a.dvs[0] + h * a.dvs[1];
  write_grad_tile<TIO, DK, NP>(smem, dk_acc, a.p.sm_scale, dkb, tok_addr(a.dks, a.p.tm), a.dks[3], a.p.dk, a.dk_vec != 0, T, inv_rope, wave, n, g, tid);
  write_grad_tile<TIO, DV, NP>(smem, dv_acc, 1.0f, dvb, tok_addr(a.dvs, a.p.tm), a.dvs[3], a.p.dv, a.dv_vec != 0, T, no_rope, wave, n, g, tid);
}

// =============================================================================================
// dQ
template <typename TIO, int DK, int DV, int NP>
__global__ __launch_bounds__(256) void attn_bwd_q_kernel(const BwdArgs a) {
  typedef typename ComputeOf<TIO>::type CT;
  extern __shared__ __align__(16) char smem[];
  constexpr bool SPLIT = sizeof(TIO) == 4;   // see the dK / dV kernel
  constexpr int PQ = DK * (SPLIT ? 4 : 2) + 16, PV = DV * 2 + 16;
  constexpr int OWN = 64 * NP;
  constexpr int KC = DK / 32, VC = DV / 32, KB = DK / 16;

  const int tid = threadIdx.x;
  const int lane = tid & 63, n = lane & 15, g = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const DltGeom& G = a.p.g;

  TileCtx<NP, false> T;
  T.init(G, a.plan, a.p.H, wave, n);
  const int b = T.b, h = T.h;
  const int rlo = T.rlo, rhi = T.rhi, X0 = T.X0, X1 = T.X1, wxlo = T.wxlo, wxhi = T.wxhi;

  char* sOwnQ = smem;
  char* sOwnDO = smem + OWN * PQ;
  char* sK = smem + a.plan.off_a;
  char* sV = smem + a.plan.off_b;

  const TIO* qb = reinterpret_cast<const TIO*>(a.q) + b * a.qs[0] + h * a.qs[1];
  const TIO* kb_ = reinterpret_cast<const TIO*>(a.k) + b * a.ks[0] + h * a.ks[1];
  const TIO* vb_ = reinterpret_cast<const TIO*>(a.v) + b * a.vs[0] + h * a.vs[1];
  const TIO* dob = reinterpret_cast<const TIO*>(a.d_o) + b * a.dos[0] + h * a.dos[1];
  RopeDev fwd_rope = a.p.rope;  fwd_rope.inverse = 0;
  if (a.p.rope_prerot) fwd_rope.enabled = 0;  // q and k arrive rotated
  RopeDev inv_rope = a.p.rope;  inv_rope.inverse = 1;
  RopeDev no_rope = a.p.rope;   no_rope.enabled = 0;

  stage_tile_qk<TIO, CT, DK>(sOwnQ, PQ, qb, tok_addr(a.qs, a.p.tm), a.qs[3], a.p.dk, a.q_vec != 0, OWN,
                          [&](int row) { return T.own_token(row); }, fwd_rope, tid);
  stage_tile<TIO, CT, DV>(sOwnDO, PV, dob, tok_addr(a.dos, a.p.tm), a.dos[3], a.p.dv, a.do_vec != 0, OWN,
                          [&](int row) { return T.own_token(row); }, no_rope, tid);
  __syncthreads();
  u32x4 qf[NP][KC], qlo[SPLIT ? NP : 1][KC], dof[NP][VC];
  float lse_q[NP], del_q[NP];
#pragma unroll
  for (int p = 0; p < NP; p++) {
    const int row = wave * 16 * NP + 16 * p + n;
#pragma unroll
    for (int c = 0; c < KC; c++) {
      qf[p][c] = lds_read16(sOwnQ + row * PQ + (32 * c + 8 * g) * 2);
      if constexpr (SPLIT) qlo[p][c] = lds_read16(sOwnQ + row * PQ + DK * 2 + (32 * c + 8 * g) * 2);
    }
#pragma unroll
    for (int c = 0; c < VC; c++) dof[p][c] = lds_read16(sOwnDO + row * PV + (32 * c + 8 * g) * 2);
    const int64_t t = T.own_token(wave * 16 * NP + 16 * p + n);
    const int64_t off = b * a.ls[0] + h * a.ls[1] + (t >= 0 ? t : 0) * a.ls[2];
    lse_q[p] = t >= 0 ? a.lse[off] : 0.f;
    del_q[p] = t >= 0 ? a.delta[off] : 0.f;
  }

  f32x4 dq_acc[NP][KB];
#pragma unroll
  for (int p = 0; p < NP; p++)
#pragma unroll
    for (int d = 0; d < KB; d++) dq_acc[p][d] = f32x4{0.f, 0.f, 0.f, 0.f};

  const int CX = a.plan.chunk_x;
  const bool rowfit = a.plan.rowfit != 0;
  const float scale = a.scale_log2;
  bool first_chunk = true;

  for (int kr0 = rlo; kr0 <= rhi; kr0 += a.plan.chunk_rows) {
    const int nr = dlt_imin(a.plan.chunk_rows, rhi - kr0 + 1);
    for (int cx0 = X0; cx0 < X1; cx0 += rowfit ? 0x40000000 : CX) {
      const int stage_w = rowfit ? dlt_imin(CX, X1 - cx0 + 32) : CX;
      if (!first_chunk) __syncthreads();
      first_chunk = false;
      for (int ri = 0; ri < nr; ri++) {
        const int64_t row_tok0 = (int64_t)(kr0 + ri) * G.XLk + cx0;
        auto tok = [&](int xi) { return cx0 + xi < G.XLk ? row_tok0 + xi : (int64_t)-1; };
        stage_tile_qk<TIO, CT, DK>(sK + ri * CX * PQ, PQ, kb_, tok_addr(a.ks, a.p.tm), a.ks[3], a.p.dk, a.k_vec != 0, stage_w, tok, fwd_rope, tid);
        stage_tile<TIO, CT, DV>(sV + ri * CX * PV, PV, vb_, tok_addr(a.vs, a.p.tm), a.vs[3], a.p.dv, a.v_vec != 0, stage_w, tok, no_rope, tid);
      }
      __syncthreads();

      const int kstart = rowfit ? wxlo : cx0;
      const int kend = rowfit ? wxhi : dlt_imin(wxhi, cx0 + CX);
      for (int ri = 0; ri < nr; ri++) {
        for (int kx0 = kstart; kx0 < kend; kx0 += 32) {
          if (kx0 + 32 <= wxlo) continue;
          const int kb = ri * CX + (kx0 - cx0);
          u32x4 ka[2][KC], kl[SPLIT ? 2 : 1][KC], va[2][VC], kt[KB];
#pragma unroll
          for (int mb = 0; mb < 2; mb++) {
#pragma unroll
            for (int c = 0; c < KC; c++) {
              ka[mb][c] = lds_read16(sK + (kb + 16 * mb + n) * PQ + (32 * c + 8 * g) * 2);
              if constexpr (SPLIT) kl[mb][c] = lds_read16(sK + (kb + 16 * mb + n) * PQ + DK * 2 + (32 * c + 8 * g) * 2);
            }
#pragma unroll
            for (int c = 0; c < VC; c++) va[mb][c] = lds_read16(sV + (kb + 16 * mb + n) * PV + (32 * c + 8 * g) * 2);
          }
#pragma unroll
          for (int d = 0; d < KB; d++) kt[d] = lds_read_tokens_as_k(sK, PQ, kb, 16 * d, n, g);
#pragma unroll
          for (int p = 0; p < NP; p++) {
            if (T.patch_skips(p, kx0)) continue;
            f32x4 s[2], dp[2];
#pragma unroll
            for (int mb = 0; mb < 2; mb++) {
              s[mb] = f32x4{0.f, 0.f, 0.f, 0.f};
              dp[mb] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
              for (int c = 0; c < KC; c++) {
                if constexpr (SPLIT) {
                  s[mb] = Mma<CT>::mfma(kl[mb][c], qf[p][c], s[mb]);
                  s[mb] = Mma<CT>::mfma(ka[mb][c], qlo[p][c], s[mb]);
                }
                s[mb] = Mma<CT>::mfma(ka[mb][c], qf[p][c], s[mb]);
              }
#pragma unroll
              for (int c = 0; c < VC; c++) dp[mb] = Mma<CT>::mfma(va[mb][c], dof[p][c], dp[mb]);
            }
            float ds[8];
            const bool need_mask = T.patch_needs_mask(p, kx0);
#pragma unroll
            for (int mb = 0; mb < 2; mb++)
#pragma unroll
              for (int i = 0; i < 4; i++) {
                float pv = fast_exp2(s[mb][i] * scale - lse_q[p]);
                if (need_mask) pv = T.valid(p, kx0, g, mb, i) ? pv : 0.f;
                ds[4 * mb + i] = pv * (dp[mb][i] - del_q[p]);
              }
            const u32x4 dsb = pack8<CT>(ds);
#pragma unroll
            for (int d = 0; d < KB; d++) dq_acc[p][d] = Mma<CT>::mfma(kt[d], dsb, dq_acc[p][d]);
          }
        }
      }
    }
  }

  __syncthreads();
  TIO* dqb = reinterpret_cast<TIO*>(a.dq) + b * a.dqs[0] + h * a.dqs[1];
  write_grad_tile<TIO, DK, NP>(smem, dq_acc, a.p.sm_scale, dqb, tok_addr(a.dqs, a.p.tm), a.dqs[3], a.p.dk, a.dq_vec != 0, T, inv_rope, wave, n, g, tid);
}
