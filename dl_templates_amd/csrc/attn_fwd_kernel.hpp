// Forward attention kernel (windowed 2D and dense) for gfx950.
//
// Replaces tiled_swa_fwd_kernel / tiled_swa_fwd_large_kernel (src/tiled_swa.py:15-244) and
// _attn_fwd (src/flash_attn.py:81-172).
//
// Work split: a workgroup of 4 waves owns 64*NP consecutive queries of one grid row of one
// (batch, head); each wave owns NP blocks of 16 queries.  The keys/values those queries may
// attend (their halo: grid rows [rlo, rhi], x in [X0, X1)) are streamed through LDS in
// chunks; every wave computes S^T = K Q^T per 32-key block with bf16/fp16 MFMA (keys are the
// MFMA rows, so the fp32 result already has the layout of the B operand of O^T += V^T P^T),
// applies the window mask from per-lane [xlo, xhi) intervals, and keeps an online softmax in
// the log2 domain (running max via two cross-lane exchanges, running sum per lane).
#pragma once
#include "attn_common.hpp"

struct FwdArgs {
  AttnProblem p;
  AttnPlan plan;
  const void *q, *k, *v;
  void* o;
  float* lse;
  int64_t qs[5], ks[5], vs[5], os[5], ls[3];
  int32_t q_vec, k_vec, v_vec, o_vec;
  float scale_log2;
};

template <typename TIO, int DK, int DV, int NP>
__global__ __launch_bounds__(256) void attn_fwd_kernel(const FwdArgs a) {
  typedef typename ComputeOf<TIO>::type CT;
  typedef typename TileOf<TIO>::type TL;
  extern __shared__ __align__(16) char smem[];
  // fp32 tensors: q and k are staged as hi + lo bf16 pairs (stage_tile_split) and a score is three products
  constexpr bool SPLIT = sizeof(TIO) == 4;
  constexpr int PQ = DK * (SPLIT ? 4 : 2) + 16, PK = PQ, PV = DV * 2 + 16;
  constexpr int PO = DV * (int)sizeof(TL) + 16;
  constexpr int OWN = 64 * NP;
  constexpr int KC = DK / 32, VB = DV / 16;

  const int tid = threadIdx.x;
  const int lane = tid & 63, n = lane & 15, g = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const DltGeom& G = a.p.g;

  TileCtx<NP, false> T;
  T.init(G, a.plan, a.p.H, wave, n);
  const int b = T.b, h = T.h, r_own = T.r_own, xlast = T.xlast;
  const int rlo = T.rlo, rhi = T.rhi, X0 = T.X0, X1 = T.X1, wxlo = T.wxlo, wxhi = T.wxhi, wfirst = T.wfirst;

  char* sQ = smem;
  char* sK = smem + a.plan.off_a;
  char* sV = smem + a.plan.off_b;

  const TIO* qb = reinterpret_cast<const TIO*>(a.q) + b * a.qs[0] + h * a.qs[1];
  const TIO* kb_ = reinterpret_cast<const TIO*>(a.k) + b * a.ks[0] + h * a.ks[1];
  const TIO* vb_ = reinterpret_cast<const TIO*>(a.v) + b * a.vs[0] + h * a.vs[1];
  TIO* ob = reinterpret_cast<TIO*>(a.o) + b * a.os[0] + h * a.os[1];
  RopeDev no_rope = a.p.rope;
  no_rope.enabled = 0;

  // ---- own queries -> LDS -> B-operand fragments
  stage_tile_qk<TIO, CT, DK>(sQ, PQ, qb, tok_addr(a.qs, a.p.tm), a.qs[3], a.p.dk, a.q_vec != 0, OWN,
                             [&](int row) { return T.own_token(row); }, a.p.rope, tid);
  __syncthreads();
  u32x4 qf[NP][KC], qlo[SPLIT ? NP : 1][KC];
#pragma unroll
  for (int p = 0; p < NP; p++)
#pragma unroll
    for (int c = 0; c < KC; c++) {
      qf[p][c] = lds_read16(sQ + (wave * 16 * NP + 16 * p + n) * PQ + (32 * c + 8 * g) * 2);
      if constexpr (SPLIT) qlo[p][c] = lds_read16(sQ + (wave * 16 * NP + 16 * p + n) * PQ + DK * 2 + (32 * c + 8 * g) * 2);
    }

  float m_run[NP], l_run[NP];
  f32x4 acc[NP][VB];
#pragma unroll
  for (int p = 0; p < NP; p++) {
    m_run[p] = -INFINITY; l_run[p] = 0.f;
#pragma unroll
    for (int d = 0; d < VB; d++) acc[p][d] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  const int CX = a.plan.chunk_x;
  const bool rowfit = a.plan.rowfit != 0;
  const float scale = a.scale_log2;
  bool first_chunk = true;

  for (int kr0 = rlo; kr0 <= rhi; kr0 += a.plan.chunk_rows) {
    const int nr = dlt_imin(a.plan.chunk_rows, rhi - kr0 + 1);
    for (int cx0 = X0; cx0 < X1; cx0 += rowfit ? 0x40000000 : CX) {
      // ---- stage the chunk: nr halo rows x stage_w tokens of K and V
      const int stage_w = rowfit ? dlt_imin(CX, X1 - cx0 + 32) : CX;
      if (!first_chunk) __syncthreads();
      first_chunk = false;
      for (int ri = 0; ri < nr; ri++) {
        const int64_t row_tok0 = (int64_t)(kr0 + ri) * G.XLk + cx0;
        auto tok = [&](int xi) { return cx0 + xi < G.XLk ? row_tok0 + xi : (int64_t)-1; };
        stage_tile_qk<TIO, CT, DK>(sK + ri * CX * PK, PK, kb_, tok_addr(a.ks, a.p.tm), a.ks[3], a.p.dk, a.k_vec != 0, stage_w, tok, a.p.rope, tid);
        stage_tile<TIO, CT, DV>(sV + ri * CX * PV, PV, vb_, tok_addr(a.vs, a.p.tm), a.vs[3], a.p.dv, a.v_vec != 0, stage_w, tok, no_rope, tid);
      }
      __syncthreads();

      // ---- compute
      const int kstart = rowfit ? wxlo : cx0;
      const int kend = rowfit ? wxhi : dlt_imin(wxhi, cx0 + CX);
      for (int ri = 0; ri < nr; ri++) {
        for (int kx0 = kstart; kx0 < kend; kx0 += 32) {
          if (kx0 + 32 <= wxlo) continue;
          const int kb = ri * CX + (kx0 - cx0);
          u32x4 ka[2][KC], kl[SPLIT ? 2 : 1][KC], vt[VB];
#pragma unroll
          for (int mb = 0; mb < 2; mb++)
#pragma unroll
            for (int c = 0; c < KC; c++) {
              ka[mb][c] = lds_read16(sK + (kb + 16 * mb + n) * PK + (32 * c + 8 * g) * 2);
              if constexpr (SPLIT) kl[mb][c] = lds_read16(sK + (kb + 16 * mb + n) * PK + DK * 2 + (32 * c + 8 * g) * 2);
            }
#pragma unroll
          for (int d = 0; d < VB; d++) vt[d] = lds_read_tokens_as_k(sV, PV, kb, 16 * d, n, g);

#pragma unroll
          for (int p = 0; p < NP; p++) {
            if (T.patch_skips(p, kx0)) continue;
            f32x4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < KC; c++) {
              if constexpr (SPLIT) {   // the small terms first
                s0 = Mma<CT>::mfma(kl[0][c], qf[p][c], s0);
                s1 = Mma<CT>::mfma(kl[1][c], qf[p][c], s1);
                s0 = Mma<CT>::mfma(ka[0][c], qlo[p][c], s0);
                s1 = Mma<CT>::mfma(ka[1][c], qlo[p][c], s1);
              }
              s0 = Mma<CT>::mfma(ka[0][c], qf[p][c], s0);
              s1 = Mma<CT>::mfma(ka[1][c], qf[p][c], s1);
            }
            float t[8];
            if (T.patch_needs_mask(p, kx0)) {
#pragma unroll
              for (int i = 0; i < 4; i++) {
                t[i] = T.valid(p, kx0, g, 0, i) ? s0[i] * scale : -INFINITY;
                t[4 + i] = T.valid(p, kx0, g, 1, i) ? s1[i] * scale : -INFINITY;
              }
            } else {
#pragma unroll
              for (int i = 0; i < 4; i++) { t[i] = s0[i] * scale; t[4 + i] = s1[i] * scale; }
            }
            float mloc = fmaxf(fmaxf(fmaxf(t[0], t[1]), fmaxf(t[2], t[3])), fmaxf(fmaxf(t[4], t[5]), fmaxf(t[6], t[7])));
            mloc = wave_max4(mloc);
            const float m_new = fmaxf(m_run[p], mloc);
            const float m_use = m_new == -INFINITY ? 0.f : m_new;
            const float alpha = fast_exp2(m_run[p] - m_use);
            m_run[p] = m_new;
            float psum = 0.f;
#pragma unroll
            for (int i = 0; i < 8; i++) { t[i] = fast_exp2(t[i] - m_use); psum += t[i]; }
            l_run[p] = l_run[p] * alpha + psum;
            if (__builtin_amdgcn_ballot_w64(alpha != 1.f)) {
#pragma unroll
              for (int d = 0; d < VB; d++) acc[p][d] *= alpha;
            }
            const u32x4 pb = pack8<CT>(t);
#pragma unroll
            for (int d = 0; d < VB; d++) acc[p][d] = Mma<CT>::mfma(vt[d], pb, acc[p][d]);
          }
        }
      }
    }
  }

  // ---- epilogue: normalise, O^T fragments -> LDS tile -> coalesced rows; lse2 from lanes g == 0
  __syncthreads();
  char* sO = smem;
#pragma unroll
  for (int p = 0; p < NP; p++) {
    const float lt = wave_sum4(l_run[p]);
    const float inv = lt > 0.f ? fast_rcp(lt) : 0.f;
    const int row = wave * 16 * NP + 16 * p + n;
    TL* orow = reinterpret_cast<TL*>(sO + row * PO);
#pragma unroll
    for (int d = 0; d < VB; d++)
#pragma unroll
      for (int i = 0; i < 4; i++) orow[16 * d + 4 * g + i] = (TL)(acc[p][d][i] * inv);
    const int xq = wfirst + 16 * p + n;
    if (g == 0 && xq <= xlast)
      store_stream4(a.lse + (b * a.ls[0] + h * a.ls[1] + ((int64_t)r_own * G.XLq + xq) * a.ls[2]), m_run[p] + fast_log2(lt));
  }
  __syncthreads();
  store_tile<TIO, TL, DV>(sO, PO, ob, tok_addr(a.os, a.p.tm), a.os[3], a.p.dv, a.o_vec != 0, OWN,
                          [&](int row) { return T.own_token(row); }, no_rope, tid);
}
