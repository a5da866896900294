// Dense and causal flash attention forward for gfx950 with separate qk / vo head dims.
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
#include "swa1_common.hpp"

#ifndef FLASH_NP_DEF
#define FLASH_NP_DEF 2
#endif
#ifndef FLASH_CK_DEF
#define FLASH_CK_DEF 64
#endif
constexpr int FLASH_NP = FLASH_NP_DEF;  // 16-query blocks per wave (forward and dQ)
constexpr int FLASH_CK = FLASH_CK_DEF;  // streamed tokens per LDS chunk
// key blocks per wave in the dK/dV kernel: its two accumulator sets only fit twice for small dims
constexpr int flash_np_kv(int dk, int dv) { return dk + dv > 128 ? 1 : 2; }

struct FlashArgs {
  const void *q, *k, *v;
  void* o;
  float* lse;
  int64_t qs[4], ks[4], vs[4], os[4], ls[3];
  int32_t B, H, Lq, Lk, dk, dv;
  int32_t nblk;       // workgroups per (batch, head)
  int32_t causal;
  int32_t o_vec;
  int32_t lds_bytes;
  float scale_log2;
};

template <typename TIO, int DK, int DV, int NP, int CK, bool CAUSAL>
__global__ __launch_bounds__(256, 2) void flash_fwd_kernel(const FlashArgs a) {
  typedef typename ComputeOf<TIO>::type CT;
  typedef typename TileOf<TIO>::type TL;
  extern __shared__ __align__(16) char smem[];
  constexpr int PK = DK * 2 + 16, PV = DV * 2 + 16, PO = DV * (int)sizeof(TL) + 16;
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
  const int bh = lin / a.nblk;
  // causal: the blocks with the most keys to visit are launched first
  const int xb = CAUSAL ? a.nblk - 1 - (lin - bh * a.nblk) : lin - bh * a.nblk;
  const int x0 = xb * OWN;
  const int wq0 = x0 + wave * 16 * NP;                            // first query of this wave
  const int k_end = CAUSAL ? dlt_imin(a.Lk, x0 + OWN) : a.Lk;     // keys [0, k_end) are visited
  const int b = bh / a.H, h = bh - b * a.H;
  const TIO* qb = reinterpret_cast<const TIO*>(a.q) + b * a.qs[0] + h * a.qs[1];
  const char* kb_ = reinterpret_cast<const char*>(reinterpret_cast<const TIO*>(a.k) + b * a.ks[0] + h * a.ks[1]);
  const char* vb_ = reinterpret_cast<const char*>(reinterpret_cast<const TIO*>(a.v) + b * a.vs[0] + h * a.vs[1]);
  TIO* ob = reinterpret_cast<TIO*>(a.o) + b * a.os[0] + h * a.os[1];
  const int sn2k = (int)a.ks[2] * 2, sn2v = (int)a.vs[2] * 2;
  RopeDev no_rope = RopeDev{};

  // ---- staging plan (chunk invariant): vector `it` of this thread = chunk ck*/vc* of key kkey/vkey + it * step
  const int kc_ = tid % KCH, kkey0 = tid / KCH;
  const int vc_ = tid % VCH, vkey0 = tid / VCH;
  const bool on_k = 8 * kc_ < a.dk, on_v = 8 * vc_ < a.dv;
  u32x4 rk[NKI], rv[NVI];
#pragma unroll
  for (int it = 0; it < NKI; it++) rk[it] = u32x4{0u, 0u, 0u, 0u};
#pragma unroll
  for (int it = 0; it < NVI; it++) rv[it] = u32x4{0u, 0u, 0u, 0u};
  auto issue = [&](int k0) {
#pragma unroll
    for (int it = 0; it < NKI; it++) {
      const int key = dlt_imin(k0 + kkey0 + it * (256 / KCH), a.Lk - 1);
      if (on_k) rk[it] = *reinterpret_cast<const u32x4*>(kb_ + (uint32_t)(key * sn2k + 16 * kc_));
    }
#pragma unroll
    for (int it = 0; it < NVI; it++) {
      const int key = dlt_imin(k0 + vkey0 + it * (256 / VCH), a.Lk - 1);
      if (on_v) rv[it] = *reinterpret_cast<const u32x4*>(vb_ + (uint32_t)(key * sn2v + 16 * vc_));
    }
  };
  auto commit = [&]() {
#pragma unroll
    for (int it = 0; it < NKI; it++) lds_write16(sK + (kkey0 + it * (256 / KCH)) * PK + 16 * kc_, rk[it]);
#pragma unroll
    for (int it = 0; it < NVI; it++) lds_write16(sV + (vkey0 + it * (256 / VCH)) * PV + 16 * vc_, rv[it]);
  };
  issue(0);

  // ---- own queries -> B-operand fragments
  u32x4 qf[NP][KC];
  int64_t tq[NP];
  int klim[NP];  // last key this lane's query may see
#pragma unroll
  for (int p = 0; p < NP; p++) {
    const int xq = x0 + wave * 16 * NP + 16 * p + n;
    tq[p] = xq < a.Lq ? (int64_t)xq : (int64_t)-1;
    klim[p] = CAUSAL ? dlt_imin(xq, a.Lk - 1) : a.Lk - 1;
    swa1_load_own<TIO, CT, DK>(qf[p], qb, a.qs[2], a.dk, tq[p], g, no_rope, false);
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

  commit();
  __syncthreads();

  for (int k0 = 0; k0 < k_end; k0 += CK) {
    const bool has_next = k0 + CK < k_end;
    if (has_next) issue(k0 + CK);
    // some keys of this chunk lie past Lk or (causal) above the wave's first query
    const bool tail = k0 + CK > a.Lk || (CAUSAL && k0 + CK - 1 > wq0);
    // causal: every key of the chunk lies above every query of this wave (wave-uniform)
    const bool live = !CAUSAL || k0 <= wq0 + 16 * NP - 1;

    u32x4 pb[NP][NKB];
    if (live) {
      float t[NP][NKB][8];
#pragma unroll
      for (int kb = 0; kb < NKB; kb++) {
        u32x4 ka[2][KC];
#pragma unroll
        for (int mb = 0; mb < 2; mb++)
#pragma unroll
          for (int c = 0; c < KC; c++) ka[mb][c] = lds_read16(sK + (32 * kb + 16 * mb + n) * PK + (32 * c + 8 * g) * 2);
#pragma unroll
        for (int p = 0; p < NP; p++) {
          f32x4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int c = 0; c < KC; c++) {
            s0 = Mma<CT>::mfma(ka[0][c], qf[p][c], s0);
            s1 = Mma<CT>::mfma(ka[1][c], qf[p][c], s1);
          }
#pragma unroll
          for (int i = 0; i < 4; i++) { t[p][kb][i] = s0[i]; t[p][kb][4 + i] = s1[i]; }
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
        float mloc = -INFINITY;
#pragma unroll
        for (int kb = 0; kb < NKB; kb++)
          mloc = fmaxf(mloc, fmaxf(fmaxf(fmaxf(t[p][kb][0], t[p][kb][1]), fmaxf(t[p][kb][2], t[p][kb][3])),
                                   fmaxf(fmaxf(t[p][kb][4], t[p][kb][5]), fmaxf(t[p][kb][6], t[p][kb][7]))));
        mloc = wave_max4(mloc);
        const float m_new = fmaxf(m_run[p], mloc);
        const float alpha = fast_exp2((m_run[p] - m_new) * scale);
        const float neg_m2 = -m_new * scale;
        m_run[p] = m_new;
#pragma unroll
        for (int kb = 0; kb < NKB; kb++) {
#pragma unroll
          for (int i = 0; i < 8; i++) t[p][kb][i] = fast_exp2(fmaf(t[p][kb][i], scale, neg_m2));
          pb[p][kb] = pack8<CT>(t[p][kb]);
        }
        if (__builtin_amdgcn_ballot_w64(alpha != 1.f)) {
#pragma unroll
          for (int d = 0; d < VB; d++) acc[p][d] *= alpha;
          acc_l[p] *= alpha;
        }
      }
    }
    if (live) {
#pragma unroll
      for (int kb = 0; kb < NKB; kb++) {
#pragma unroll
        for (int d = 0; d < VB; d++) {
          const u32x4 vt = lds_read_tokens_as_k(sV, PV, 32 * kb, 16 * d, n, g);
#pragma unroll
          for (int p = 0; p < NP; p++) acc[p][d] = Mma<CT>::mfma(vt, pb[p][kb], acc[p][d]);
        }
#pragma unroll
        for (int p = 0; p < NP; p++) acc_l[p] = Mma<CT>::mfma(ones, pb[p][kb], acc_l[p]);
      }
    }
    __syncthreads();
    if (has_next) {
      commit();
      __syncthreads();
    }
  }

  // ---- epilogue: normalise, O^T fragments -> LDS tile -> coalesced rows
#pragma unroll
  for (int p = 0; p < NP; p++) {
    const float lt = __shfl(acc_l[p][0], n);
    const float inv = lt > 0.f ? fast_rcp(lt) : 0.f;
    TL* orow = reinterpret_cast<TL*>(smem + (wave * 16 * NP + 16 * p + n) * PO);
#pragma unroll
    for (int d = 0; d < VB; d++)
#pragma unroll
      for (int i = 0; i < 4; i++) orow[16 * d + 4 * g + i] = (TL)(acc[p][d][i] * inv);
    if (g == 0 && tq[p] >= 0) a.lse[b * a.ls[0] + h * a.ls[1] + tq[p] * a.ls[2]] = m_run[p] * scale + fast_log2(lt);
  }
  __syncthreads();
  store_tile<TIO, TL, DV>(smem, PO, ob, a.os[2], a.os[3], a.dv, a.o_vec != 0, OWN,
                          [&](int row) { return x0 + row < a.Lq ? (int64_t)(x0 + row) : (int64_t)-1; }, no_rope, tid);
}

// =============================================================================================
// Dense and causal backward: replaces _attn_bwd_dkdv / _attn_bwd_dq / _attn_bwd
// (src/flash_attn.py:204-449; causal masking :361-379, :416-434), Lq != Lk allowed when not
// causal, with the decoupled structure of the reference
// (dK/dV pass over key blocks, dQ pass over query blocks) as two kernels; no host-side
// pre-scaling pass over k (src/flash_attn.py:509-510), no atomics.
struct FlashBwdArgs {
  const void *q, *k, *v, *d_o;
  const float *lse, *delta;
  void *dq, *dk, *dv;
  int64_t qs[4], ks[4], vs[4], dos[4], dqs[4], dks[4], dvs[4], ls[3];
  int32_t B, H, Lq, Lk, dk_, dv_;
  int32_t nblk_q, nblk_k;
  int32_t causal;
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
    ac = tid % ACH; akey0 = tid / ACH;
    bc = tid % BCH; bkey0 = tid / BCH;
    on_a = 8 * ac < dact_a; on_b = 8 * bc < dact_b;
#pragma unroll
    for (int it = 0; it < NAI; it++) ra[it] = u32x4{0u, 0u, 0u, 0u};
#pragma unroll
    for (int it = 0; it < NBI; it++) rb[it] = u32x4{0u, 0u, 0u, 0u};
  }
  // tokens past `len` are clamped onto the last token (the caller masks them)
  DLT_DEV void issue(const char* a, int sn2a, const char* b, int sn2b, int t0, int len) {
#pragma unroll
    for (int it = 0; it < NAI; it++) {
      const int tok = dlt_imin(t0 + akey0 + it * (256 / ACH), len - 1);
      if (on_a) ra[it] = *reinterpret_cast<const u32x4*>(a + (uint32_t)(tok * sn2a + 16 * ac));
    }
#pragma unroll
    for (int it = 0; it < NBI; it++) {
      const int tok = dlt_imin(t0 + bkey0 + it * (256 / BCH), len - 1);
      if (on_b) rb[it] = *reinterpret_cast<const u32x4*>(b + (uint32_t)(tok * sn2b + 16 * bc));
    }
  }
  DLT_DEV void commit(char* sa, int pa, char* sb, int pb) const {
#pragma unroll
    for (int it = 0; it < NAI; it++) lds_write16(sa + (akey0 + it * (256 / ACH)) * pa + 16 * ac, ra[it]);
#pragma unroll
    for (int it = 0; it < NBI; it++) lds_write16(sb + (bkey0 + it * (256 / BCH)) * pb + 16 * bc, rb[it]);
  }
};

// accumulators (C layout, [dim][own token]) of NP blocks -> LDS tile -> HBM rows
template <typename TIO, int D, int NP>
DLT_DEV void flash_write_grad(char* sT, f32x4 (&acc)[NP][D / 16], float mul, TIO* base, int64_t sn, int64_t sd, int dact,
                              bool vec, int x0, int len, int wave, int n, int g, int tid) {
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
  store_tile<TIO, TL, D>(sT, PT, base, sn, sd, dact, vec, 64 * NP,
                         [&](int r) { return x0 + r < len ? (int64_t)(x0 + r) : (int64_t)-1; }, no_rope, tid);
  __syncthreads();
}

// ---- dQ: own = queries, K and V stream
template <typename TIO, int DK, int DV, int NP, int CK, bool CAUSAL>
__global__ __launch_bounds__(256, 2) void flash_bwd_q_kernel(const FlashBwdArgs a) {
  typedef typename ComputeOf<TIO>::type CT;
  extern __shared__ __align__(16) char smem[];
  constexpr int PK = DK * 2 + 16, PV = DV * 2 + 16;
  constexpr int KC = DK / 32, VC = DV / 32, KB = DK / 16, NKB = CK / 32;
  constexpr int OWN = 64 * NP;

  const int tid = threadIdx.x;
  const int lane = tid & 63, n = lane & 15, g = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  char* sK = smem;
  char* sV = smem + CK * PK;

  const int lin = xcd_remap(blockIdx.x, gridDim.x);
  const int bh = lin / a.nblk_q;
  const int xb = CAUSAL ? a.nblk_q - 1 - (lin - bh * a.nblk_q) : lin - bh * a.nblk_q;
  const int x0 = xb * OWN;
  const int wq0 = x0 + wave * 16 * NP;
  const int k_end = CAUSAL ? dlt_imin(a.Lk, x0 + OWN) : a.Lk;
  const int b = bh / a.H, h = bh - b * a.H;
  const TIO* qb = reinterpret_cast<const TIO*>(a.q) + b * a.qs[0] + h * a.qs[1];
  const TIO* dob = reinterpret_cast<const TIO*>(a.d_o) + b * a.dos[0] + h * a.dos[1];
  const char* kb_ = reinterpret_cast<const char*>(reinterpret_cast<const TIO*>(a.k) + b * a.ks[0] + h * a.ks[1]);
  const char* vb_ = reinterpret_cast<const char*>(reinterpret_cast<const TIO*>(a.v) + b * a.vs[0] + h * a.vs[1]);
  const int sn2k = (int)a.ks[2] * 2, sn2v = (int)a.vs[2] * 2;
  RopeDev no_rope = RopeDev{};

  PairStage<DK, DV, CK> st;
  st.init(tid, a.dk_, a.dv_);
  st.issue(kb_, sn2k, vb_, sn2v, 0, a.Lk);

  u32x4 qf[NP][KC], dof[NP][VC];
  float nlse[NP], del_n[NP];
  int klim[NP];
#pragma unroll
  for (int p = 0; p < NP; p++) {
    const int xq = x0 + wave * 16 * NP + 16 * p + n;
    const int64_t tq = xq < a.Lq ? (int64_t)xq : (int64_t)-1;
    klim[p] = CAUSAL ? dlt_imin(xq, a.Lk - 1) : a.Lk - 1;
    swa1_load_own<TIO, CT, DK>(qf[p], qb, a.qs[2], a.dk_, tq, g, no_rope, false);
    swa1_load_own<TIO, CT, DV>(dof[p], dob, a.dos[2], a.dv_, tq, g, no_rope, false);
    const int64_t off = b * a.ls[0] + h * a.ls[1] + (tq >= 0 ? tq : 0) * a.ls[2];
    nlse[p] = tq >= 0 ? -a.lse[off] : 0.f;
    del_n[p] = tq >= 0 ? a.delta[off] : 0.f;
  }
  f32x4 dq_acc[NP][KB];
#pragma unroll
  for (int p = 0; p < NP; p++)
#pragma unroll
    for (int d = 0; d < KB; d++) dq_acc[p][d] = f32x4{0.f, 0.f, 0.f, 0.f};
  const float scale = a.scale_log2;

  st.commit(sK, PK, sV, PV);
  __syncthreads();

  for (int k0 = 0; k0 < k_end; k0 += CK) {
    const bool has_next = k0 + CK < k_end;
    if (has_next) st.issue(kb_, sn2k, vb_, sn2v, k0 + CK, a.Lk);
    const bool tail = k0 + CK > a.Lk || (CAUSAL && k0 + CK - 1 > wq0);
    const bool live = !CAUSAL || k0 <= wq0 + 16 * NP - 1;
#pragma unroll
    for (int kb = 0; kb < NKB; kb++) {
      if (!live) continue;
      u32x4 ka[2][KC], va[2][VC];
#pragma unroll
      for (int mb = 0; mb < 2; mb++) {
#pragma unroll
        for (int c = 0; c < KC; c++) ka[mb][c] = lds_read16(sK + (32 * kb + 16 * mb + n) * PK + (32 * c + 8 * g) * 2);
#pragma unroll
        for (int c = 0; c < VC; c++) va[mb][c] = lds_read16(sV + (32 * kb + 16 * mb + n) * PV + (32 * c + 8 * g) * 2);
      }
      u32x4 dsb[NP];
#pragma unroll
      for (int p = 0; p < NP; p++) {
        f32x4 s[2], dp[2];
#pragma unroll
        for (int mb = 0; mb < 2; mb++) {
          s[mb] = f32x4{0.f, 0.f, 0.f, 0.f};
          dp[mb] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int c = 0; c < KC; c++) s[mb] = Mma<CT>::mfma(ka[mb][c], qf[p][c], s[mb]);
#pragma unroll
          for (int c = 0; c < VC; c++) dp[mb] = Mma<CT>::mfma(va[mb][c], dof[p][c], dp[mb]);
        }
        float ds[8];
#pragma unroll
        for (int mb = 0; mb < 2; mb++)
#pragma unroll
          for (int i = 0; i < 4; i++) {
            float pv = fast_exp2(fmaf(s[mb][i], scale, nlse[p]));
            if (tail) pv = (k0 + 32 * kb + 16 * mb + 4 * g + i) <= klim[p] ? pv : 0.f;
            ds[4 * mb + i] = pv * (dp[mb][i] - del_n[p]);
          }
        dsb[p] = pack8<CT>(ds);
      }
#pragma unroll
      for (int d = 0; d < KB; d++) {
        const u32x4 kt = lds_read_tokens_as_k(sK, PK, 32 * kb, 16 * d, n, g);
#pragma unroll
        for (int p = 0; p < NP; p++) dq_acc[p][d] = Mma<CT>::mfma(kt, dsb[p], dq_acc[p][d]);
      }
    }
    __syncthreads();
    if (has_next) {
      st.commit(sK, PK, sV, PV);
      __syncthreads();
    }
  }
  TIO* dqb = reinterpret_cast<TIO*>(a.dq) + b * a.dqs[0] + h * a.dqs[1];
  flash_write_grad<TIO, DK, NP>(smem, dq_acc, a.sm_scale, dqb, a.dqs[2], a.dqs[3], a.dk_, a.dq_vec != 0, x0, a.Lq, wave, n, g, tid);
}

// ---- dK / dV: own = keys, Q, dO, lse2 and delta stream
template <typename TIO, int DK, int DV, int NP, int CK, bool CAUSAL>
__global__ __launch_bounds__(256, 2) void flash_bwd_kv_kernel(const FlashBwdArgs a) {
  typedef typename ComputeOf<TIO>::type CT;
  extern __shared__ __align__(16) char smem[];
  constexpr int PQ = DK * 2 + 16, PD = DV * 2 + 16;
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
  const int bh = lin / a.nblk_k;
  const int x0 = (lin - bh * a.nblk_k) * OWN;
  const int b = bh / a.H, h = bh - b * a.H;
  const TIO* kb_ = reinterpret_cast<const TIO*>(a.k) + b * a.ks[0] + h * a.ks[1];
  const TIO* vb_ = reinterpret_cast<const TIO*>(a.v) + b * a.vs[0] + h * a.vs[1];
  const char* qb = reinterpret_cast<const char*>(reinterpret_cast<const TIO*>(a.q) + b * a.qs[0] + h * a.qs[1]);
  const char* dob = reinterpret_cast<const char*>(reinterpret_cast<const TIO*>(a.d_o) + b * a.dos[0] + h * a.dos[1]);
  const float* lseb = a.lse + b * a.ls[0] + h * a.ls[1];
  const float* delb = a.delta + b * a.ls[0] + h * a.ls[1];
  const int sn2q = (int)a.qs[2] * 2, sn2d = (int)a.dos[2] * 2;
  RopeDev no_rope = RopeDev{};

  PairStage<DK, DV, CK> st;
  st.init(tid, a.dk_, a.dv_);
  // causal: queries below the first own key see none of the own keys
  const int q_start = CAUSAL ? (x0 / CK) * CK : 0;
  const int wk0 = x0 + wave * 16 * NP;  // first own key of this wave
  st.issue(qb, sn2q, dob, sn2d, q_start, a.Lq);
  float r_lse = 0.f, r_del = 0.f;
  auto issue_scalars = [&](int q0) {
    if (tid < CK) {
      const int64_t tok = dlt_imin(q0 + tid, a.Lq - 1);
      r_lse = lseb[tok * a.ls[2]];
      r_del = delb[tok * a.ls[2]];
    }
  };
  issue_scalars(q_start);

  u32x4 kf[NP][KC], vf[NP][VC];
  int qmin[NP];  // first query that sees this lane's key
#pragma unroll
  for (int p = 0; p < NP; p++) {
    const int xk = x0 + wave * 16 * NP + 16 * p + n;
    const int64_t tk = xk < a.Lk ? (int64_t)xk : (int64_t)-1;
    qmin[p] = CAUSAL ? xk : 0;
    swa1_load_own<TIO, CT, DK>(kf[p], kb_, a.ks[2], a.dk_, tk, g, no_rope, false);
    swa1_load_own<TIO, CT, DV>(vf[p], vb_, a.vs[2], a.dv_, tk, g, no_rope, false);
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

  st.commit(sQ, PQ, sDO, PD);
  if (tid < CK) { sLse[tid] = r_lse; sDel[tid] = r_del; }
  __syncthreads();

  for (int q0 = q_start; q0 < a.Lq; q0 += CK) {
    const bool has_next = q0 + CK < a.Lq;
    if (has_next) {
      st.issue(qb, sn2q, dob, sn2d, q0 + CK, a.Lq);
      issue_scalars(q0 + CK);
    }
    // some queries of the chunk lie past Lq or (causal) below the wave's last own key
    const bool tail = q0 + CK > a.Lq || (CAUSAL && q0 < wk0 + 16 * NP - 1);
    // causal: every query of the chunk lies below every own key of this wave
    const bool live = !CAUSAL || q0 + CK - 1 >= wk0;
#pragma unroll
    for (int qb_ = 0; qb_ < NQB; qb_++) {
      if (!live) continue;
      u32x4 qa[2][KC], da[2][VC];
      f32x4 lq[2], dl[2];
#pragma unroll
      for (int mb = 0; mb < 2; mb++) {
#pragma unroll
        for (int c = 0; c < KC; c++) qa[mb][c] = lds_read16(sQ + (32 * qb_ + 16 * mb + n) * PQ + (32 * c + 8 * g) * 2);
#pragma unroll
        for (int c = 0; c < VC; c++) da[mb][c] = lds_read16(sDO + (32 * qb_ + 16 * mb + n) * PD + (32 * c + 8 * g) * 2);
        lq[mb] = *reinterpret_cast<const f32x4*>(sLse + 32 * qb_ + 16 * mb + 4 * g);
        dl[mb] = *reinterpret_cast<const f32x4*>(sDel + 32 * qb_ + 16 * mb + 4 * g);
      }
      u32x4 pb[NP], dsb[NP];
#pragma unroll
      for (int p = 0; p < NP; p++) {
        f32x4 s[2], dp[2];
#pragma unroll
        for (int mb = 0; mb < 2; mb++) {
          s[mb] = f32x4{0.f, 0.f, 0.f, 0.f};
          dp[mb] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int c = 0; c < KC; c++) s[mb] = Mma<CT>::mfma(qa[mb][c], kf[p][c], s[mb]);
#pragma unroll
          for (int c = 0; c < VC; c++) dp[mb] = Mma<CT>::mfma(da[mb][c], vf[p][c], dp[mb]);
        }
        float pr[8], ds[8];
#pragma unroll
        for (int mb = 0; mb < 2; mb++)
#pragma unroll
          for (int i = 0; i < 4; i++) {
            float pv = fast_exp2(fmaf(s[mb][i], scale, -lq[mb][i]));
            if (tail) {
              const int qi = q0 + 32 * qb_ + 16 * mb + 4 * g + i;
              pv = (qi >= qmin[p] && qi < a.Lq) ? pv : 0.f;
            }
            pr[4 * mb + i] = pv;
            ds[4 * mb + i] = pv * (dp[mb][i] - dl[mb][i]);
          }
        pb[p] = pack8<CT>(pr);
        dsb[p] = pack8<CT>(ds);
      }
#pragma unroll
      for (int d = 0; d < VB; d++) {
        const u32x4 dt = lds_read_tokens_as_k(sDO, PD, 32 * qb_, 16 * d, n, g);
#pragma unroll
        for (int p = 0; p < NP; p++) dv_acc[p][d] = Mma<CT>::mfma(dt, pb[p], dv_acc[p][d]);
      }
#pragma unroll
      for (int d = 0; d < KB; d++) {
        const u32x4 qt = lds_read_tokens_as_k(sQ, PQ, 32 * qb_, 16 * d, n, g);
#pragma unroll
        for (int p = 0; p < NP; p++) dk_acc[p][d] = Mma<CT>::mfma(qt, dsb[p], dk_acc[p][d]);
      }
    }
    __syncthreads();
    if (has_next) {
      st.commit(sQ, PQ, sDO, PD);
      if (tid < CK) { sLse[tid] = r_lse; sDel[tid] = r_del; }
      __syncthreads();
    }
  }
  TIO* dkb = reinterpret_cast<TIO*>(a.dk) + b * a.dks[0] + h * a.dks[1];
  TIO* dvb = reinterpret_cast<TIO*>(a.dv) + b * a.dvs[0] + h * a.dvs[1];
  flash_write_grad<TIO, DK, NP>(smem, dk_acc, a.sm_scale, dkb, a.dks[2], a.dks[3], a.dk_, a.dk_vec != 0, x0, a.Lk, wave, n, g, tid);
  flash_write_grad<TIO, DV, NP>(smem, dv_acc, 1.0f, dvb, a.dvs[2], a.dvs[3], a.dv_, a.dv_vec != 0, x0, a.Lk, wave, n, g, tid);
}
