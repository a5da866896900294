// Dense (non-causal) flash attention forward for gfx950 with separate qk / vo head dims.
//
// Replaces _attn_fwd_inner / _attn_fwd (src/flash_attn.py:9-172) for the non-causal case and
// extends it to Lq != Lk.  A workgroup of 4 waves owns 64*NP consecutive queries of one
// (batch, head); a wave owns NP blocks of 16 queries whose fragments come straight from HBM.
// K and V stream through LDS in chunks of CK keys; the next chunk travels HBM -> registers
// while the current one is consumed.  Per chunk and query block: S^T = K Q^T for all 32-key
// blocks, ONE online-softmax update on the raw scores (p = exp2(fma(s, c, -m c))), then
// O^T += V^T P^T with the K / V^T operand fragments shared by the NP query blocks and the row
// sums produced by one extra MFMA against a row of ones.  Keys past Lk are clamped loads
// masked by an additive -inf bias that only the last chunk applies.
#pragma once
#include "swa1_common.hpp"

constexpr int FLASH_NP = 2;   // 16-query blocks per wave
constexpr int FLASH_CK = 64;  // keys per LDS chunk

struct FlashArgs {
  const void *q, *k, *v;
  void* o;
  float* lse;
  int64_t qs[4], ks[4], vs[4], os[4], ls[3];
  int32_t B, H, Lq, Lk, dk, dv;
  int32_t nblk;       // workgroups per (batch, head)
  int32_t o_vec;
  int32_t lds_bytes;
  float scale_log2;
};

template <typename TIO, int DK, int DV, int NP, int CK>
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
  const int x0 = (lin - bh * a.nblk) * OWN;
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
#pragma unroll
  for (int p = 0; p < NP; p++) {
    const int xq = x0 + wave * 16 * NP + 16 * p + n;
    tq[p] = xq < a.Lq ? (int64_t)xq : (int64_t)-1;
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

  for (int k0 = 0; k0 < a.Lk; k0 += CK) {
    const bool has_next = k0 + CK < a.Lk;
    if (has_next) issue(k0 + CK);
    const bool tail = k0 + CK > a.Lk;  // some keys of this chunk lie past Lk

    u32x4 pb[NP][NKB];
    {
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
              t[p][kb][i] = key < a.Lk ? t[p][kb][i] : -INFINITY;
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
