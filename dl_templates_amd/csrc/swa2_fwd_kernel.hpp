// Forward kernel for token grids at head dim 128 (b_size == 1, no rotation): replaces tiled_swa_fwd_kernel
// (src/tiled_swa.py:15-133) for the shapes of benchmark config 4.  Structure in swa2_common.hpp; per chunk a wave
//   1. computes S^T = K Q^T for its three blocks of 4 x 8 keys, masked to -inf outside the window,
//   2. runs one online-softmax update on the raw scores (p = exp2((s - m) scale)),
//   3. accumulates O^T += V^T P^T; the row sums come from one extra MFMA against a row of ones.
#pragma once
#include "swa2_common.hpp"
#include <type_traits>

struct Swa2FwdArgs {
  AttnProblem p;
  Swa2Plan plan;
  const void *q, *k, *v;
  void* o;
  float* lse;
  int64_t qs[4], ks[4], vs[4], os[4], ls[3];
  float scale_log2;
};

// per-lane window of an own token in the coordinates of the band's halo
struct Swa2Win {
  int rlo, rhi;      // visible halo rows [rlo, rhi]
  int clo, cspan;    // visible window columns [clo, clo + cspan] (cspan < 0: the token lies outside the grid)
  int ch_lo, ch_hi;  // chunks that hold visible rows of the wave's patch (wave-uniform)
};

DLT_DEV Swa2Win swa2_window(const Swa2Geom& G, int rg, int pc, int n) {
  Swa2Win w;
  const int qr = 4 * rg + (n >> 2), qc = n & 3;
  const int c_p = G.c0 + 4 * pc;
  const bool ok = (G.r0 + qr < G.TR) && (c_p + qc < G.TC);
  w.rlo = dlt_imax(qr, G.WR - G.r0);
  w.rhi = dlt_imin(qr + 2 * G.WR, G.TR - 1 - G.r0 + G.WR);
  w.clo = dlt_imax(qc, G.WC - c_p);
  const int chi = dlt_imin(qc + 2 * G.WC, G.TC - 1 - c_p + G.WC);
  w.cspan = ok ? chi - w.clo : -1;
  // halo rows of the patch that hold grid rows
  const int plo = dlt_imax(4 * rg, G.WR - G.r0), phi = dlt_imin(4 * rg + 3 + 2 * G.WR, G.TR - 1 - G.r0 + G.WR);
  const bool patch_ok = (G.r0 + 4 * rg < G.TR) && (c_p < G.TC) && plo <= phi;
  w.ch_lo = patch_ok ? plo >> 2 : 1;
  w.ch_hi = patch_ok ? phi >> 2 : 0;
  return w;
}

template <typename TIO>
__global__ __launch_bounds__(SWA2_THREADS) void swa2_fwd_kernel(const Swa2FwdArgs a) {
  typedef typename ComputeOf<TIO>::type CT;
  extern __shared__ __align__(16) char smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63, n = lane & 15, g = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int pc = wave & 3, rg = wave >> 2;
  const Swa2Geom G = swa2_geom(a.p, a.plan);

  const char* qb = reinterpret_cast<const char*>(a.q) + 2 * (G.b * a.qs[0] + G.h * a.qs[1]);
  const char* kb_ = reinterpret_cast<const char*>(a.k) + 2 * (G.b * a.ks[0] + G.h * a.ks[1]);
  const char* vb_ = reinterpret_cast<const char*>(a.v) + 2 * (G.b * a.vs[0] + G.h * a.vs[1]);
  TIO* ob = reinterpret_cast<TIO*>(a.o) + G.b * a.os[0] + G.h * a.os[1];
  float* lseb = a.lse + G.b * a.ls[0] + G.h * a.ls[1];
  const int64_t os2 = a.os[2], ls2 = a.ls[2];
  const float scale = a.scale_log2;

  // staging: waves 0-3 copy the four halo rows of K, waves 4-7 those of V
  const bool stage_k = wave < 4;
  const char* sbase = stage_k ? kb_ : vb_;
  const int ssn2 = (int)(stage_k ? a.ks[2] : a.vs[2]) * 2;
  const uint32_t srow = (uint32_t)(G.TC * ssn2);
  Swa2Stage st;
  swa2_stage_init(st, G, wave, lane, ssn2);
  swa2_issue(st, G, G.ch_first, sbase, srow, smem + (G.ch_first & 1) * SWA2_BUF, wave);

  // own queries straight into B-operand fragments: lane (n, g) holds head dims 32 c + 8 g .. + 7 of query n
  const int r_p = G.r0 + 4 * rg, c_p = G.c0 + 4 * pc;
  const int tq = (r_p + (n >> 2) < G.TR && c_p + (n & 3) < G.TC) ? (r_p + (n >> 2)) * G.TC + c_p + (n & 3) : -1;
  u32x4 qf[4];
  {
    const char* p = qb + ((uint32_t)((tq >= 0 ? tq : 0) * ((int)a.qs[2] * 2)) + 16 * g);
#pragma unroll
    for (int c = 0; c < 4; c++) qf[c] = *reinterpret_cast<const u32x4*>(p + 64 * c);
  }
  const Swa2Win W = swa2_window(G, rg, pc, n);
  Swa2Lane L;
  swa2_lane_init(L, pc, n, g);

  float m_run = -INFINITY;
  f32x4 acc[8], acc_l = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int d = 0; d < 8; d++) acc[d] = f32x4{0.f, 0.f, 0.f, 0.f};
  const unsigned one2 = pack2<CT>(1.f, 1.f);
  const u32x4 ones = n == 0 ? u32x4{one2, one2, one2, one2} : u32x4{0u, 0u, 0u, 0u};
  const int ncg = (4 + 2 * G.WC + 3) >> 2;   // column groups of the wave window that can hold a visible token

  swa2_wait_copies();   // also: the own fragments have arrived
  __syncthreads();

  // `cur` (the chunk being read) and `nxt` (the buffer the next chunk is copied into) are distinct buffers: the restrict
  // qualifiers let the compiler see that the operand reads do not depend on the copies in flight, so that it does not
  // wait for those in front of every LDS read
  auto consume = [&](const int ch, Swa2Lds __restrict__ cur, char* __restrict__ nxt, auto more_tag) {
    constexpr bool more = decltype(more_tag)::value;   // a later chunk exists: its copies are issued between the products
    Swa2Lds sK = cur;
    Swa2Lds sV = sK + SWA2_REGION;
    const char* nrow = swa2_issue_row(G, ch + 1, sbase, srow, wave);
    char* ndst = swa2_issue_dst(nxt, wave);
    const int hrow = 4 * ch + g;
    const bool row_vis = (hrow >= W.rlo) & (hrow <= W.rhi);
    // ---- scores of the chunk, one column group (16 keys) at a time.  Per group: the operands of the next group are
    //      requested, one copy instruction of the next chunk is issued, and the four products of this group are issued
    //      with the masking and the running maxima of the previous group between them.
    float t[3][8];
    float mx[4] = {-INFINITY, -INFINITY, -INFINITY, -INFINITY};
    u32x4 ka[2][4];
    f32x4 sc[2];
    auto mask_max = [&](const int cg, const f32x4& sv) {
      const int kb = cg >> 1, h4 = 4 * (cg & 1);
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const bool vis = row_vis & (cg < ncg) & ((unsigned)(4 * cg + i - W.clo) <= (unsigned)W.cspan);
        t[kb][h4 + i] = vis ? sv[i] : -INFINITY;
      }
      mx[cg & 3] = fmaxf(fmaxf(mx[cg & 3], t[kb][h4]), t[kb][h4 + 1]);
      mx[(cg + 2) & 3] = fmaxf(fmaxf(mx[(cg + 2) & 3], t[kb][h4 + 2]), t[kb][h4 + 3]);
    };
    swa2_read_a<0>(sK, L, ka[0]);
#pragma unroll
    for (int cg = 0; cg < 6; cg++) {
      if (more) {
        if (cg == 0) swa2_issue_one<0>(st, nrow, ndst);
        if (cg == 1) swa2_issue_one<1>(st, nrow, ndst);
        if (cg == 2) swa2_issue_one<2>(st, nrow, ndst);
        if (cg == 3) swa2_issue_one<3>(st, nrow, ndst);
        if (cg == 4) swa2_issue_one<4>(st, nrow, ndst);
        if (cg == 5) swa2_issue_one<5>(st, nrow, ndst);
      }
      __builtin_amdgcn_sched_barrier(0);
      if (cg == 0) swa2_read_a<1>(sK, L, ka[1]);
      if (cg == 1) swa2_read_a<2>(sK, L, ka[0]);
      if (cg == 2) swa2_read_a<3>(sK, L, ka[1]);
      if (cg == 3) swa2_read_a<4>(sK, L, ka[0]);
      if (cg == 4) swa2_read_a<5>(sK, L, ka[1]);
      __builtin_amdgcn_sched_barrier(0);
      const u32x4(&kc)[4] = ka[cg & 1];
      f32x4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int c = 0; c < 4; c++) s = Mma<CT>::mfma(kc[c], qf[c], s);
      sc[cg & 1] = s;
      if (cg > 0) mask_max(cg - 1, sc[(cg - 1) & 1]);
      SWA2_MIX(4, 2)
      __builtin_amdgcn_sched_barrier(0);
    }
    mask_max(5, sc[1]);
    // The reference maximum m_run only moves when some score exceeds it by more than 2^8 after scaling: p then stays
    // below 2^8, well inside the range of the 16-bit operand and of the fp32 sums, and the rescaling of the 8 + 1
    // accumulators is skipped for most chunks.  o and lse do not depend on which reference was used.
    const float mloc = wave_max4(fmaxf(fmaxf(mx[0], mx[1]), fmaxf(mx[2], mx[3])));
    if (__builtin_amdgcn_ballot_w64((mloc - m_run) * scale > 8.f)) {
      keep_branch();
      const float m_new = fmaxf(m_run, mloc);
      const float alpha = fast_exp2((m_run - m_new) * scale);   // m_new is finite here
      m_run = m_new;
#pragma unroll
      for (int d = 0; d < 8; d++) acc[d] *= alpha;
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
    swa2_read_tr<0, 0, 4>(sV, L, va[0]);
    probs(0, 0, pb[0]);
    probs(0, 1, pb[0]);
#pragma unroll
    for (int kb = 0; kb < 3; kb++) {
      if (more) {
        if (kb == 0) swa2_issue_one<6>(st, nrow, ndst);
        if (kb == 1) swa2_issue_one<7>(st, nrow, ndst);
        if (kb == 2) swa2_issue_one<8>(st, nrow, ndst);
      }
      __builtin_amdgcn_sched_barrier(0);
      if (kb == 0) swa2_read_tr<0, 4, 4>(sV, L, va[1]);
      if (kb == 1) swa2_read_tr<1, 4, 4>(sV, L, va[1]);
      if (kb == 2) swa2_read_tr<2, 4, 4>(sV, L, va[1]);
      __builtin_amdgcn_sched_barrier(0);
      const u32x4 pk = pb[kb & 1];
#pragma unroll
      for (int d = 0; d < 4; d++) acc[d] = Mma<CT>::mfma(va[0][d], pk, acc[d]);
      if (kb < 2) probs(kb + 1, 0, pb[(kb + 1) & 1]);
      SWA2_MIX(4, 3)
      __builtin_amdgcn_sched_barrier(0);
      if (kb == 0) swa2_read_tr<1, 0, 4>(sV, L, va[0]);
      if (kb == 1) swa2_read_tr<2, 0, 4>(sV, L, va[0]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int d = 0; d < 4; d++) acc[4 + d] = Mma<CT>::mfma(va[1][d], pk, acc[4 + d]);
      acc_l = Mma<CT>::mfma(ones, pk, acc_l);
      if (kb < 2) probs(kb + 1, 1, pb[(kb + 1) & 1]);
      SWA2_MIX(5, 2)
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // chunk ch + 1 travels HBM -> LDS (other buffer) while chunk ch is consumed; one barrier per chunk
  // Every wave runs ch_last - ch_first rounds of (work, wait for its copies, workgroup barrier).  The chunks that hold
  // visible rows of its patch are contiguous; the rounds before and after them only copy.  Three loops instead of one
  // with a branch keep the accumulators in place (a branch inside the loop had them copied on every round).
  const int act_lo = dlt_imax(G.ch_first, W.ch_lo), act_hi = dlt_imin(G.ch_last - 1, W.ch_hi);
  auto copy_only = [&](int ch) {
    swa2_issue(st, G, ch + 1, sbase, srow, smem + ((ch + 1) & 1) * SWA2_BUF, wave);
    swa2_wait_copies();
    __syncthreads();
  };
  int ch = G.ch_first;
  for (; ch < G.ch_last && ch < act_lo; ch++) copy_only(ch);
  for (; ch <= act_hi; ch++) {
    consume(ch, (Swa2Lds)smem + (ch & 1) * SWA2_BUF, smem + ((ch + 1) & 1) * SWA2_BUF, std::true_type{});
    swa2_wait_copies();
    __syncthreads();
  }
  for (; ch < G.ch_last; ch++) copy_only(ch);
  if (G.ch_last >= W.ch_lo && G.ch_last <= W.ch_hi) consume(G.ch_last, (Swa2Lds)smem + (G.ch_last & 1) * SWA2_BUF, smem + ((G.ch_last + 1) & 1) * SWA2_BUF, std::false_type{});
  __syncthreads();

  // ---- epilogue (the loop ended with a barrier: the chunk buffers are free)
  const float lt = wave_sum4(acc_l[0]);   // only row 0 of the ones operand is set: the other lane groups hold zeros
  const float inv = lt > 0.f ? fast_rcp(lt) : 0.f;
  if (g == 0 && tq >= 0) lseb[(int64_t)tq * ls2] = m_run * scale + fast_log2(lt);
  swa2_store_own<TIO, CT>(smem + wave * 4096, acc, inv, ob, os2, G, r_p, c_p, lane);
}
