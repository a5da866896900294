// Flash kernels with asynchronous staging: the variants of flash_kernel.hpp for head dims that are exactly 64 or
// 128 (no padded dims: a copy cannot zero-fill).  Streamed chunks travel HBM -> LDS by the DMA path of the vector
// memory unit (16 bytes per lane, no staging registers, no LDS write instructions) into one of two chunk buffers
// while the other one is consumed: one workgroup barrier per chunk instead of two.  LDS rows are 2 D bytes without
// padding; the 16-byte piece c of token t is stored at piece c ^ (m (t & 7)), m = D / 64, which keeps the operand
// reads (16 lanes x 16 bytes), the transposing reads (32 lanes x 8 bytes) and the 64 x 16 bytes a copy instruction
// writes on distinct banks.  The arithmetic, the masks and the chunk walk are those of flash_kernel.hpp.
#pragma once
#include "flash_kernel.hpp"
#include "swa2_common.hpp"

template <int D>
struct FlashDRow {
  static constexpr int ROW = 2 * D;          // bytes of a token row
  static constexpr int PIECES = D / 8;       // 16-byte pieces of a row
  static constexpr int SWZ = PIECES / 8;     // swizzle multiplier
  static constexpr int TPI = 64 / PIECES;    // tokens per copy instruction
  static_assert(D == 64 || D == 128, "asynchronous staging: head dim 64 or 128");
};

// Lane constants for the operand reads of a swizzled [token][D] tile.
//   a[c]:  A operand (token = MFMA row): token n of a 16-token group (groups start at multiples of 16, so t & 7 = n & 7),
//          head dims 32 c + 8 g .. + 7 = piece 4 c + g
//   tr[d]: transposing read (tokens along k): token 4 g + (n >> 2) of a 32-token block (the second half of the block lies
//          16 rows further: same t & 7), 8 bytes at head dim 16 d + 4 (n & 3)
template <int D>
struct FlashDLane {
  int a[D / 32];
  int tr[D / 16];
};

template <int D>
DLT_DEV void flashd_lane_init(FlashDLane<D>& L, int n, int g) {
  typedef FlashDRow<D> R;
#pragma unroll
  for (int c = 0; c < D / 32; c++) L.a[c] = n * R::ROW + 16 * ((4 * c + g) ^ (R::SWZ * (n & 7)));
  const int t2 = 4 * g + (n >> 2);
#pragma unroll
  for (int d = 0; d < D / 16; d++) L.tr[d] = t2 * R::ROW + 16 * ((2 * d + ((n & 3) >> 1)) ^ (R::SWZ * (t2 & 7))) + 8 * (n & 1);
}

// A-operand pieces of the 16 tokens that start at row T0 (a multiple of 16) of a tile
template <int D, int T0>
DLT_DEV void flashd_read_a(Swa2Lds tile, const FlashDLane<D>& L, u32x4 (&x)[D / 32]) {
#pragma unroll
  for (int c = 0; c < D / 32; c++) x[c] = swa2_lds16(tile + T0 * FlashDRow<D>::ROW + L.a[c]);
}

// A operand with tokens along k for the 32 tokens that start at row T0 (a multiple of 32): head dims 16 d .. + 15 are its rows
template <int D, int T0>
DLT_DEV u32x4 flashd_read_tr(Swa2Lds tile, const FlashDLane<D>& L, int d) {
  const u32x2 lo = swa2_lds_tr(tile + T0 * FlashDRow<D>::ROW + L.tr[d]);
  const u32x2 hi = swa2_lds_tr(tile + (T0 + 16) * FlashDRow<D>::ROW + L.tr[d]);
  u32x4 r;
  r.x = lo.x; r.y = lo.y; r.z = hi.x; r.w = hi.y;
  return r;
}

// Copy of one chunk of CK tokens of a [token][D] tensor by the 4 waves of a workgroup: wave w copies tokens
// w CK / 4 .. + CK / 4 - 1 in NI instructions; instruction i, lane l writes LDS slot l of its 1 KB = physical piece
// l % PIECES of token w CK / 4 + TPI i + l / PIECES, and therefore fetches the logical piece (l % PIECES) ^ (SWZ (token & 7)).
template <int D, int CK>
struct FlashDStage {
  typedef FlashDRow<D> R;
  static constexpr int NI = CK / 4 / R::TPI;
  int tok0;   // token of the lane in instruction 0
  int lp;     // physical piece the lane writes

  DLT_DEV void init(int wave, int lane) {
    tok0 = wave * (CK / 4) + lane / R::PIECES;
    lp = lane % R::PIECES;
  }
  // tokens past the end of the chunk are clamped onto its last token (the caller masks them)
  template <typename AD>
  DLT_DEV void issue(const char* base, const AD& ad, const FlashChunk& c, char* region, int wave) const {
#pragma unroll
    for (int i = 0; i < NI; i++) {
      const int t = tok0 + R::TPI * i;
      const uint32_t off = ad(c, dlt_imin(t, c.nvalid - 1)) + 16u * (uint32_t)(lp ^ (R::SWZ * (t & 7)));
      char* dst = region + (wave * (CK / 4) + R::TPI * i) * R::ROW;   // wave-uniform
      dlt_copy16_to_lds(base, off, dst);
    }
  }
};

// per-token fp32 scalars of a chunk: 64 tokens per instruction, 4 bytes per lane (32-bit byte offsets inside a
// (batch, head) slab: checked by the host)
template <int CK>
DLT_DEV void flashd_issue_scalars(const float* base, int stride, const FlashChunk& c, char* dst, int lane) {
#pragma unroll
  for (int j = 0; j < CK / 64; j++) {
    const uint32_t off = (uint32_t)((c.tok0 + dlt_imin(64 * j + lane, c.nvalid - 1)) * stride) * 4u;
    dlt_copy4_to_lds(reinterpret_cast<const char*>(base), off, dst + 256 * j);
  }
}

// at most N of this wave's copies (the youngest ones) are still in flight
template <int N>
DLT_DEV void flashd_wait_copies() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }

// chunk buffers per workgroup: a copy is started NBUF - 1 chunks ahead of its use; three where two workgroups
// still fit a CU
#ifndef FLASHD_NBUF
#define FLASHD_NBUF(dk, dv) ((dk) + (dv) > 192 ? 2 : 3)
#endif
constexpr int flashd_nbuf(int dk, int dv) { return FLASHD_NBUF(dk, dv); }

template <int DK, int DV, int CK>
struct FlashDBuf {
  static constexpr int REG_A = CK * 2 * DK;            // first tensor of a chunk
  static constexpr int REG_B = CK * 2 * DV;            // second tensor
  static constexpr int SCAL = 2 * CK * 4;              // lse2 then delta (dK/dV kernel)
  static constexpr int BUF = REG_A + REG_B;            // forward, dQ
  static constexpr int BUF_KV = REG_A + REG_B + SCAL;  // dK/dV
};

// ---- dK / dV: own = keys; Q, dO, lse2 and delta stream.  Replaces _attn_bwd_dkdv (src/flash_attn.py:204-307).
template <typename TIO, int DK, int DV, int NP, int CK, int MODE>
__global__ __launch_bounds__(256, NP >= 4 ? 1 : 2) void flashd_bwd_kv_kernel(const FlashBwdArgs a) {
  typedef typename ComputeOf<TIO>::type CT;
  typedef FlashDBuf<DK, DV, CK> B;
  extern __shared__ __align__(16) char smem[];
  constexpr bool CAUSAL = MODE == 1, TILE = MODE >= 2, IMG = MODE == 3;
  constexpr int KC = DK / 32, VC = DV / 32, KB = DK / 16, VB = DV / 16, NQB = CK / 32;
  constexpr int OWN = 64 * NP;

  const int tid = threadIdx.x;
  const int lane = tid & 63, n = lane & 15, g = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  const int lin = xcd_remap(blockIdx.x, gridDim.x);
  int bh, r_own, x0;
  flash_block(lin, a.nblk_k, TILE ? a.g.TR : 1, OWN, false, bh, r_own, x0);
  const int b = bh / a.H, h = bh - b * a.H;
  const TIO* kb_ = reinterpret_cast<const TIO*>(a.k) + b * a.ks[0] + h * a.ks[1];
  const TIO* vb_ = reinterpret_cast<const TIO*>(a.v) + b * a.vs[0] + h * a.vs[1];
  const char* qb = reinterpret_cast<const char*>(reinterpret_cast<const TIO*>(a.q) + b * a.qs[0] + h * a.qs[1]);
  const char* dob = reinterpret_cast<const char*>(reinterpret_cast<const TIO*>(a.d_o) + b * a.dos[0] + h * a.dos[1]);
  const float* lseb = a.lse + b * a.ls[0] + h * a.ls[1];
  const float* delb = a.delta + b * a.ls[0] + h * a.ls[1];
  const FlashAddr<IMG> aq = flash_addr<IMG>(a.qs, a.tm), ad = flash_addr<IMG>(a.dos, a.tm);
  RopeDev no_rope = RopeDev{};
  const int own_base = TILE ? r_own * a.Lk : 0;

  FlashWalk<MODE, CK> W;
  if (TILE) W.init_tile(a.g, r_own, x0, OWN, true);
  else W.init_seq(CAUSAL ? (x0 / CK) * CK : 0, a.Lq);
  const int wk0 = x0 + wave * 16 * NP;  // first own key of this wave

  FlashDStage<DK, CK> stq;
  FlashDStage<DV, CK> std_;
  stq.init(wave, lane);
  std_.init(wave, lane);
  // waves 0 and 1 also copy the chunk's lse2 / delta
  const float* scal_base = wave == 0 ? lseb : delb;
  auto issue = [&](const FlashChunk& c, char* buf) {
    stq.issue(qb, aq, c, buf, wave);
    std_.issue(dob, ad, c, buf + B::REG_A, wave);
    if (wave < 2) flashd_issue_scalars<CK>(scal_base, (int)a.ls[2], c, buf + B::REG_A + B::REG_B + wave * (CK * 4), lane);
  };
  constexpr int NBUF = flashd_nbuf(DK, DV), AHEAD = NBUF - 1;
  constexpr int PER_CHUNK = FlashDStage<DK, CK>::NI + FlashDStage<DV, CK>::NI;   // copies per wave and chunk (waves 0, 1: more)
#pragma unroll
  for (int i = 0; i < AHEAD; i++)
    if (i < W.nchunks) issue(W.at(i), smem + i * B::BUF_KV);

  u32x4 kf[NP][KC], vf[NP][VC];
  int qmin[NP];           // causal: first query that sees this lane's key
  int vlo[NP], vhi[NP];   // tile mode: x interval of the queries that see this key block
#pragma unroll
  for (int p = 0; p < NP; p++) {
    const int xk = wk0 + 16 * p + n;
    const int64_t tk = xk < a.Lk ? (int64_t)(own_base + xk) : (int64_t)-1;
    qmin[p] = CAUSAL ? xk : 0;
    vlo[p] = vhi[p] = 0;
    if (TILE && wk0 + 16 * p < a.Lk) {
      int rl, rh;
      dlt_query_range(a.g, r_own, wk0 + 16 * p, rl, rh, vlo[p], vhi[p]);
    }
    swa1_load_own<TIO, CT, DK>(kf[p], kb_, 1, a.dk_, flash_own_off<IMG>(a.ks, a.tm, tk), g, no_rope, false);
    swa1_load_own<TIO, CT, DV>(vf[p], vb_, 1, a.dv_, flash_own_off<IMG>(a.vs, a.tm, tk), g, no_rope, false);
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
  FlashDLane<DK> LQ;
  FlashDLane<DV> LD;
  flashd_lane_init(LQ, n, g);
  flashd_lane_init(LD, n, g);

  swa2_wait_copies();   // also: the own fragments have arrived
  __syncthreads();

  auto chunk_tail = [&](const int ci) {
    const FlashChunk c = W.at(ci);
    return !TILE && (c.nvalid < CK || (CAUSAL && c.x < wk0 + 16 * NP - 1));
  };
  // Products of the chunk resident in `cur`; with `more` the copy of the next chunk into `nxt` is started first.
  // A block of 32 queries is a stream of NB operand reads, each feeding NP matrix instructions: per 16-query half KC
  // pieces of Q (S = Q K^T) and VC pieces of dO (dP = dO V^T), then VB transposed pieces of dO (dV^T += dO^T P) and KB
  // of Q (dK^T += Q^T dS).  The reads run RD operands ahead of their products through a ring of RD + 1 registers sets
  // and across block borders (left to itself the compiler issues every read right in front of its products: the
  // matrix pipe then idles for an LDS latency per pair of products).
  auto consume_t = [&](const int ci, Swa2Lds __restrict__ cur, char* __restrict__ nxt, auto tail_tag, auto more_tag) __attribute__((always_inline)) {
    bool tail;
    if constexpr (std::is_same<decltype(tail_tag), FlashTailDyn>::value) tail = chunk_tail(ci);
    else tail = decltype(tail_tag)::value;
    if constexpr (decltype(more_tag)::value) issue(W.at(ci + AHEAD), nxt);
    Swa2Lds sQ = cur, sDO = cur + B::REG_A;
    Swa2Lds sLse = cur + B::REG_A + B::REG_B + 16 * g, sDel = sLse + CK * 4;
    const FlashChunk c = W.at(ci);
    const int q0 = c.x;
    // causal: every query of the chunk lies below every own key of this wave
    if (CAUSAL && q0 + CK - 1 < wk0) return;
    constexpr int N1H = KC + VC, N1 = 2 * N1H, NB = N1 + VB + KB, NT = NQB * NB;
#ifndef FLASHD_RD
#define FLASHD_RD 3
#endif
    constexpr int RD = FLASHD_RD;
    u32x4 ring[RD + 1];
    auto rd = [&](auto kc) __attribute__((always_inline)) {
      constexpr int k = decltype(kc)::value;
      constexpr int qb_ = k / NB, j = k % NB;
      if constexpr (j < N1) {
        constexpr int mb = j / N1H, r = j % N1H, T0 = 32 * qb_ + 16 * mb;
        if constexpr (r < KC) ring[k % (RD + 1)] = swa2_lds16(sQ + T0 * FlashDRow<DK>::ROW + LQ.a[r]);
        else ring[k % (RD + 1)] = swa2_lds16(sDO + T0 * FlashDRow<DV>::ROW + LD.a[r - KC]);
      } else {
        constexpr int d = j - N1;
        if constexpr (d < VB) ring[k % (RD + 1)] = flashd_read_tr<DV, 32 * qb_>(sDO, LD, d);
        else ring[k % (RD + 1)] = flashd_read_tr<DK, 32 * qb_>(sQ, LQ, d - VB);
      }
    };
    swa2_for<0, RD>([&](auto kc) __attribute__((always_inline)) { rd(kc); });
    swa2_for<0, NQB>([&](auto qbc) __attribute__((always_inline)) {
      constexpr int qb_ = decltype(qbc)::value;
      bool bv[NP];
#pragma unroll
      for (int p = 0; p < NP; p++) bv[p] = !TILE || (q0 + 32 * qb_ + 32 > vlo[p] && q0 + 32 * qb_ < vhi[p]);
      float pr[NP][8], ds[NP][8];
      f32x4 sv[NP], dp[NP], lq, dl;
      u32x4 pb[NP], dsb[NP];
      swa2_for<0, NB>([&](auto jc) __attribute__((always_inline)) {
        constexpr int j = decltype(jc)::value, k = qb_ * NB + j;
        if constexpr (k + RD < NT) rd(std::integral_constant<int, k + RD>{});
        if constexpr (j < N1 && j % N1H == 0) {
          constexpr int mb = j / N1H;
          lq = __builtin_bit_cast(f32x4, swa2_lds16(sLse + (32 * qb_ + 16 * mb) * 4));
          dl = __builtin_bit_cast(f32x4, swa2_lds16(sDel + (32 * qb_ + 16 * mb) * 4));
        }
        __builtin_amdgcn_sched_barrier(0);
        const u32x4 x = ring[k % (RD + 1)];
        if constexpr (j < N1) {
          constexpr int mb = j / N1H, r = j % N1H;
#pragma unroll
          for (int p = 0; p < NP; p++) {
            if (!bv[p]) continue;
            if constexpr (r < KC) sv[p] = Mma<CT>::mfma(x, kf[p][r], r == 0 ? f32x4{0.f, 0.f, 0.f, 0.f} : sv[p]);
            else dp[p] = Mma<CT>::mfma(x, vf[p][r - KC], r == KC ? f32x4{0.f, 0.f, 0.f, 0.f} : dp[p]);
          }
          if constexpr (r == N1H - 1) {
            // P and dS of the half: p = exp2(s scale - lse2), dS = p (dP - delta)
#pragma unroll
            for (int p = 0; p < NP; p++) {
              const bool hv = !TILE || (q0 + 32 * qb_ + 16 * mb >= vlo[p] && q0 + 32 * qb_ + 16 * mb < vhi[p]);
#pragma unroll
              for (int i = 0; i < 4; i++) {
                float pv = bv[p] ? fast_exp2(fmaf(sv[p][i], scale, -lq[i])) : 0.f;
                if (tail) {
                  const int qi = q0 + 32 * qb_ + 16 * mb + 4 * g + i;
                  pv = (qi >= qmin[p] && qi < a.Lq) ? pv : 0.f;
                }
                if (TILE) pv = hv ? pv : 0.f;
                pr[p][4 * mb + i] = pv;
                ds[p][4 * mb + i] = bv[p] ? pv * (dp[p][i] - dl[i]) : 0.f;
              }
            }
            if constexpr (mb == 1) {
#pragma unroll
              for (int p = 0; p < NP; p++) {
                pb[p] = pack8<CT>(pr[p]);
                dsb[p] = pack8<CT>(ds[p]);
              }
            }
          }
        } else {
          constexpr int d = j - N1;
#pragma unroll
          for (int p = 0; p < NP; p++) {
            if (!bv[p]) continue;
            if constexpr (d < VB) dv_acc[p][d] = Mma<CT>::mfma(x, pb[p], dv_acc[p][d]);
            else dk_acc[p][d - VB] = Mma<CT>::mfma(x, dsb[p], dk_acc[p][d - VB]);
          }
        }
      });
    });
  };
  // Chunk ci lives in buffer ci % NBUF; its copy is started AHEAD chunks before it is consumed (the latency of a copy
  // is longer than the products of one chunk take).  Without a causal mask only the last chunk can be short: the loop
  // bodies then hold no per-pair test.
  int ci = 0, bi = 0;   // bi = ci % NBUF
  auto buf_of = [&](int i) { return smem + (i >= NBUF ? i - NBUF : i) * B::BUF_KV; };
  for (; ci + AHEAD < W.nchunks; ci++) {
    if (CAUSAL) consume_t(ci, (Swa2Lds)buf_of(bi), buf_of(bi + AHEAD), FlashTailDyn{}, std::true_type{});
    else consume_t(ci, (Swa2Lds)buf_of(bi), buf_of(bi + AHEAD), std::false_type{}, std::true_type{});
    flashd_wait_copies<PER_CHUNK>();   // all but the copies just issued: chunk ci + 1 has landed
    __syncthreads();
    bi = bi + 1 == NBUF ? 0 : bi + 1;
  }
  for (; ci + 1 < W.nchunks; ci++) {
    if (CAUSAL) consume_t(ci, (Swa2Lds)buf_of(bi), buf_of(bi + AHEAD), FlashTailDyn{}, std::false_type{});
    else consume_t(ci, (Swa2Lds)buf_of(bi), buf_of(bi + AHEAD), std::false_type{}, std::false_type{});
    swa2_wait_copies();
    __syncthreads();
    bi = bi + 1 == NBUF ? 0 : bi + 1;
  }
  if (W.nchunks > 0) {
    if (CAUSAL) consume_t(ci, (Swa2Lds)buf_of(bi), buf_of(bi + AHEAD), FlashTailDyn{}, std::false_type{});
    else if (chunk_tail(ci)) consume_t(ci, (Swa2Lds)buf_of(bi), buf_of(bi + AHEAD), std::true_type{}, std::false_type{});
    else consume_t(ci, (Swa2Lds)buf_of(bi), buf_of(bi + AHEAD), std::false_type{}, std::false_type{});
  }
  __syncthreads();
  TIO* dkb = reinterpret_cast<TIO*>(a.dk) + b * a.dks[0] + h * a.dks[1];
  TIO* dvb = reinterpret_cast<TIO*>(a.dv) + b * a.dvs[0] + h * a.dvs[1];
  flash_write_grad<TIO, DK, NP>(smem, dk_acc, a.sm_scale, dkb, flash_tok<IMG>(a.dks, a.tm), a.dks[3], a.dk_, a.dk_vec != 0, own_base, x0, a.Lk, wave, n, g, tid);
  flash_write_grad<TIO, DV, NP>(smem, dv_acc, 1.0f, dvb, flash_tok<IMG>(a.dvs, a.tm), a.dvs[3], a.dv_, a.dv_vec != 0, own_base, x0, a.Lk, wave, n, g, tid);
}
