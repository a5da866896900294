// Flash kernels with asynchronous staging: the variants of flash_kernel.hpp for the classes of head dim 64 and 128
// (head dims below the class in multiples of 8: template flag PAD, the copies skip the missing 16-byte pieces, whose
// LDS slots are zeroed once).  Streamed chunks travel HBM -> LDS by the DMA path of the vector
// memory unit (16 bytes per lane, no staging registers, no LDS write instructions) into a ring of two or three chunk
// buffers while an earlier chunk is consumed: one workgroup barrier per chunk instead of two.  LDS rows are 2 D bytes without
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

// Copy of one chunk of CK tokens of a [token][D] tensor by the NW waves of a workgroup: wave w copies tokens
// w CK / NW .. + CK / NW - 1 in NI instructions; instruction i, lane l writes LDS slot l of its 1 KB = physical piece
// l % PIECES of token w CK / NW + TPI i + l / PIECES, and therefore fetches the logical piece (l % PIECES) ^ (SWZ (token & 7)).
template <int D, int CK, int NW = 4>
struct FlashDStage {
  typedef FlashDRow<D> R;
  static constexpr int NI = CK / NW / R::TPI;
  static_assert(NI >= 1 && NI * R::TPI * NW == CK, "chunk must split evenly over the waves' copy instructions");
  int tok0;      // token of the lane in instruction 0
  int lp;        // physical piece the lane writes
  int npieces;   // 16-byte pieces a row of the tensor really has (head dim / 8 <= PIECES)

  DLT_DEV void init(int wave, int lane, int dact) {
    tok0 = wave * (CK / NW) + lane / R::PIECES;
    lp = lane % R::PIECES;
    npieces = dact >> 3;
  }
  // tokens past the end of the chunk are clamped onto its last token (the caller masks them).  With a head dim below
  // the padded one the lanes of the missing pieces copy nothing: their LDS slots were zeroed once (flashd_zero_pads) and
  // no copy ever writes them (PAD: a compile-time flag of the kernels, the test costs the exact-dim kernels 1.5 %).  Every
  // instruction still has active lanes, so the count of copies in flight is the same.
  template <bool PAD, typename AD>
  DLT_DEV void issue(const char* base, const AD& ad, const FlashChunk& c, char* region, int wave) const {
#pragma unroll
    for (int i = 0; i < NI; i++) {
      const int t = tok0 + R::TPI * i;
      const int lgp = lp ^ (R::SWZ * (t & 7));
      const uint32_t off = ad(c, dlt_imin(t, c.nvalid - 1)) + 16u * (uint32_t)lgp;
      char* dst = region + (wave * (CK / NW) + R::TPI * i) * R::ROW;   // wave-uniform
      if (!PAD || lgp < npieces) dlt_copy16_to_lds(base, off, dst);
    }
  }
};

// zeroes the 16-byte slots of a swizzled [ntok][D] region that hold head dims at or beyond 8 * npieces
template <int D>
DLT_DEV void flashd_zero_pads(char* region, int ntok, int npieces, int tid, int nthreads) {
  typedef FlashDRow<D> R;
  if (npieces == R::PIECES) return;
  for (int s = tid; s < ntok * R::PIECES; s += nthreads) {
    const int t = s / R::PIECES, pp = s % R::PIECES;
    if ((pp ^ (R::SWZ * (t & 7))) >= npieces) *reinterpret_cast<u32x4*>(region + s * 16) = u32x4{0u, 0u, 0u, 0u};
  }
}

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

// operands the LDS reads of a chunk loop run ahead of their products (measured on config 5 with exact waits: depths 1
// to 6 lie within 1 %, the deeper ones cost registers; the kernels are bound by the number of LDS reads, not by
// their latency)
#ifndef FLASHD_RD
#define FLASHD_RD 1
#endif

// how the scheduler is asked to place an element-wise piece behind the NP products of its operand
#ifndef FLASHD_EW_MIX
#define FLASHD_EW_MIX SWA2_MIX(NP, 12 / NP)
#endif

// at most N of this wave's copies (the youngest ones) are still in flight
template <int N>
DLT_DEV void flashd_wait_copies() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }

// chunk buffers per workgroup: a copy is started NBUF - 1 chunks ahead of its use; three where two workgroups
// still fit a CU
#ifndef FLASHD_NBUF
#define FLASHD_NBUF(dk, dv) ((dk) + (dv) > 192 ? 2 : 3)
#endif
constexpr int flashd_nbuf(int dk, int dv) { return FLASHD_NBUF(dk, dv); }
// the same for 8-wave workgroups of the backward kernels (one per CU, 64-token chunks; measured slower than 4-wave
// workgroups and not instantiated by default: FLASHD_BWD_NW in flash_inst.hpp)
#ifndef FLASHD_NBUF8
#define FLASHD_NBUF8 3
#endif

template <int DK, int DV, int CK>
struct FlashDBuf {
  static constexpr int REG_A = CK * 2 * DK;            // first tensor of a chunk
  static constexpr int REG_B = CK * 2 * DV;            // second tensor
  static constexpr int SCAL = 2 * CK * 4;              // lse2 then delta (dK/dV kernel)
  static constexpr int BUF = REG_A + REG_B;            // forward, dQ
  static constexpr int BUF_KV = REG_A + REG_B + SCAL;  // dK/dV
};

// ---- dK / dV: own = keys; Q, dO, lse2 and delta stream.  Replaces _attn_bwd_dkdv (src/flash_attn.py:204-307).
template <typename TIO, int DK, int DV, int NP, int CK, int NW, int MODE, bool PAD>
__global__ __launch_bounds__(64 * NW, NW == 4 ? 2 : 1) void flashd_bwd_kv_kernel(const FlashBwdArgs a) {
  typedef typename ComputeOf<TIO>::type CT;
  typedef FlashDBuf<DK, DV, CK> B;
  extern __shared__ __align__(16) char smem[];
  constexpr bool CAUSAL = MODE == 1;
  static_assert(MODE < 2, "asynchronous staging: dense and causal only");
  constexpr int KC = DK / 32, VC = DV / 32, KB = DK / 16, VB = DV / 16, NQB = CK / 32;
  constexpr int OWN = 16 * NP * NW;

  const int tid = threadIdx.x;
  const int lane = tid & 63, n = lane & 15, g = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  const int lin = xcd_remap(blockIdx.x, gridDim.x);
  int bh, r_own, x0;
  if constexpr (CAUSAL) flash_block_causal(lin, a.nblk_k, a.B * a.H, a.causal_group, OWN, false, bh, r_own, x0);
  else flash_block(lin, a.nblk_k, 1, OWN, bh, r_own, x0);
  const int b = bh / a.H, h = bh - b * a.H;
  const TIO* kb_ = reinterpret_cast<const TIO*>(a.k) + b * a.ks[0] + h * a.ks[1];
  const TIO* vb_ = reinterpret_cast<const TIO*>(a.v) + b * a.vs[0] + h * a.vs[1];
  const char* qb = reinterpret_cast<const char*>(reinterpret_cast<const TIO*>(a.q) + b * a.qs[0] + h * a.qs[1]);
  const char* dob = reinterpret_cast<const char*>(reinterpret_cast<const TIO*>(a.d_o) + b * a.dos[0] + h * a.dos[1]);
  const float* lseb = a.lse + b * a.ls[0] + h * a.ls[1];
  const float* delb = a.delta + b * a.ls[0] + h * a.ls[1];
  const FlashAddr<false> aq = flash_addr<false>(a.qs, a.tm), ad = flash_addr<false>(a.dos, a.tm);
  RopeDev no_rope = RopeDev{};

  FlashWalk<MODE, CK> W;
  W.init_seq(CAUSAL ? (x0 / CK) * CK : 0, a.Lq);
  const int wk0 = x0 + wave * 16 * NP;  // first own key of this wave

  FlashDStage<DK, CK, NW> stq;
  FlashDStage<DV, CK, NW> std_;
  stq.init(wave, lane, a.dk_);
  std_.init(wave, lane, a.dv_);
  // waves 0 and 1 also copy the chunk's lse2 / delta
  const float* scal_base = wave == 0 ? lseb : delb;
  auto issue = [&](const FlashChunk& c, char* buf) {
    stq.template issue<PAD>(qb, aq, c, buf, wave);
    std_.template issue<PAD>(dob, ad, c, buf + B::REG_A, wave);
    if (wave < 2) flashd_issue_scalars<CK>(scal_base, (int)a.ls[2], c, buf + B::REG_A + B::REG_B + wave * (CK * 4), lane);
  };
  constexpr int NBUF = NW == 4 ? flashd_nbuf(DK, DV) : FLASHD_NBUF8, AHEAD = NBUF - 1;
  constexpr int PER_CHUNK = FlashDStage<DK, CK, NW>::NI + FlashDStage<DV, CK, NW>::NI;   // copies per wave and chunk (waves 0, 1: more)
  // head dims below the padded ones: the slots of the missing pieces are zeroed once, no copy writes them
#pragma unroll
  for (int i = 0; PAD && i < NBUF; i++) {
    flashd_zero_pads<DK>(smem + i * B::BUF_KV, CK, a.dk_ >> 3, tid, 64 * NW);
    flashd_zero_pads<DV>(smem + i * B::BUF_KV + B::REG_A, CK, a.dv_ >> 3, tid, 64 * NW);
  }
#pragma unroll
  for (int i = 0; i < AHEAD; i++)
    if (i < W.nchunks) issue(W.at(i), smem + i * B::BUF_KV);

  u32x4 kf[NP][KC], vf[NP][VC];
  int qmin[NP];           // causal: first query that sees this lane's key
#pragma unroll
  for (int p = 0; p < NP; p++) {
    const int xk = wk0 + 16 * p + n;
    const int64_t tk = xk < a.Lk ? (int64_t)xk : (int64_t)-1;
    qmin[p] = CAUSAL ? xk : 0;
    swa1_load_own<TIO, CT, DK>(kf[p], kb_, 1, a.dk_, flash_own_off<false>(a.ks, a.tm, tk), g, no_rope, false);
    swa1_load_own<TIO, CT, DV>(vf[p], vb_, 1, a.dv_, flash_own_off<false>(a.vs, a.tm, tk), g, no_rope, false);
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
  // the compiler does not see that wait: tell it that the own fragments are loaded, or it waits for them (and with them
  // for every copy in flight) at their first use inside every round of the chunk loop
  pin_loaded(kf);
  pin_loaded(vf);
  // The own values are negated and the dP products start from the staged delta of the lane's four queries, read from LDS
  // straight into the C operand of the first product of a chain: the matrix pipe delivers -(dP - delta), and dS = -p (.)
  // (the sign is an operand modifier).
#pragma unroll
  for (int p = 0; p < NP; p++)
#pragma unroll
    for (int c = 0; c < VC; c++) {
      vf[p][c].x ^= 0x80008000u; vf[p][c].y ^= 0x80008000u; vf[p][c].z ^= 0x80008000u; vf[p][c].w ^= 0x80008000u;
    }
  __syncthreads();

  auto chunk_tail = [&](const int ci) {
    const FlashChunk c = W.at(ci);
    return c.nvalid < CK || (CAUSAL && c.x < wk0 + 16 * NP - 1);
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
    if (CAUSAL && !std::is_same<decltype(tail_tag), std::false_type>::value && q0 + CK - 1 < wk0) return;
    // Order of a chunk's operands: the first products (S, dP) of every 16-query half of every block, then the second
    // products (dV, dK) block by block.  The element-wise work of a half (P, dS: vector instructions that depend on its
    // first products) is issued in pieces behind the matrix instructions of the FOLLOWING segment, which do not depend on
    // it: a wave issues in order, and with the element-wise work directly behind the products it waits for, matrix pipe
    // and vector ALU take turns instead of running side by side.
    constexpr int N1H = KC + VC, NH = 2 * NQB, N1 = NH * N1H, NP2 = VB + KB, NT = N1 + NQB * NP2;
    constexpr int NU = 2 * NP;   // element-wise pieces of a half: (own block p, pair of queries)
    static_assert(N1H >= NU && NP2 >= NU, "a segment must have room for the element-wise pieces of a half");
    constexpr int RD = FLASHD_RD;
    u32x4 ring[RD + 1];
    auto rd = [&](auto kc) __attribute__((always_inline)) {
      constexpr int k = decltype(kc)::value;
      if constexpr (k < N1) {
        constexpr int hh = k / N1H, r = k % N1H, T0 = 16 * hh;
        if constexpr (r < KC) ring[k % (RD + 1)] = swa2_lds16(sQ + T0 * FlashDRow<DK>::ROW + LQ.a[r]);
        else ring[k % (RD + 1)] = swa2_lds16(sDO + T0 * FlashDRow<DV>::ROW + LD.a[r - KC]);
      } else {
        constexpr int qb_ = (k - N1) / NP2, d = (k - N1) % NP2;
        if constexpr (d < VB) ring[k % (RD + 1)] = flashd_read_tr<DV, 32 * qb_>(sDO, LD, d);
        else ring[k % (RD + 1)] = flashd_read_tr<DK, 32 * qb_>(sQ, LQ, d - VB);
      }
    };
    swa2_for<0, RD>([&](auto kc) __attribute__((always_inline)) { rd(kc); });
    f32x4 sv[2][NP], dp[2][NP], lq[2], dl[2];   // indexed by the parity of the half
    // delta of the lane's four queries of a half is the C operand of its first dP product: read one half ahead
    dl[0] = __builtin_bit_cast(f32x4, swa2_lds16(sDel));
    u32x4 pb[NQB][NP], dsb[NQB][NP];
    // piece u of the element-wise work of half hh: p = exp2(s scale - lse2), dS = p (dP - delta) for own block u / 2,
    // queries 2 (u % 2), 2 (u % 2) + 1 of the lane's four
    auto ew = [&](auto hhc, auto uc) __attribute__((always_inline)) {
      constexpr int hh = decltype(hhc)::value, u = decltype(uc)::value;
      constexpr int qb_ = hh / 2, mb = hh % 2, p = u / 2, i0_ = 2 * (u % 2);
      float pr[2], ds[2];
#pragma unroll
      for (int t = 0; t < 2; t++) {
        const int i = i0_ + t;
        float pv = fast_exp2(fmaf(sv[hh & 1][p][i], scale, -lq[hh & 1][i]));
        if (tail) {
          const int qi = q0 + 16 * hh + 4 * g + i;
          pv = (qi >= qmin[p] && qi < a.Lq) ? pv : 0.f;
        }
        pr[t] = pv;
        ds[t] = -pv * dp[hh & 1][p][i];
      }
      const unsigned pw = pack2<CT>(pr[0], pr[1]), dw = pack2<CT>(ds[0], ds[1]);
      if constexpr (mb == 0 && i0_ == 0) { pb[qb_][p].x = pw; dsb[qb_][p].x = dw; }
      if constexpr (mb == 0 && i0_ == 2) { pb[qb_][p].y = pw; dsb[qb_][p].y = dw; }
      if constexpr (mb == 1 && i0_ == 0) { pb[qb_][p].z = pw; dsb[qb_][p].z = dw; }
      if constexpr (mb == 1 && i0_ == 2) { pb[qb_][p].w = pw; dsb[qb_][p].w = dw; }
    };
    swa2_for<0, NT>([&](auto kc) __attribute__((always_inline)) {
      constexpr int k = decltype(kc)::value;
      if constexpr (k + RD < NT) rd(std::integral_constant<int, k + RD>{});
      if constexpr (k < N1 && k % N1H == 0) {
        constexpr int hh = k / N1H;
        lq[hh & 1] = __builtin_bit_cast(f32x4, swa2_lds16(sLse + 16 * hh * 4));
      }
      if constexpr (k < N1 && k % N1H == KC && k / N1H + 1 < NH) {
        // (the dP products of half hh - 1 consumed the registers this overwrites)
        constexpr int hn = k / N1H + 1;
        dl[hn & 1] = __builtin_bit_cast(f32x4, swa2_lds16(sDel + 16 * hn * 4));
      }
      __builtin_amdgcn_sched_barrier(0);
      const u32x4 x = ring[k % (RD + 1)];
      if constexpr (k < N1) {
        constexpr int hh = k / N1H, r = k % N1H;
#pragma unroll
        for (int p = 0; p < NP; p++) {
          if constexpr (r < KC) sv[hh & 1][p] = Mma<CT>::mfma(x, kf[p][r], r == 0 ? f32x4{0.f, 0.f, 0.f, 0.f} : sv[hh & 1][p]);
          else dp[hh & 1][p] = Mma<CT>::mfma(x, vf[p][r - KC], r == KC ? dl[hh & 1] : dp[hh & 1][p]);
        }
        if constexpr (hh >= 1 && r < NU) {
          ew(std::integral_constant<int, hh - 1>{}, std::integral_constant<int, r>{});
          FLASHD_EW_MIX
        }
      } else {
        constexpr int qb_ = (k - N1) / NP2, d = (k - N1) % NP2;
#pragma unroll
        for (int p = 0; p < NP; p++) {
          if constexpr (d < VB) dv_acc[p][d] = Mma<CT>::mfma(x, pb[qb_][p], dv_acc[p][d]);
          else dk_acc[p][d - VB] = Mma<CT>::mfma(x, dsb[qb_][p], dk_acc[p][d - VB]);
        }
        if constexpr (qb_ == 0 && d < NU) {
          ew(std::integral_constant<int, NH - 1>{}, std::integral_constant<int, d>{});
          FLASHD_EW_MIX
        }
      }
    });
  };
  // Chunk ci lives in buffer ci % NBUF; its copy is started AHEAD chunks before it is consumed (the latency of a copy
  // is longer than the products of one chunk take).  Without a causal mask only the last chunk can be short: the loop
  // bodies then hold no per-pair test.
  int ci = 0, bi = 0;   // bi = ci % NBUF
  auto buf_of = [&](int i) { return smem + (i >= NBUF ? i - NBUF : i) * B::BUF_KV; };
  if constexpr (CAUSAL) {
    // the chunks on the diagonal come first: per-chunk and per-pair tests; every later chunk but the last is full and
    // lies below every own key, its body holds no test (as without a mask)
    for (; ci + AHEAD < W.nchunks && W.at(ci).x < x0 + OWN - 1; ci++) {
      consume_t(ci, (Swa2Lds)buf_of(bi), buf_of(bi + AHEAD), FlashTailDyn{}, std::true_type{});
      flashd_wait_copies<(AHEAD - 1) * PER_CHUNK>();
      __syncthreads();
      bi = bi + 1 == NBUF ? 0 : bi + 1;
    }
  }
  for (; ci + AHEAD < W.nchunks; ci++) {
    consume_t(ci, (Swa2Lds)buf_of(bi), buf_of(bi + AHEAD), std::false_type{}, std::true_type{});
    flashd_wait_copies<(AHEAD - 1) * PER_CHUNK>();   // chunk ci + 1 has landed: all copies but those of the AHEAD - 1 chunks behind it
    __syncthreads();
    bi = bi + 1 == NBUF ? 0 : bi + 1;
  }
  // without a mask a full last chunk runs here too (same test-free body): the code below, whose per-pair tests cost
  // registers the compiler finds by spilling, is then not executed at all
  const int n_plain = (!CAUSAL && W.nchunks > 0 && !chunk_tail(W.nchunks - 1)) ? W.nchunks : W.nchunks - 1;
  for (; ci < n_plain; ci++) {
    if (CAUSAL) consume_t(ci, (Swa2Lds)buf_of(bi), buf_of(bi + AHEAD), FlashTailDyn{}, std::false_type{});
    else consume_t(ci, (Swa2Lds)buf_of(bi), buf_of(bi + AHEAD), std::false_type{}, std::false_type{});
    swa2_wait_copies();
    __syncthreads();
    bi = bi + 1 == NBUF ? 0 : bi + 1;
  }
  if (ci < W.nchunks) {
    if (CAUSAL) consume_t(ci, (Swa2Lds)buf_of(bi), buf_of(bi + AHEAD), FlashTailDyn{}, std::false_type{});
    else consume_t(ci, (Swa2Lds)buf_of(bi), buf_of(bi + AHEAD), std::true_type{}, std::false_type{});
  }
  __syncthreads();
  TIO* dkb = reinterpret_cast<TIO*>(a.dk) + b * a.dks[0] + h * a.dks[1];
  TIO* dvb = reinterpret_cast<TIO*>(a.dv) + b * a.dvs[0] + h * a.dvs[1];
  flash_write_grad<TIO, DK, NP>(smem, dk_acc, a.sm_scale, dkb, flash_tok<false>(a.dks, a.tm), a.dks[3], a.dk_, a.dk_vec != 0, 0, x0, a.Lk, wave, n, g, tid, OWN);
  flash_write_grad<TIO, DV, NP>(smem, dv_acc, 1.0f, dvb, flash_tok<false>(a.dvs, a.tm), a.dvs[3], a.dv_, a.dv_vec != 0, 0, x0, a.Lk, wave, n, g, tid, OWN);
}

// ---- forward: own = queries; K and V stream.  Replaces _attn_fwd (src/flash_attn.py:81-172).
// Per chunk: S^T = K Q^T for every 32-key block (a stream of NKB 2 KC operand reads, NP products each), one softmax
// update per query block, then O^T += V^T P^T (NKB VB transposed operands) with the row sums from a ones-row product.
// The reads of the second stream are already in flight while the softmax runs.
template <typename TIO, int DK, int DV, int NP, int CK, int NW, int MODE, bool PAD>
__global__ __launch_bounds__(64 * NW, NW == 4 ? 2 : 1) void flashd_fwd_kernel(const FlashArgs a) {
  typedef typename ComputeOf<TIO>::type CT;
  typedef typename TileOf<TIO>::type TL;
  typedef FlashDBuf<DK, DV, CK> B;
  extern __shared__ __align__(16) char smem[];
  constexpr bool CAUSAL = MODE == 1;
  static_assert(MODE < 2, "asynchronous staging: dense and causal only");
  constexpr int PO = DV * (int)sizeof(TL) + 16;
  constexpr int KC = DK / 32, VB = DV / 16, NKB = CK / 32;
  constexpr int OWN = 16 * NP * NW;
  constexpr int NBUF = NW == 4 ? flashd_nbuf(DK, DV) : 2, AHEAD = NBUF - 1;   // forward: 128-key chunks
  constexpr int PER_CHUNK = FlashDStage<DK, CK, NW>::NI + FlashDStage<DV, CK, NW>::NI;

  const int tid = threadIdx.x;
  const int lane = tid & 63, n = lane & 15, g = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  const int lin = xcd_remap(blockIdx.x, gridDim.x);
  int bh, r_own, x0;
  if constexpr (CAUSAL) flash_block_causal(lin, a.nblk, a.B * a.H, a.causal_group, OWN, true, bh, r_own, x0);
  else flash_block(lin, a.nblk, 1, OWN, bh, r_own, x0);
  const int wq0 = x0 + wave * 16 * NP;
  const int b = bh / a.H, h = bh - b * a.H;
  const TIO* qb = reinterpret_cast<const TIO*>(a.q) + b * a.qs[0] + h * a.qs[1];
  const char* kb_ = reinterpret_cast<const char*>(reinterpret_cast<const TIO*>(a.k) + b * a.ks[0] + h * a.ks[1]);
  const char* vb_ = reinterpret_cast<const char*>(reinterpret_cast<const TIO*>(a.v) + b * a.vs[0] + h * a.vs[1]);
  TIO* ob = reinterpret_cast<TIO*>(a.o) + b * a.os[0] + h * a.os[1];
  const FlashAddr<false> ak = flash_addr<false>(a.ks, a.tm), av = flash_addr<false>(a.vs, a.tm);
  RopeDev no_rope = RopeDev{};

  FlashWalk<MODE, CK> W;
  W.init_seq(0, CAUSAL ? dlt_imin(a.Lk, x0 + OWN) : a.Lk);

  FlashDStage<DK, CK, NW> stk;
  FlashDStage<DV, CK, NW> stv;
  stk.init(wave, lane, a.dk);
  stv.init(wave, lane, a.dv);
  // head dims below the padded ones: the slots of the missing pieces are zeroed once, no copy writes them
#pragma unroll
  for (int i = 0; PAD && i < NBUF; i++) {
    flashd_zero_pads<DK>(smem + i * B::BUF, CK, a.dk >> 3, tid, 64 * NW);
    flashd_zero_pads<DV>(smem + i * B::BUF + B::REG_A, CK, a.dv >> 3, tid, 64 * NW);
  }
  auto issue = [&](const FlashChunk& c, char* buf) {
    stk.template issue<PAD>(kb_, ak, c, buf, wave);
    stv.template issue<PAD>(vb_, av, c, buf + B::REG_A, wave);
  };
#pragma unroll
  for (int i = 0; i < AHEAD; i++)
    if (i < W.nchunks) issue(W.at(i), smem + i * B::BUF);

  u32x4 qf[NP][KC];
  int64_t tq[NP];
  int klim[NP];
#pragma unroll
  for (int p = 0; p < NP; p++) {
    const int xq = wq0 + 16 * p + n;
    tq[p] = xq < a.Lq ? (int64_t)xq : (int64_t)-1;
    klim[p] = CAUSAL ? dlt_imin(xq, a.Lk - 1) : a.Lk - 1;
    swa1_load_own<TIO, CT, DK>(qf[p], qb, 1, a.dk, flash_own_off<false>(a.qs, a.tm, tq[p]), g, no_rope, false);
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
  FlashDLane<DK> LK;
  FlashDLane<DV> LV;
  flashd_lane_init(LK, n, g);
  flashd_lane_init(LV, n, g);

  swa2_wait_copies();   // also: the own fragments have arrived
  // the compiler does not see that wait: tell it that the own fragments are loaded, or it waits for them (and with them
  // for every copy in flight) at their first use inside every round of the chunk loop
  pin_loaded(qf);
  __syncthreads();

  auto chunk_tail = [&](const int ci) {
    const FlashChunk c = W.at(ci);
    return c.nvalid < CK || (CAUSAL && c.x + CK - 1 > wq0);
  };
  auto consume_t = [&](const int ci, Swa2Lds __restrict__ cur, char* __restrict__ nxt, auto tail_tag, auto more_tag) __attribute__((always_inline)) {
    bool tail;
    if constexpr (std::is_same<decltype(tail_tag), FlashTailDyn>::value) tail = chunk_tail(ci);
    else tail = decltype(tail_tag)::value;
    if constexpr (decltype(more_tag)::value) issue(W.at(ci + AHEAD), nxt);
    Swa2Lds sK = cur, sV = cur + B::REG_A;
    const FlashChunk c = W.at(ci);
    const int k0 = c.x;
    // causal: every key of the chunk lies above every query of this wave
    if (CAUSAL && !std::is_same<decltype(tail_tag), std::false_type>::value && k0 > wq0 + 16 * NP - 1) return;
    constexpr int N1 = NKB * 2 * KC, NT = N1 + NKB * VB;
    constexpr int RD = FLASHD_RD;
    u32x4 ring[RD + 1];
    auto rd = [&](auto kc) __attribute__((always_inline)) {
      constexpr int k = decltype(kc)::value;
      if constexpr (k < N1) {
        constexpr int kb = k / (2 * KC), mb = (k / KC) % 2, r = k % KC;
        ring[k % (RD + 1)] = swa2_lds16(sK + (32 * kb + 16 * mb) * FlashDRow<DK>::ROW + LK.a[r]);
      } else {
        constexpr int kb = (k - N1) / VB, d = (k - N1) % VB;
        ring[k % (RD + 1)] = flashd_read_tr<DV, 32 * kb>(sV, LV, d);
      }
    };
    swa2_for<0, RD>([&](auto kc) __attribute__((always_inline)) { rd(kc); });
    float t[NP][NKB][8];
    u32x4 pb[NP][NKB];
    f32x4 s[NP];
    swa2_for<0, NT>([&](auto kc) __attribute__((always_inline)) {
      constexpr int k = decltype(kc)::value;
      if constexpr (k + RD < NT) rd(std::integral_constant<int, k + RD>{});
      __builtin_amdgcn_sched_barrier(0);
      const u32x4 x = ring[k % (RD + 1)];
      if constexpr (k < N1) {
        constexpr int kb = k / (2 * KC), mb = (k / KC) % 2, r = k % KC;
#pragma unroll
        for (int p = 0; p < NP; p++) s[p] = Mma<CT>::mfma(x, qf[p][r], r == 0 ? f32x4{0.f, 0.f, 0.f, 0.f} : s[p]);
        if constexpr (r == KC - 1) {
#pragma unroll
          for (int p = 0; p < NP; p++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
              float v = s[p][i];
              if (tail) v = (k0 + 32 * kb + 16 * mb + 4 * g + i) <= klim[p] ? v : -INFINITY;
              t[p][kb][4 * mb + i] = v;
            }
        }
        if constexpr (k == N1 - 1) {
          // one softmax update per query block on the raw scores of the chunk
#pragma unroll
          for (int p = 0; p < NP; p++) {
            float mx[4] = {-INFINITY, -INFINITY, -INFINITY, -INFINITY};
#pragma unroll
            for (int kb2 = 0; kb2 < NKB; kb2++)
#pragma unroll
              for (int i = 0; i < 4; i++) mx[i] = fmaxf(fmaxf(mx[i], t[p][kb2][2 * i]), t[p][kb2][2 * i + 1]);
            const float mloc = wave_max4(fmaxf(fmaxf(mx[0], mx[1]), fmaxf(mx[2], mx[3])));
            // the reference maximum only moves when a score exceeds it by more than 2^8 after scaling (see flash_kernel.hpp)
            if (__builtin_amdgcn_ballot_w64((mloc - m_run[p]) * scale > 8.f)) {
              keep_branch();
              const float m_new = fmaxf(m_run[p], mloc);
              const float alpha = fast_exp2((m_run[p] - m_new) * scale);
              m_run[p] = m_new;
#pragma unroll
              for (int d = 0; d < VB; d++) acc[p][d] *= alpha;
              acc_l[p] *= alpha;
            }
            const float neg_m2 = m_run[p] == -INFINITY ? 0.f : -m_run[p] * scale;
#pragma unroll
            for (int kb2 = 0; kb2 < NKB; kb2++) {
#pragma unroll
              for (int i = 0; i < 8; i++) t[p][kb2][i] = fast_exp2(fmaf(t[p][kb2][i], scale, neg_m2));
              pb[p][kb2] = pack8<CT>(t[p][kb2]);
            }
          }
        }
      } else {
        constexpr int kb = (k - N1) / VB, d = (k - N1) % VB;
#pragma unroll
        for (int p = 0; p < NP; p++) acc[p][d] = Mma<CT>::mfma(x, pb[p][kb], acc[p][d]);
        if constexpr (d == VB - 1) {
#pragma unroll
          for (int p = 0; p < NP; p++) acc_l[p] = Mma<CT>::mfma(ones, pb[p][kb], acc_l[p]);
        }
      }
    });
  };
  int ci = 0, bi = 0;
  auto buf_of = [&](int i) { return smem + (i >= NBUF ? i - NBUF : i) * B::BUF; };
  if constexpr (CAUSAL) {
    // the chunks below the first query of the workgroup: every wave sees every pair, the body holds no test (as without
    // a mask); the chunks on the diagonal follow with the per-chunk and per-pair tests
    const int nfull = dlt_imin(x0, W.len) / CK;
    for (; ci + AHEAD < W.nchunks && ci < nfull; ci++) {
      consume_t(ci, (Swa2Lds)buf_of(bi), buf_of(bi + AHEAD), std::false_type{}, std::true_type{});
      flashd_wait_copies<(AHEAD - 1) * PER_CHUNK>();
      __syncthreads();
      bi = bi + 1 == NBUF ? 0 : bi + 1;
    }
  }
  for (; ci + AHEAD < W.nchunks; ci++) {
    if (CAUSAL) consume_t(ci, (Swa2Lds)buf_of(bi), buf_of(bi + AHEAD), FlashTailDyn{}, std::true_type{});
    else consume_t(ci, (Swa2Lds)buf_of(bi), buf_of(bi + AHEAD), std::false_type{}, std::true_type{});
    flashd_wait_copies<(AHEAD - 1) * PER_CHUNK>();
    __syncthreads();
    bi = bi + 1 == NBUF ? 0 : bi + 1;
  }
  // without a mask a full last chunk runs here too (same test-free body): the code below, whose per-pair tests cost
  // registers the compiler finds by spilling, is then not executed at all
  const int n_plain = (!CAUSAL && W.nchunks > 0 && !chunk_tail(W.nchunks - 1)) ? W.nchunks : W.nchunks - 1;
  for (; ci < n_plain; ci++) {
    if (CAUSAL) consume_t(ci, (Swa2Lds)buf_of(bi), buf_of(bi + AHEAD), FlashTailDyn{}, std::false_type{});
    else consume_t(ci, (Swa2Lds)buf_of(bi), buf_of(bi + AHEAD), std::false_type{}, std::false_type{});
    swa2_wait_copies();
    __syncthreads();
    bi = bi + 1 == NBUF ? 0 : bi + 1;
  }
  if (ci < W.nchunks) {
    if (CAUSAL) consume_t(ci, (Swa2Lds)buf_of(bi), buf_of(bi + AHEAD), FlashTailDyn{}, std::false_type{});
    else consume_t(ci, (Swa2Lds)buf_of(bi), buf_of(bi + AHEAD), std::true_type{}, std::false_type{});
  }
  __syncthreads();

  // ---- epilogue: normalise, O^T fragments -> LDS tile -> coalesced rows
#pragma unroll
  for (int p = 0; p < NP; p++) {
    const float lt = wave_sum4(acc_l[p][0]);
    const float inv = lt > 0.f ? fast_rcp(lt) : 0.f;
    TL* orow = reinterpret_cast<TL*>(smem + (wave * 16 * NP + 16 * p + n) * PO);
#pragma unroll
    for (int d = 0; d < VB; d++)
#pragma unroll
      for (int i = 0; i < 4; i++) orow[16 * d + 4 * g + i] = (TL)(acc[p][d][i] * inv);
    if (g == 0 && tq[p] >= 0) store_stream4(a.lse + (b * a.ls[0] + h * a.ls[1] + tq[p] * a.ls[2]), m_run[p] * scale + fast_log2(lt));
  }
  __syncthreads();
  int tw = tid;   // opaque copy: keeps the tile writer's addresses out of the registers that live across the chunk loop
  asm volatile("" : "+v"(tw));
  if (tw < 256)   // the tile writer walks the rows with 256 threads
    store_tile<TIO, TL, DV>(smem, PO, ob, flash_tok<false>(a.os, a.tm), a.os[3], a.dv, a.o_vec != 0, OWN,
                            [&](int row) { return x0 + row < a.Lq ? (int64_t)(x0 + row) : (int64_t)-1; }, no_rope, tw);
}

// ---- dQ: own = queries; K and V stream.  Replaces _attn_bwd_dq (src/flash_attn.py:310-449) and, with fuse_delta, the
// delta pre-pass (:186-202).  Per 32-key block: per 16-key half KC pieces of K (S = K Q^T) and VC pieces of V
// (dP = V dO^T), then KB transposed pieces of K (dQ^T += K^T dS).
template <typename TIO, int DK, int DV, int NP, int CK, int NW, int MODE, bool PAD>
__global__ __launch_bounds__(64 * NW, NW == 4 ? 2 : 1) void flashd_bwd_q_kernel(const FlashBwdArgs a) {
  typedef typename ComputeOf<TIO>::type CT;
  typedef FlashDBuf<DK, DV, CK> B;
  extern __shared__ __align__(16) char smem[];
  constexpr bool CAUSAL = MODE == 1;
  static_assert(MODE < 2, "asynchronous staging: dense and causal only");
  constexpr int KC = DK / 32, VC = DV / 32, KB = DK / 16, NKB = CK / 32;
  constexpr int OWN = 16 * NP * NW;
  constexpr int NBUF = NW == 4 ? flashd_nbuf(DK, DV) : FLASHD_NBUF8, AHEAD = NBUF - 1;
  constexpr int PER_CHUNK = FlashDStage<DK, CK, NW>::NI + FlashDStage<DV, CK, NW>::NI;

  const int tid = threadIdx.x;
  const int lane = tid & 63, n = lane & 15, g = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  const int lin = xcd_remap(blockIdx.x, gridDim.x);
  int bh, r_own, x0;
  if constexpr (CAUSAL) flash_block_causal(lin, a.nblk_q, a.B * a.H, a.causal_group, OWN, true, bh, r_own, x0);
  else flash_block(lin, a.nblk_q, 1, OWN, bh, r_own, x0);
  const int wq0 = x0 + wave * 16 * NP;
  const int b = bh / a.H, h = bh - b * a.H;
  const TIO* qb = reinterpret_cast<const TIO*>(a.q) + b * a.qs[0] + h * a.qs[1];
  const TIO* dob = reinterpret_cast<const TIO*>(a.d_o) + b * a.dos[0] + h * a.dos[1];
  const char* kb_ = reinterpret_cast<const char*>(reinterpret_cast<const TIO*>(a.k) + b * a.ks[0] + h * a.ks[1]);
  const char* vb_ = reinterpret_cast<const char*>(reinterpret_cast<const TIO*>(a.v) + b * a.vs[0] + h * a.vs[1]);
  const FlashAddr<false> ak = flash_addr<false>(a.ks, a.tm), av = flash_addr<false>(a.vs, a.tm);
  RopeDev no_rope = RopeDev{};

  FlashWalk<MODE, CK> W;
  W.init_seq(0, CAUSAL ? dlt_imin(a.Lk, x0 + OWN) : a.Lk);

  FlashDStage<DK, CK, NW> stk;
  FlashDStage<DV, CK, NW> stv;
  stk.init(wave, lane, a.dk_);
  stv.init(wave, lane, a.dv_);
  // head dims below the padded ones: the slots of the missing pieces are zeroed once, no copy writes them
#pragma unroll
  for (int i = 0; PAD && i < NBUF; i++) {
    flashd_zero_pads<DK>(smem + i * B::BUF, CK, a.dk_ >> 3, tid, 64 * NW);
    flashd_zero_pads<DV>(smem + i * B::BUF + B::REG_A, CK, a.dv_ >> 3, tid, 64 * NW);
  }
  auto issue = [&](const FlashChunk& c, char* buf) {
    stk.template issue<PAD>(kb_, ak, c, buf, wave);
    stv.template issue<PAD>(vb_, av, c, buf + B::REG_A, wave);
  };
#pragma unroll
  for (int i = 0; i < AHEAD; i++)
    if (i < W.nchunks) issue(W.at(i), smem + i * B::BUF);

  u32x4 qf[NP][KC], dof[NP][VC];
  float nlse[NP], del_n[NP];
  int klim[NP];
#pragma unroll
  for (int p = 0; p < NP; p++) {
    const int xq = wq0 + 16 * p + n;
    const int64_t tq = xq < a.Lq ? (int64_t)xq : (int64_t)-1;
    klim[p] = CAUSAL ? dlt_imin(xq, a.Lk - 1) : a.Lk - 1;
    swa1_load_own<TIO, CT, DK>(qf[p], qb, 1, a.dk_, flash_own_off<false>(a.qs, a.tm, tq), g, no_rope, false);
    swa1_load_own<TIO, CT, DV>(dof[p], dob, 1, a.dv_, flash_own_off<false>(a.dos, a.tm, tq), g, no_rope, false);
    const int64_t off = b * a.ls[0] + h * a.ls[1] + (tq >= 0 ? tq : 0) * a.ls[2];
    nlse[p] = tq >= 0 ? -a.lse[off] : 0.f;
    if (a.fuse_delta != 0) {
      const TIO* ob = reinterpret_cast<const TIO*>(a.o) + b * a.os[0] + h * a.os[1];
      u32x4 of[VC];
      swa1_load_own<TIO, CT, DV>(of, ob, 1, a.dv_, flash_own_off<false>(a.os, a.tm, tq), g, no_rope, false);
      float part = 0.f;
#pragma unroll
      for (int c_ = 0; c_ < VC; c_++) {
        float fo[8], fd[8];
        unpack8<CT>(of[c_], fo);
        unpack8<CT>(dof[p][c_], fd);
#pragma unroll
        for (int j = 0; j < 8; j++) part += fo[j] * fd[j];
      }
      del_n[p] = wave_sum4(part);
      if (g == 0 && tq >= 0) store_stream4(a.delta_out + off, del_n[p]);
    } else {
      del_n[p] = tq >= 0 ? a.delta[off] : 0.f;
    }
  }
  f32x4 dq_acc[NP][KB];
#pragma unroll
  for (int p = 0; p < NP; p++)
#pragma unroll
    for (int d = 0; d < KB; d++) dq_acc[p][d] = f32x4{0.f, 0.f, 0.f, 0.f};
  const float scale = a.scale_log2;
  FlashDLane<DK> LK;
  FlashDLane<DV> LV;
  flashd_lane_init(LK, n, g);
  flashd_lane_init(LV, n, g);

  swa2_wait_copies();   // also: the own fragments and scalars have arrived
  // the compiler does not see that wait: tell it that the own fragments are loaded, or it waits for them (and with them
  // for every copy in flight) at their first use inside every round of the chunk loop
  pin_loaded(qf);
  pin_loaded(dof);
#pragma unroll
  for (int p = 0; p < NP; p++) { pin_loaded(nlse[p]); pin_loaded(del_n[p]); }
  // The dP products start from -delta of the lane's query (the C operand of the first product of a chain): the matrix
  // pipe delivers dP - delta.  (Folding the scale into the own queries and -lse2 into the score products the same way
  // would save two more vector instructions per score, but rounds q sm_scale to 16 bits: at bf16 the forward error grew
  // from 1.0e-2 to 2.6e-2 at sm_scale sqrt(d) = 4.)
  f32x4 dinit[NP];
#pragma unroll
  for (int p = 0; p < NP; p++) dinit[p] = f32x4{-del_n[p], -del_n[p], -del_n[p], -del_n[p]};
  __syncthreads();

  auto chunk_tail = [&](const int ci) {
    const FlashChunk c = W.at(ci);
    return c.nvalid < CK || (CAUSAL && c.x + CK - 1 > wq0);
  };
  auto consume_t = [&](const int ci, Swa2Lds __restrict__ cur, char* __restrict__ nxt, auto tail_tag, auto more_tag) __attribute__((always_inline)) {
    bool tail;
    if constexpr (std::is_same<decltype(tail_tag), FlashTailDyn>::value) tail = chunk_tail(ci);
    else tail = decltype(tail_tag)::value;
    if constexpr (decltype(more_tag)::value) issue(W.at(ci + AHEAD), nxt);
    Swa2Lds sK = cur, sV = cur + B::REG_A;
    const FlashChunk c = W.at(ci);
    const int k0 = c.x;
    if (CAUSAL && !std::is_same<decltype(tail_tag), std::false_type>::value && k0 > wq0 + 16 * NP - 1) return;
    constexpr int N1H = KC + VC, N1 = 2 * N1H, NB = N1 + KB, NT = NKB * NB;
    constexpr int RD = FLASHD_RD;
    u32x4 ring[RD + 1];
    auto rd = [&](auto kc) __attribute__((always_inline)) {
      constexpr int k = decltype(kc)::value;
      constexpr int kb = k / NB, j = k % NB;
      if constexpr (j < N1) {
        constexpr int mb = j / N1H, r = j % N1H, T0 = 32 * kb + 16 * mb;
        if constexpr (r < KC) ring[k % (RD + 1)] = swa2_lds16(sK + T0 * FlashDRow<DK>::ROW + LK.a[r]);
        else ring[k % (RD + 1)] = swa2_lds16(sV + T0 * FlashDRow<DV>::ROW + LV.a[r - KC]);
      } else {
        ring[k % (RD + 1)] = flashd_read_tr<DK, 32 * kb>(sK, LK, j - N1);
      }
    };
    swa2_for<0, RD>([&](auto kc) __attribute__((always_inline)) { rd(kc); });
    swa2_for<0, NKB>([&](auto kbc) __attribute__((always_inline)) {
      constexpr int kb = decltype(kbc)::value;
      float ds[NP][8];
      f32x4 sv[NP], dp[NP];
      u32x4 dsb[NP];
      swa2_for<0, NB>([&](auto jc) __attribute__((always_inline)) {
        constexpr int j = decltype(jc)::value, k = kb * NB + j;
        if constexpr (k + RD < NT) rd(std::integral_constant<int, k + RD>{});
        __builtin_amdgcn_sched_barrier(0);
        const u32x4 x = ring[k % (RD + 1)];
        if constexpr (j < N1) {
          constexpr int mb = j / N1H, r = j % N1H;
#pragma unroll
          for (int p = 0; p < NP; p++) {
            if constexpr (r < KC) sv[p] = Mma<CT>::mfma(x, qf[p][r], r == 0 ? f32x4{0.f, 0.f, 0.f, 0.f} : sv[p]);
            else dp[p] = Mma<CT>::mfma(x, dof[p][r - KC], r == KC ? dinit[p] : dp[p]);
          }
          if constexpr (r == N1H - 1) {
#pragma unroll
            for (int p = 0; p < NP; p++) {
#pragma unroll
              for (int i = 0; i < 4; i++) {
                float pv = fast_exp2(fmaf(sv[p][i], scale, nlse[p]));
                if (tail) pv = (k0 + 32 * kb + 16 * mb + 4 * g + i) <= klim[p] ? pv : 0.f;
                ds[p][4 * mb + i] = pv * dp[p][i];
              }
            }
            if constexpr (mb == 1) {
#pragma unroll
              for (int p = 0; p < NP; p++) dsb[p] = pack8<CT>(ds[p]);
            }
          }
        } else {
#pragma unroll
          for (int p = 0; p < NP; p++) dq_acc[p][j - N1] = Mma<CT>::mfma(x, dsb[p], dq_acc[p][j - N1]);
        }
      });
    });
  };
  int ci = 0, bi = 0;
  auto buf_of = [&](int i) { return smem + (i >= NBUF ? i - NBUF : i) * B::BUF; };
  if constexpr (CAUSAL) {
    // the chunks below the first query of the workgroup: every wave sees every pair, the body holds no test (as without
    // a mask); the chunks on the diagonal follow with the per-chunk and per-pair tests
    const int nfull = dlt_imin(x0, W.len) / CK;
    for (; ci + AHEAD < W.nchunks && ci < nfull; ci++) {
      consume_t(ci, (Swa2Lds)buf_of(bi), buf_of(bi + AHEAD), std::false_type{}, std::true_type{});
      flashd_wait_copies<(AHEAD - 1) * PER_CHUNK>();
      __syncthreads();
      bi = bi + 1 == NBUF ? 0 : bi + 1;
    }
  }
  for (; ci + AHEAD < W.nchunks; ci++) {
    if (CAUSAL) consume_t(ci, (Swa2Lds)buf_of(bi), buf_of(bi + AHEAD), FlashTailDyn{}, std::true_type{});
    else consume_t(ci, (Swa2Lds)buf_of(bi), buf_of(bi + AHEAD), std::false_type{}, std::true_type{});
    flashd_wait_copies<(AHEAD - 1) * PER_CHUNK>();
    __syncthreads();
    bi = bi + 1 == NBUF ? 0 : bi + 1;
  }
  // without a mask a full last chunk runs here too (same test-free body): the code below, whose per-pair tests cost
  // registers the compiler finds by spilling, is then not executed at all
  const int n_plain = (!CAUSAL && W.nchunks > 0 && !chunk_tail(W.nchunks - 1)) ? W.nchunks : W.nchunks - 1;
  for (; ci < n_plain; ci++) {
    if (CAUSAL) consume_t(ci, (Swa2Lds)buf_of(bi), buf_of(bi + AHEAD), FlashTailDyn{}, std::false_type{});
    else consume_t(ci, (Swa2Lds)buf_of(bi), buf_of(bi + AHEAD), std::false_type{}, std::false_type{});
    swa2_wait_copies();
    __syncthreads();
    bi = bi + 1 == NBUF ? 0 : bi + 1;
  }
  if (ci < W.nchunks) {
    if (CAUSAL) consume_t(ci, (Swa2Lds)buf_of(bi), buf_of(bi + AHEAD), FlashTailDyn{}, std::false_type{});
    else consume_t(ci, (Swa2Lds)buf_of(bi), buf_of(bi + AHEAD), std::true_type{}, std::false_type{});
  }
  __syncthreads();
  TIO* dqb = reinterpret_cast<TIO*>(a.dq) + b * a.dqs[0] + h * a.dqs[1];
  flash_write_grad<TIO, DK, NP>(smem, dq_acc, a.sm_scale, dqb, flash_tok<false>(a.dqs, a.tm), a.dqs[3], a.dk_, a.dq_vec != 0, 0, x0, a.Lq, wave, n, g, tid, OWN);
}
