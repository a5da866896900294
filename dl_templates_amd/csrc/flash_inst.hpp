// Included by flash_inst_<DK>_<DV>.hip with DLT_DK / DLT_DV defined: dense flash kernels for
// one pair of padded head dims.
#include <cstdlib>
#include "flash_dma_kernel.hpp"

#define DLT_FCAT3_(a, b, c) a##b##_##c
#define DLT_FCAT3(a, b, c) DLT_FCAT3_(a, b, c)

namespace {
// shape of the asynchronously staged forward kernel: keys per chunk, waves per workgroup (16 NP queries per wave).
// 8 waves on 128-key chunks at 64/128 and 128/128 (K / V copied once per 256 queries), 4 waves on 64-key chunks at 64/64
// (there the 8-wave shape only ties with the register-staged kernel)
#ifndef FLASHD_FWD_NP
#define FLASHD_FWD_NP FLASH_NP
#endif
#ifndef FLASHD_FWD_CK
#define FLASHD_FWD_CK(dk, dv) ((dk) + (dv) > 128 ? 128 : 64)
#endif
#ifndef FLASHD_FWD_NW
#define FLASHD_FWD_NW(dk, dv) ((dk) + (dv) > 128 ? 8 : 4)
#endif
// query blocks per wave of the asynchronously staged dQ kernel: two in every class (without staging registers two blocks
// fit at 128/128 as well: -18 % there; three blocks measured 8 % slower at 64/64 and 64/128)
#ifndef FLASHD_DQ_NP
#define FLASHD_DQ_NP(dk, dv) 2
#endif
// waves per workgroup of the asynchronously staged backward kernels (64-token chunks)
#ifndef FLASHD_BWD_NW
#define FLASHD_BWD_NW 4
#endif

// DLT_FLASH_SYNC_STAGING=1 keeps the register-staged kernels for every class (A/B timing)
inline bool flash_async_staging() {
  static const bool on = [] { const char* e = std::getenv("DLT_FLASH_SYNC_STAGING"); return !(e != nullptr && e[0] == '1'); }();
  return on;
}

template <typename KernT>
int flash_set_lds(KernT kern, int bytes) { return dlt_ensure_lds(reinterpret_cast<const void*>(kern), bytes); }

template <typename TIO, int MODE>
int flash_launch_fwd_c(const FlashArgs& a, int grid, hipStream_t stream) {
  if constexpr (DLT_DK >= 64 && DLT_DV >= 64 && MODE < 2) {
    // dense / causal, head dims that are multiples of 8: chunks are copied HBM -> LDS asynchronously.  Measured per
    // class and mode against the register-staged kernel: dense -2 % (64/64), -4 % (64/128), -7 % (128/128); causal -4 %
    // (64/64), -18 % (128/128); head dims below the class (80/80, 96/96): -18 % on the step.
    if (a.dk % 8 == 0 && a.dv % 8 == 0 && flash_async_staging()) {
      constexpr int NP = FLASHD_FWD_NP, CK = FLASHD_FWD_CK(DLT_DK, DLT_DV), NW = FLASHD_FWD_NW(DLT_DK, DLT_DV);
      // head dims below the padded ones (multiples of 8): the kernel variant whose copies skip the missing pieces
      auto kern = (a.dk != DLT_DK || a.dv != DLT_DV) ? flashd_fwd_kernel<TIO, DLT_DK, DLT_DV, NP, CK, NW, MODE, true>
                                                     : flashd_fwd_kernel<TIO, DLT_DK, DLT_DV, NP, CK, NW, MODE, false>;
      constexpr int own = 16 * NP * NW;
      constexpr int tile = own * (DLT_DV * 2 + 16);
      constexpr int bufs = (NW == 4 ? flashd_nbuf(DLT_DK, DLT_DV) : 2) * FlashDBuf<DLT_DK, DLT_DV, CK>::BUF;
      constexpr int lds = bufs > tile ? bufs : tile;
      const int rc = flash_set_lds(kern, lds);
      if (rc != DLT_OK) return rc;
      FlashArgs ad = a;
      ad.nblk = (a.Lq + own - 1) / own;
      dlt_timing_before(DLT_K_FWD, stream);
      hipLaunchKernelGGL(kern, dim3(a.B * a.H * ad.nblk), dim3(64 * NW), lds, stream, ad);
      dlt_timing_after(stream);
      DLT_CHECK_LAUNCH("flash forward launch");
      return DLT_OK;
    }
  }
  auto kern = flash_fwd_kernel<TIO, DLT_DK, DLT_DV, FLASH_NP, flash_ck_fwd(DLT_DK, DLT_DV), MODE>;
  {
    const int rc = dlt_ensure_lds(reinterpret_cast<const void*>(kern), a.lds_bytes);
    if (rc != DLT_OK) return rc;
  }
  dlt_timing_before(DLT_K_FWD, stream);
  hipLaunchKernelGGL(kern, dim3(grid), dim3(256), a.lds_bytes, stream, a);
  dlt_timing_after(stream);
  DLT_CHECK_LAUNCH("flash forward launch");
  return DLT_OK;
}

template <typename TIO>
int flash_launch_fwd_t(const FlashArgs& a, int grid, hipStream_t stream) {
  if (a.tile) return a.tm.img ? flash_launch_fwd_c<TIO, 3>(a, grid, stream) : flash_launch_fwd_c<TIO, 2>(a, grid, stream);
  return a.causal ? flash_launch_fwd_c<TIO, 1>(a, grid, stream) : flash_launch_fwd_c<TIO, 0>(a, grid, stream);
}

template <typename TIO, int MODE>
int flash_launch_bwd_c(const FlashBwdArgs& a, int grid_kv, int grid_q, hipStream_t stream) {
  // dQ first: with fuse_delta it produces the delta vector the dK/dV kernel consumes
  bool dq_done = false;
  if constexpr (DLT_DK >= 64 && DLT_DV >= 64 && MODE < 2) {
    if (a.dk_ % 8 == 0 && a.dv_ % 8 == 0 && flash_async_staging()) {
      constexpr int NP = FLASHD_DQ_NP(DLT_DK, DLT_DV), CK = 64, NW = FLASHD_BWD_NW;
      auto kern = (a.dk_ != DLT_DK || a.dv_ != DLT_DV) ? flashd_bwd_q_kernel<TIO, DLT_DK, DLT_DV, NP, CK, NW, MODE, true>
                                                       : flashd_bwd_q_kernel<TIO, DLT_DK, DLT_DV, NP, CK, NW, MODE, false>;
      constexpr int own = 16 * NP * NW;
      constexpr int tile = own * (DLT_DK * 2 + 16);
      constexpr int bufs = (NW == 4 ? flashd_nbuf(DLT_DK, DLT_DV) : FLASHD_NBUF8) * FlashDBuf<DLT_DK, DLT_DV, CK>::BUF;
      constexpr int lds = bufs > tile ? bufs : tile;
      int rc = flash_set_lds(kern, lds);
      if (rc != DLT_OK) return rc;
      FlashBwdArgs ad = a;
      ad.nblk_q = (a.Lq + own - 1) / own;
      dlt_timing_before(DLT_K_BWD_Q, stream);
      hipLaunchKernelGGL(kern, dim3(a.B * a.H * ad.nblk_q), dim3(64 * NW), lds, stream, ad);
      dlt_timing_after(stream);
      DLT_CHECK_LAUNCH("flash dQ launch");
      dq_done = true;
    }
  }
  if (!dq_done) {
    auto kern = flash_bwd_q_kernel<TIO, DLT_DK, DLT_DV, flash_np_q(DLT_DK, DLT_DV), flash_ck_q(DLT_DK, DLT_DV), MODE>;
    int rc = flash_set_lds(kern, a.lds_q);
    if (rc != DLT_OK) return rc;
    dlt_timing_before(DLT_K_BWD_Q, stream);
    hipLaunchKernelGGL(kern, dim3(grid_q), dim3(256), a.lds_q, stream, a);
    dlt_timing_after(stream);
    DLT_CHECK_LAUNCH("flash dQ launch");
  }
  if constexpr (DLT_DK >= 64 && DLT_DV >= 64 && MODE < 2) {
    // dense / causal, head dims that are multiples of 8: chunks are copied HBM -> LDS asynchronously (in tile mode,
    // where whole blocks are skipped, the register-staged kernel measured 1.5 % faster)
    const bool scalars_fit = a.ls[2] >= 0 && ((int64_t)a.Lq - 1) * a.ls[2] * 4 + 4 <= (((int64_t)1 << 31) - 1);   // 32-bit offsets of the lse2 / delta copies
    if (a.dk_ % 8 == 0 && a.dv_ % 8 == 0 && scalars_fit && flash_async_staging()) {
      constexpr int NP = flash_np_kv(DLT_DK, DLT_DV), CK = 64, NW = FLASHD_BWD_NW;
      auto kern = (a.dk_ != DLT_DK || a.dv_ != DLT_DV) ? flashd_bwd_kv_kernel<TIO, DLT_DK, DLT_DV, NP, CK, NW, MODE, true>
                                                       : flashd_bwd_kv_kernel<TIO, DLT_DK, DLT_DV, NP, CK, NW, MODE, false>;
      constexpr int own = 16 * NP * NW;
      constexpr int tile_k = own * (DLT_DK * 2 + 16), tile_v = own * (DLT_DV * 2 + 16);
      constexpr int bufs = (NW == 4 ? flashd_nbuf(DLT_DK, DLT_DV) : FLASHD_NBUF8) * FlashDBuf<DLT_DK, DLT_DV, CK>::BUF_KV;
      constexpr int lds = bufs > tile_v ? (bufs > tile_k ? bufs : tile_k) : (tile_v > tile_k ? tile_v : tile_k);
      int rc = flash_set_lds(kern, lds);
      if (rc != DLT_OK) return rc;
      FlashBwdArgs ad = a;
      ad.nblk_k = (a.Lk + own - 1) / own;
      dlt_timing_before(DLT_K_BWD_KV, stream);
      hipLaunchKernelGGL(kern, dim3(a.B * a.H * ad.nblk_k), dim3(64 * NW), lds, stream, ad);
      dlt_timing_after(stream);
      DLT_CHECK_LAUNCH("flash dK/dV launch");
      return DLT_OK;
    }
  }
  {
    auto kern = flash_bwd_kv_kernel<TIO, DLT_DK, DLT_DV, flash_np_kv(DLT_DK, DLT_DV), flash_ck_kv(DLT_DK, DLT_DV), MODE>;
    int rc = flash_set_lds(kern, a.lds_kv);
    if (rc != DLT_OK) return rc;
    dlt_timing_before(DLT_K_BWD_KV, stream);
    hipLaunchKernelGGL(kern, dim3(grid_kv), dim3(256), a.lds_kv, stream, a);
    dlt_timing_after(stream);
    DLT_CHECK_LAUNCH("flash dK/dV launch");
  }
  return DLT_OK;
}

template <typename TIO>
int flash_launch_bwd_t(const FlashBwdArgs& a, int grid_kv, int grid_q, hipStream_t stream) {
  if (a.tile) return a.tm.img ? flash_launch_bwd_c<TIO, 3>(a, grid_kv, grid_q, stream) : flash_launch_bwd_c<TIO, 2>(a, grid_kv, grid_q, stream);
  return a.causal ? flash_launch_bwd_c<TIO, 1>(a, grid_kv, grid_q, stream) : flash_launch_bwd_c<TIO, 0>(a, grid_kv, grid_q, stream);
}
}  // namespace

int DLT_FCAT3(dlt_flash_launch_bwd_, DLT_DK, DLT_DV)(const FlashBwdArgs& a, int dtype, int grid_kv, int grid_q, hipStream_t stream) {
  return dtype == DLT_BF16 ? flash_launch_bwd_t<bf16_t>(a, grid_kv, grid_q, stream) : flash_launch_bwd_t<f16_t>(a, grid_kv, grid_q, stream);
}

int DLT_FCAT3(dlt_flash_launch_fwd_, DLT_DK, DLT_DV)(const FlashArgs& a, int dtype, int grid, hipStream_t stream) {
  return dtype == DLT_BF16 ? flash_launch_fwd_t<bf16_t>(a, grid, stream) : flash_launch_fwd_t<f16_t>(a, grid, stream);
}
