// Streaming token-grid kernels: instantiations and launchers for one head dim (DLT_SWA2_D), included by one
// translation unit per head dim.
#include "swa2_bwd_kernel.hpp"
#include "swa2s_fwd_kernel.hpp"

#define DLT_SWA2_CAT_(a, b) a##b
#define DLT_SWA2_CAT(a, b) DLT_SWA2_CAT_(a, b)

namespace {
template <typename KernT>
int swa2_set_lds(KernT kern, int bytes) { return dlt_ensure_lds(reinterpret_cast<const void*>(kern), bytes); }

template <typename TIO, int NCG>
int swa2_launch_fwd_t(const Swa2FwdArgs& a, int grid, hipStream_t stream) {
  typedef Swa2Cfg<DLT_SWA2_D, NCG> C;
  auto kern = swa2_fwd_kernel<TIO, DLT_SWA2_D, NCG>;
  if constexpr (DLT_SWA2_D == 128) {
    if (a.plan.band == 16) kern = swa2s_fwd_kernel<TIO, DLT_SWA2_D, NCG>;   // two stacked patches per wave
  } else if (a.plan.band != 8) {
    return dlt_set_error(DLT_ERR_UNSUPPORTED, "streaming token-grid kernels: no instantiation for bands of %d rows", a.plan.band);
  }
  int rc = swa2_set_lds(kern, C::LDS);
  if (rc != DLT_OK) return rc;
  dlt_timing_before(DLT_K_FWD, stream);
  hipLaunchKernelGGL(kern, dim3(grid), dim3(SWA2_THREADS), C::LDS, stream, a);
  dlt_timing_after(stream);
  DLT_CHECK_LAUNCH("token-grid forward launch (streaming kernels)");
  return DLT_OK;
}

template <typename TIO, int NCG>
int swa2_launch_bwd_t(const Swa2BwdArgs& a, int grid, hipStream_t stream) {
  typedef Swa2Cfg<DLT_SWA2_D, NCG> C;
  auto kq = swa2_bwd_q_kernel<TIO, DLT_SWA2_D, NCG>;
  auto kkv = swa2_bwd_kv_kernel<TIO, DLT_SWA2_D, NCG>;
  int rc = swa2_set_lds(kq, C::LDS);
  if (rc != DLT_OK) return rc;
  rc = swa2_set_lds(kkv, C::LDS_KV);
  if (rc != DLT_OK) return rc;
  // dQ first: it publishes delta for the dK/dV kernel
  dlt_timing_before(DLT_K_BWD_Q, stream);
  hipLaunchKernelGGL(kq, dim3(grid), dim3(SWA2_THREADS), C::LDS, stream, a);
  dlt_timing_after(stream);
  DLT_CHECK_LAUNCH("token-grid dQ launch (streaming kernels)");
  dlt_timing_before(DLT_K_BWD_KV, stream);
  hipLaunchKernelGGL(kkv, dim3(grid), dim3(SWA2_THREADS), C::LDS_KV, stream, a);
  dlt_timing_after(stream);
  DLT_CHECK_LAUNCH("token-grid dK/dV launch (streaming kernels)");
  return DLT_OK;
}
// ncg: column groups of a wave's window, 4 (windows up to 13 columns) or 6 (up to 21); any other value has no
// instantiation and is rejected
template <typename TIO>
int swa2_pick_fwd(const Swa2FwdArgs& a, int ncg, int grid, hipStream_t stream) {
  switch (ncg) {
    case 4: return swa2_launch_fwd_t<TIO, 4>(a, grid, stream);
    case 6: return swa2_launch_fwd_t<TIO, 6>(a, grid, stream);
    default: return dlt_set_error(DLT_ERR_UNSUPPORTED, "streaming token-grid kernels: no instantiation for %d column groups", ncg);
  }
}
template <typename TIO>
int swa2_pick_bwd(const Swa2BwdArgs& a, int ncg, int grid, hipStream_t stream) {
  switch (ncg) {
    case 4: return swa2_launch_bwd_t<TIO, 4>(a, grid, stream);
    case 6: return swa2_launch_bwd_t<TIO, 6>(a, grid, stream);
    default: return dlt_set_error(DLT_ERR_UNSUPPORTED, "streaming token-grid kernels: no instantiation for %d column groups", ncg);
  }
}
}  // namespace

int DLT_SWA2_CAT(dlt_swa2_launch_fwd_, DLT_SWA2_D)(const Swa2FwdArgs& a, int ncg, int grid, hipStream_t stream) {
  return a.p.dtype == DLT_BF16 ? swa2_pick_fwd<bf16_t>(a, ncg, grid, stream) : swa2_pick_fwd<f16_t>(a, ncg, grid, stream);
}
int DLT_SWA2_CAT(dlt_swa2_launch_bwd_, DLT_SWA2_D)(const Swa2BwdArgs& a, int ncg, int grid, hipStream_t stream) {
  return a.p.dtype == DLT_BF16 ? swa2_pick_bwd<bf16_t>(a, ncg, grid, stream) : swa2_pick_bwd<f16_t>(a, ncg, grid, stream);
}
