// Streaming token-grid kernels for head dim 128: instantiations and launchers.
#include "swa2_bwd_kernel.hpp"

namespace {
template <typename KernT>
int swa2_set_lds(KernT kern, int bytes) { return dlt_ensure_lds(reinterpret_cast<const void*>(kern), bytes); }

template <typename TIO>
int swa2_launch_fwd_t(const Swa2FwdArgs& a, int grid, hipStream_t stream) {
  auto kern = swa2_fwd_kernel<TIO>;
  int rc = swa2_set_lds(kern, SWA2_LDS);
  if (rc != DLT_OK) return rc;
  dlt_timing_before(DLT_K_FWD, stream);
  hipLaunchKernelGGL(kern, dim3(grid), dim3(SWA2_THREADS), SWA2_LDS, stream, a);
  dlt_timing_after(stream);
  DLT_CHECK_LAUNCH("token-grid forward launch (head dim 128)");
  return DLT_OK;
}

template <typename TIO>
int swa2_launch_bwd_t(const Swa2BwdArgs& a, int grid, hipStream_t stream) {
  auto kq = swa2_bwd_q_kernel<TIO>;
  auto kkv = swa2_bwd_kv_kernel<TIO>;
  int rc = swa2_set_lds(kq, SWA2_LDS);
  if (rc != DLT_OK) return rc;
  rc = swa2_set_lds(kkv, SWA2_LDS_KV);
  if (rc != DLT_OK) return rc;
  // dQ first: it publishes delta for the dK/dV kernel
  dlt_timing_before(DLT_K_BWD_Q, stream);
  hipLaunchKernelGGL(kq, dim3(grid), dim3(SWA2_THREADS), SWA2_LDS, stream, a);
  dlt_timing_after(stream);
  DLT_CHECK_LAUNCH("token-grid dQ launch (head dim 128)");
  dlt_timing_before(DLT_K_BWD_KV, stream);
  hipLaunchKernelGGL(kkv, dim3(grid), dim3(SWA2_THREADS), SWA2_LDS_KV, stream, a);
  dlt_timing_after(stream);
  DLT_CHECK_LAUNCH("token-grid dK/dV launch (head dim 128)");
  return DLT_OK;
}
}  // namespace

int dlt_swa2_launch_fwd(const Swa2FwdArgs& a, int grid, hipStream_t stream) {
  return a.p.dtype == DLT_BF16 ? swa2_launch_fwd_t<bf16_t>(a, grid, stream) : swa2_launch_fwd_t<f16_t>(a, grid, stream);
}


int dlt_swa2_launch_bwd(const Swa2BwdArgs& a, int grid, hipStream_t stream) {
  return a.p.dtype == DLT_BF16 ? swa2_launch_bwd_t<bf16_t>(a, grid, stream) : swa2_launch_bwd_t<f16_t>(a, grid, stream);
}
