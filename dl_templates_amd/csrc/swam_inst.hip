// Marching token-grid kernels (head dim 64): instantiations and launchers.
#include "swam_bwd_kernel.hpp"

namespace {
template <typename KernT>
int swam_set_lds(KernT kern, int bytes) { return dlt_ensure_lds(reinterpret_cast<const void*>(kern), bytes); }

template <typename TIO, int ROPE>
int swam_launch_fwd_r(const SwamFwdArgs& a, int grid, hipStream_t stream) {
  auto kern = swam_fwd_kernel<TIO, ROPE>;
  const int lds = swam_ring(64);
  int rc = swam_set_lds(kern, lds);
  if (rc != DLT_OK) return rc;
  dlt_timing_before(DLT_K_FWD, stream);
  hipLaunchKernelGGL(kern, dim3(grid), dim3(SWAM_THREADS), lds, stream, a);
  dlt_timing_after(stream);
  DLT_CHECK_LAUNCH("marching token-grid forward launch");
  return DLT_OK;
}

template <typename TIO, int ROPE>
int swam_launch_bwd_r(const SwamBwdArgs& a, int grid, hipStream_t stream) {
  // dQ first: it produces the delta vector the dK/dV kernel consumes
  {
    auto kern = swam_bwd_q_kernel<TIO, ROPE>;
    const int lds = swam_ring(64);
    int rc = swam_set_lds(kern, lds);
    if (rc != DLT_OK) return rc;
    dlt_timing_before(DLT_K_BWD_Q, stream);
    hipLaunchKernelGGL(kern, dim3(grid), dim3(SWAM_THREADS), lds, stream, a);
    dlt_timing_after(stream);
    DLT_CHECK_LAUNCH("marching token-grid dQ launch");
  }
  {
    auto kern = swam_bwd_kv_kernel<TIO, ROPE>;
    const int lds = swam_ring(64) + 2 * SWAM_NSLOT * SWAM_TOK * 4;
    int rc = swam_set_lds(kern, lds);
    if (rc != DLT_OK) return rc;
    dlt_timing_before(DLT_K_BWD_KV, stream);
    hipLaunchKernelGGL(kern, dim3(grid), dim3(SWAM_THREADS), lds, stream, a);
    dlt_timing_after(stream);
    DLT_CHECK_LAUNCH("marching token-grid dK/dV launch");
  }
  return DLT_OK;
}
}  // namespace

// rope: gradients of rotated q, k are rotated back as they are stored
int dlt_swam_launch_bwd(const SwamBwdArgs& a, int rope, int grid, hipStream_t stream) {
  if (a.p.dtype == DLT_BF16)
    return rope ? swam_launch_bwd_r<bf16_t, 3>(a, grid, stream) : swam_launch_bwd_r<bf16_t, 0>(a, grid, stream);
  return rope ? swam_launch_bwd_r<f16_t, 3>(a, grid, stream) : swam_launch_bwd_r<f16_t, 0>(a, grid, stream);
}

int dlt_swam_launch_fwd(const SwamFwdArgs& a, int rope, int grid, hipStream_t stream) {
  if (a.p.dtype == DLT_BF16)
    return rope ? swam_launch_fwd_r<bf16_t, 2>(a, grid, stream) : swam_launch_fwd_r<bf16_t, 0>(a, grid, stream);
  return rope ? swam_launch_fwd_r<f16_t, 2>(a, grid, stream) : swam_launch_fwd_r<f16_t, 0>(a, grid, stream);
}
