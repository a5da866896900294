// Marching token-grid kernels (head dim 64): instantiations and launchers.
#include "swam_bwd_kernel.hpp"

namespace {
template <typename KernT>
int swam_set_lds(KernT kern, int bytes) { return dlt_ensure_lds(reinterpret_cast<const void*>(kern), bytes); }

template <typename TIO, int ROPE, bool TL>
int swam_launch_fwd_r(const SwamFwdArgs& a, int grid, hipStream_t stream) {
  auto kern = swam_fwd_kernel<TIO, ROPE, TL>;
  const int lds = swam_ring(64) + (TL ? SWAM_TAB_BYTES : 0);
  int rc = swam_set_lds(kern, lds);
  if (rc != DLT_OK) return rc;
  dlt_timing_before(DLT_K_FWD, stream);
  hipLaunchKernelGGL(kern, dim3(grid), dim3(SWAM_THREADS), lds, stream, a);
  dlt_timing_after(stream);
  DLT_CHECK_LAUNCH("marching token-grid forward launch");
  return DLT_OK;
}

template <typename TIO, int ROPE, bool TL>
int swam_launch_bwd_r(const SwamBwdArgs& a, int grid, hipStream_t stream) {
  // dQ first: it produces the delta vector the dK/dV kernel consumes
  {
    auto kern = swam_bwd_q_kernel<TIO, ROPE, TL>;
    const int lds = swam_ring(64) + (TL ? SWAM_TAB_BYTES : 0);
    int rc = swam_set_lds(kern, lds);
    if (rc != DLT_OK) return rc;
    dlt_timing_before(DLT_K_BWD_Q, stream);
    hipLaunchKernelGGL(kern, dim3(grid), dim3(SWAM_THREADS), lds, stream, a);
    dlt_timing_after(stream);
    DLT_CHECK_LAUNCH("marching token-grid dQ launch");
  }
  {
    auto kern = swam_bwd_kv_kernel<TIO, ROPE, TL>;
    const int lds = swam_ring(64) + 2 * SWAM_NSLOT * SWAM_TOK * 4 + (TL ? SWAM_TAB_BYTES : 0);
    int rc = swam_set_lds(kern, lds);
    if (rc != DLT_OK) return rc;
    dlt_timing_before(DLT_K_BWD_KV, stream);
    hipLaunchKernelGGL(kern, dim3(grid), dim3(SWAM_THREADS), lds, stream, a);
    dlt_timing_after(stream);
    DLT_CHECK_LAUNCH("marching token-grid dK/dV launch");
  }
  return DLT_OK;
}

// the rotary tables fit the LDS copy (both tables: 64 bytes per position)
bool swam_tabs_fit(const RopeDev& rope) { return (rope.row_len + rope.col_len) * 64 <= SWAM_TAB_BYTES; }

template <typename TIO>
int swam_pick_bwd(const SwamBwdArgs& a, int rope, int grid, hipStream_t stream) {
  if (!rope) return swam_launch_bwd_r<TIO, 0, false>(a, grid, stream);
  return swam_tabs_fit(a.p.rope) ? swam_launch_bwd_r<TIO, 3, true>(a, grid, stream) : swam_launch_bwd_r<TIO, 3, false>(a, grid, stream);
}
template <typename TIO>
int swam_pick_fwd(const SwamFwdArgs& a, int rope, int grid, hipStream_t stream) {
  if (!rope) return swam_launch_fwd_r<TIO, 0, false>(a, grid, stream);
  return swam_tabs_fit(a.p.rope) ? swam_launch_fwd_r<TIO, 2, true>(a, grid, stream) : swam_launch_fwd_r<TIO, 2, false>(a, grid, stream);
}
}  // namespace

// rope: gradients of rotated q, k are rotated back as they are stored
int dlt_swam_launch_bwd(const SwamBwdArgs& a, int rope, int grid, hipStream_t stream) {
  return a.p.dtype == DLT_BF16 ? swam_pick_bwd<bf16_t>(a, rope, grid, stream) : swam_pick_bwd<f16_t>(a, rope, grid, stream);
}

int dlt_swam_launch_fwd(const SwamFwdArgs& a, int rope, int grid, hipStream_t stream) {
  return a.p.dtype == DLT_BF16 ? swam_pick_fwd<bf16_t>(a, rope, grid, stream) : swam_pick_fwd<f16_t>(a, rope, grid, stream);
}
