// Included by swa1_inst_<D>.hip with DLT_D defined: token-grid kernels for one head-dim class.
#include "swa1_fwd_kernel.hpp"
#include "swa1_bwd_kernel.hpp"

#define DLT_CAT2_(a, b) a##b
#define DLT_CAT2(a, b) DLT_CAT2_(a, b)

namespace {
template <typename KernT>
int swa1_set_lds(KernT kern, int bytes) { return dlt_ensure_lds(reinterpret_cast<const void*>(kern), bytes); }

template <typename TIO, int NCGMAX, int ROPE>
int swa1_launch_fwd_r(const Swa1FwdArgs& a, int grid, hipStream_t stream) {
  auto kern = swa1_fwd_kernel<TIO, DLT_D, NCGMAX, SWA1_FWD_CR, ROPE>;
  int rc = swa1_set_lds(kern, a.plan.lds_bytes);
  if (rc != DLT_OK) return rc;
  dlt_timing_before(DLT_K_FWD, stream);
  hipLaunchKernelGGL(kern, dim3(grid), dim3(256), a.plan.lds_bytes, stream, a);
  dlt_timing_after(stream);
  DLT_CHECK_LAUNCH("token-grid attention forward launch");
  return DLT_OK;
}

// rotation mode -> kernel variant (the rotation code is compiled out of the plain kernels)
template <typename TIO, int NCGMAX>
int swa1_launch_fwd_t(const Swa1FwdArgs& a, int grid, hipStream_t stream) {
  switch (a.rope_mode) {
    case 0: return swa1_launch_fwd_r<TIO, NCGMAX, 0>(a, grid, stream);
    case 1: return swa1_launch_fwd_r<TIO, NCGMAX, 1>(a, grid, stream);
    default: return swa1_launch_fwd_r<TIO, NCGMAX, 2>(a, grid, stream);
  }
}

template <typename TIO, int NCGMAX, int ROPE>
int swa1_launch_bwd_r(const Swa1BwdArgs& a, int grid, int lds_kv, int lds_q, hipStream_t stream) {
  // dQ first: with fuse_delta it produces the delta vector the dK/dV kernel consumes
  {
    auto kern = swa1_bwd_q_kernel<TIO, DLT_D, NCGMAX, SWA1_FWD_CR, ROPE>;
    int rc = swa1_set_lds(kern, lds_q);
    if (rc != DLT_OK) return rc;
    dlt_timing_before(DLT_K_BWD_Q, stream);
    hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds_q, stream, a);
    dlt_timing_after(stream);
    DLT_CHECK_LAUNCH("token-grid attention dQ launch");
  }
  {
    auto kern = swa1_bwd_kv_kernel<TIO, DLT_D, NCGMAX, SWA1_KV_CR, ROPE>;
    int rc = swa1_set_lds(kern, lds_kv);
    if (rc != DLT_OK) return rc;
    dlt_timing_before(DLT_K_BWD_KV, stream);
    hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds_kv, stream, a);
    dlt_timing_after(stream);
    DLT_CHECK_LAUNCH("token-grid attention dK/dV launch");
  }
  return DLT_OK;
}

template <typename TIO, int NCGMAX>
int swa1_launch_bwd_t(const Swa1BwdArgs& a, int grid, int lds_kv, int lds_q, hipStream_t stream) {
  switch (a.rope_mode) {
    case 0: return swa1_launch_bwd_r<TIO, NCGMAX, 0>(a, grid, lds_kv, lds_q, stream);
    case 1: return swa1_launch_bwd_r<TIO, NCGMAX, 1>(a, grid, lds_kv, lds_q, stream);
    case 2: return swa1_launch_bwd_r<TIO, NCGMAX, 2>(a, grid, lds_kv, lds_q, stream);
    default: return swa1_launch_bwd_r<TIO, NCGMAX, 3>(a, grid, lds_kv, lds_q, stream);  // rotated inputs, gradients rotated back on store
  }
}
}  // namespace

int DLT_CAT2(dlt_swa1_launch_bwd_, DLT_D)(const Swa1BwdArgs& a, int wclass, int grid, int lds_kv, int lds_q, hipStream_t stream) {
  if (a.p.dtype == DLT_BF16)
    return wclass == 0 ? swa1_launch_bwd_t<bf16_t, 4>(a, grid, lds_kv, lds_q, stream) : swa1_launch_bwd_t<bf16_t, 6>(a, grid, lds_kv, lds_q, stream);
  return wclass == 0 ? swa1_launch_bwd_t<f16_t, 4>(a, grid, lds_kv, lds_q, stream) : swa1_launch_bwd_t<f16_t, 6>(a, grid, lds_kv, lds_q, stream);
}

// window class 0: up to 4 column groups per wave window (WC <= 6); class 1: up to 6 (WC <= 10)
int DLT_CAT2(dlt_swa1_launch_fwd_, DLT_D)(const Swa1FwdArgs& a, int wclass, int grid, hipStream_t stream) {
  if (a.p.dtype == DLT_BF16)
    return wclass == 0 ? swa1_launch_fwd_t<bf16_t, 4>(a, grid, stream) : swa1_launch_fwd_t<bf16_t, 6>(a, grid, stream);
  return wclass == 0 ? swa1_launch_fwd_t<f16_t, 4>(a, grid, stream) : swa1_launch_fwd_t<f16_t, 6>(a, grid, stream);
}
