// Included by attn_inst_<DK>_<DV>.hip with DLT_DK / DLT_DV defined: instantiates the kernels
// for one pair of (padded) head dims and exports their launchers.
#include "attn_fwd_kernel.hpp"
#include "attn_bwd_kernel.hpp"

#define DLT_CAT3_(a, b, c) a##b##_##c
#define DLT_CAT3(a, b, c) DLT_CAT3_(a, b, c)

namespace {
template <typename KernT>
int set_lds_limit(KernT kern, int bytes) { return dlt_ensure_lds(reinterpret_cast<const void*>(kern), bytes); }

template <typename TIO, int NP>
int launch_fwd_t(const FwdArgs& a, int grid, hipStream_t stream) {
  auto kern = attn_fwd_kernel<TIO, DLT_DK, DLT_DV, NP>;
  int rc = set_lds_limit(kern, a.plan.lds_bytes);
  if (rc != DLT_OK) return rc;
  dlt_timing_before(DLT_K_FWD, stream);
  hipLaunchKernelGGL(kern, dim3(grid), dim3(256), a.plan.lds_bytes, stream, a);
  dlt_timing_after(stream);
  DLT_CHECK_LAUNCH("attention forward launch");
  return DLT_OK;
}

template <typename TIO>
int launch_delta_t(const BwdArgs& aq, hipStream_t stream) {
  constexpr int CH = DLT_DV / 8;
  const int64_t threads = (int64_t)aq.p.B * aq.p.H * aq.n_tokens_q * CH;
  dlt_timing_before(DLT_K_DELTA, stream);
  hipLaunchKernelGGL((attn_delta_kernel<TIO, DLT_DV>), dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, stream, aq);
  dlt_timing_after(stream);
  DLT_CHECK_LAUNCH("attention delta launch");
  return DLT_OK;
}

template <typename TIO, int NP>
int launch_bwd_t(const BwdArgs& akv, int grid_kv, const BwdArgs& aq, int grid_q, hipStream_t stream) {
  {
    int rc = launch_delta_t<TIO>(aq, stream);
    if (rc != DLT_OK) return rc;
  }
  {
    auto kern = attn_bwd_kv_kernel<TIO, DLT_DK, DLT_DV, NP>;
    int rc = set_lds_limit(kern, akv.plan.lds_bytes);
    if (rc != DLT_OK) return rc;
    dlt_timing_before(DLT_K_BWD_KV, stream);
    hipLaunchKernelGGL(kern, dim3(grid_kv), dim3(256), akv.plan.lds_bytes, stream, akv);
    dlt_timing_after(stream);
    DLT_CHECK_LAUNCH("attention dK/dV launch");
  }
  {
    auto kern = attn_bwd_q_kernel<TIO, DLT_DK, DLT_DV, NP>;
    int rc = set_lds_limit(kern, aq.plan.lds_bytes);
    if (rc != DLT_OK) return rc;
    dlt_timing_before(DLT_K_BWD_Q, stream);
    hipLaunchKernelGGL(kern, dim3(grid_q), dim3(256), aq.plan.lds_bytes, stream, aq);
    dlt_timing_after(stream);
    DLT_CHECK_LAUNCH("attention dQ launch");
  }
  return DLT_OK;
}
}  // namespace

int DLT_CAT3(dlt_launch_delta_, DLT_DK, DLT_DV)(const BwdArgs& a, hipStream_t stream) {
  switch (a.p.dtype) {
    case DLT_BF16: return launch_delta_t<bf16_t>(a, stream);
    case DLT_FP16: return launch_delta_t<f16_t>(a, stream);
    default: return launch_delta_t<float>(a, stream);
  }
}

#ifdef DLT_ONE_PATCH
// head-dim classes whose accumulators leave no room for two query blocks per wave: np must be 1
int DLT_CAT3(dlt_launch_bwd_, DLT_DK, DLT_DV)(const BwdArgs& akv, int grid_kv, const BwdArgs& aq, int grid_q, int np,
                                              hipStream_t stream) {
  if (np != 1) return dlt_set_error(DLT_ERR_UNSUPPORTED, "attention backward: this head-dim class takes one query block per wave");
  switch (aq.p.dtype) {
    case DLT_BF16: return launch_bwd_t<bf16_t, 1>(akv, grid_kv, aq, grid_q, stream);
    case DLT_FP16: return launch_bwd_t<f16_t, 1>(akv, grid_kv, aq, grid_q, stream);
    default: return launch_bwd_t<float, 1>(akv, grid_kv, aq, grid_q, stream);
  }
}

int DLT_CAT3(dlt_launch_fwd_, DLT_DK, DLT_DV)(const FwdArgs& a, int np, int grid, hipStream_t stream) {
  if (np != 1) return dlt_set_error(DLT_ERR_UNSUPPORTED, "attention forward: this head-dim class takes one query block per wave");
  switch (a.p.dtype) {
    case DLT_BF16: return launch_fwd_t<bf16_t, 1>(a, grid, stream);
    case DLT_FP16: return launch_fwd_t<f16_t, 1>(a, grid, stream);
    default: return launch_fwd_t<float, 1>(a, grid, stream);
  }
}
#else
int DLT_CAT3(dlt_launch_bwd_, DLT_DK, DLT_DV)(const BwdArgs& akv, int grid_kv, const BwdArgs& aq, int grid_q, int np,
                                              hipStream_t stream) {
  switch (aq.p.dtype) {
    case DLT_BF16: return np == 1 ? launch_bwd_t<bf16_t, 1>(akv, grid_kv, aq, grid_q, stream) : launch_bwd_t<bf16_t, 2>(akv, grid_kv, aq, grid_q, stream);
    case DLT_FP16: return np == 1 ? launch_bwd_t<f16_t, 1>(akv, grid_kv, aq, grid_q, stream) : launch_bwd_t<f16_t, 2>(akv, grid_kv, aq, grid_q, stream);
    default: return np == 1 ? launch_bwd_t<float, 1>(akv, grid_kv, aq, grid_q, stream) : launch_bwd_t<float, 2>(akv, grid_kv, aq, grid_q, stream);
  }
}

int DLT_CAT3(dlt_launch_fwd_, DLT_DK, DLT_DV)(const FwdArgs& a, int np, int grid, hipStream_t stream) {
  switch (a.p.dtype) {
    case DLT_BF16: return np == 1 ? launch_fwd_t<bf16_t, 1>(a, grid, stream) : launch_fwd_t<bf16_t, 2>(a, grid, stream);
    case DLT_FP16: return np == 1 ? launch_fwd_t<f16_t, 1>(a, grid, stream) : launch_fwd_t<f16_t, 2>(a, grid, stream);
    default: return np == 1 ? launch_fwd_t<float, 1>(a, grid, stream) : launch_fwd_t<float, 2>(a, grid, stream);
  }
}
#endif
