// Internal declarations shared by the translation units of libdlt_hip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/dlt.h"
#include "dlt_geom.h"

// ---- error reporting ---------------------------------------------------------------
int dlt_set_error(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
// Raises a kernel's limit of dynamic LDS to `bytes` on the current device.  The runtime call is made only when a larger
// size than any before is asked for (per kernel and device): it costs tens of microseconds of host time, which would
// otherwise sit in front of every launch.
int dlt_ensure_lds(const void* kern, int bytes);
// Routing record of the calling thread: every attention launch path notes its kernel family (DLT_FAMILY_*) here first.
// Returns true under dlt_dry_run(1): the caller then returns DLT_OK without launching anything.
bool dlt_route_note(int family);
bool dlt_route_dry();
void dlt_route_reset();
// compute units of the current device (asked once per device; 256 when the query fails)
int dlt_device_cus();

#define DLT_REQUIRE(cond, ...)                                   \
  do {                                                           \
    if (!(cond)) return dlt_set_error(DLT_ERR_INVALID, __VA_ARGS__); \
  } while (0)

#define DLT_CHECK_LAUNCH(what)                                                              \
  do {                                                                                      \
    hipError_t e__ = hipGetLastError();                                                     \
    if (e__ != hipSuccess)                                                                  \
      return dlt_set_error(DLT_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e__));         \
  } while (0)

// per-kernel timing hooks (no-ops unless dlt_timing_enable(1) was called on this thread)
void dlt_timing_before(int kernel_id, hipStream_t stream);
void dlt_timing_after(hipStream_t stream);

static inline int dlt_elem_size(int dtype) { return dtype == DLT_FP32 ? 4 : 2; }

// ---- rotary operands as the kernels see them ------------------------------------------
struct RopeDev {
  const int32_t* idx;
  const float* row_cs;
  const float* col_cs;
  int64_t rs0, cs0;
  int32_t R, row_len, col_len;
  int32_t inverse;
  int32_t enabled;
};

int dlt_validate_rope(const dlt_rope_t* rope, int64_t n_dim);
RopeDev dlt_make_rope_dev(const dlt_rope_t* rope, int inverse);
// in-place rotation of a [B, H, N, C] tensor with any strides (the standalone kernels)
int dlt_rope_inplace_4d(void* x, const int64_t* st, int B, int H, int64_t N, int C, const dlt_rope_t* rope, int inverse,
                        int dtype, hipStream_t stream);
// dst = rotate(src) for [B, H, N, C] tensors with any strides (every element is copied)
int dlt_rope_rotate_copy(const void* src, const int64_t* ss, void* dst, const int64_t* ds, int B, int H, int64_t N, int C,
                         const RopeDev& rope, int dtype, hipStream_t stream);

// ---- attention core (attn_fwd.hip / attn_bwd.hip) -------------------------------------
struct AttnTensors {
  const void *q, *k, *v, *o, *d_o;
  void *out_o, *dq, *dk, *dv;
  void *q_rot, *k_rot;  // forward: optional outputs, the rotated q and k (NULL: not wanted)
  float* lse;        // written by forward, read by backward
  float* delta;      // scratch written by the backward pre-pass
  // element strides [B, H, N, D]; entry 4 is only used with an image token map (AttnProblem::tm):
  // then [2] is the stride of a pixel column and [4] the stride of a pixel row
  int64_t qs[5], ks[5], vs[5], os[5], dos[5], dqs[5], dks[5], dvs[5], ls[3];
  int64_t qrs[5], krs[5];
};

struct AttnProblem {
  DltGeom g;
  int32_t B, H, dk, dv;
  float sm_scale;
  int32_t dtype;
  RopeDev rope;
  int32_t rope_prerot;  // backward: q and k arrive rotated; only dq and dk are rotated (back) on store
  DltTokMap tm;  // token -> element offset map of q, k, v, o and the gradients (lse2 / delta stay [B, H, N])
};

int dlt_attn_forward(const AttnProblem& p, const AttnTensors& t, hipStream_t stream);
int dlt_attn_backward(const AttnProblem& p, const AttnTensors& t, hipStream_t stream);
