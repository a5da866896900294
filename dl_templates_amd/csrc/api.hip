// extern "C" surface of libdlt_hip.so: argument validation and translation of the
// reference's call signatures into the attention-core problem description.
#include "dlt_internal.hpp"
#include <string.h>
#include <cmath>

static thread_local char g_err[512] = "";

int dlt_set_error(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

// ---- per-kernel timing ------------------------------------------------------------------
#include <vector>
#include <mutex>
namespace {
struct TimedLaunch { int kernel; hipEvent_t e0, e1; };
thread_local bool g_timing = false;
thread_local std::vector<TimedLaunch> g_launches;
thread_local std::vector<hipEvent_t> g_event_pool;

hipEvent_t take_event() {
  if (!g_event_pool.empty()) {
    hipEvent_t e = g_event_pool.back();
    g_event_pool.pop_back();
    return e;
  }
  hipEvent_t e = nullptr;
  if (hipEventCreate(&e) != hipSuccess) return nullptr;
  return e;
}
}  // namespace

void dlt_timing_before(int kernel_id, hipStream_t stream) {
  if (!g_timing) return;
  TimedLaunch t{kernel_id, take_event(), take_event()};
  if (t.e0 == nullptr || t.e1 == nullptr) return;
  (void)hipEventRecord(t.e0, stream);
  g_launches.push_back(t);
}

void dlt_timing_after(hipStream_t stream) {
  if (!g_timing || g_launches.empty()) return;
  (void)hipEventRecord(g_launches.back().e1, stream);
}

extern "C" int dlt_timing_enable(int on) {
  g_timing = on != 0;
  return DLT_OK;
}

extern "C" int dlt_timing_collect(dlt_kernel_time_t* out, int max, int* n) {
  DLT_REQUIRE(n != nullptr, "timing_collect: n is NULL");
  DLT_REQUIRE(out != nullptr || max == 0, "timing_collect: out is NULL");
  *n = (int)g_launches.size();
  int i = 0;
  for (const TimedLaunch& t : g_launches) {
    float ms = 0.f;
    hipError_t e = hipEventSynchronize(t.e1);
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, t.e0, t.e1);
    if (e != hipSuccess) {
      g_launches.clear();
      return dlt_set_error(DLT_ERR_LAUNCH, "timing_collect: %s", hipGetErrorString(e));
    }
    if (i < max) { out[i].kernel = t.kernel; out[i].ms = ms; }
    i++;
    g_event_pool.push_back(t.e0);
    g_event_pool.push_back(t.e1);
  }
  g_launches.clear();
  return DLT_OK;
}

extern "C" const char* dlt_last_error(void) { return g_err; }
extern "C" int dlt_version(void) { return 1; }

namespace {

__global__ void swa_neighbors_kernel(DltGeom g, uint8_t* mask) {
  // one thread per (query tile, kv tile): the same dlt_key_range the attention kernels call
  const int T = g.TR * g.TC;
  const int64_t id = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (id >= (int64_t)T * T) return;
  const int qi = (int)(id / T), kj = (int)(id - (int64_t)qi * T);
  const int qr = qi / g.TC, qc = qi - qr * g.TC;
  const int kr = kj / g.TC, kc = kj - kr * g.TC;
  int rlo, rhi, xlo, xhi;
  dlt_key_range(g, qr, qc * g.S, rlo, rhi, xlo, xhi);
  const int kx = kc * g.S;
  mask[id] = (uint8_t)((kr >= rlo && kr <= rhi && kx >= xlo && kx < xhi) ? 1 : 0);
}

__global__ void swa_image_offsets_kernel(DltTokMap tm, int64_t sy, int64_t sx, int64_t n_tokens, int64_t* out) {
  // one thread per token: the same dlt_token_pixel the attention kernels address image tensors with
  const int64_t n = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (n >= n_tokens) return;
  uint32_t y, x;
  dlt_token_pixel(tm, (uint32_t)n, y, x);
  out[n] = (int64_t)y * sy + (int64_t)x * sx;
}

bool is_dtype(int d) { return d == DLT_BF16 || d == DLT_FP16 || d == DLT_FP32; }

int check_ptrs(const char* who, const void* const* ptrs, const int64_t* const* strides, int n) {
  for (int i = 0; i < n; i++) {
    DLT_REQUIRE(ptrs[i] != nullptr, "%s: tensor argument %d is NULL", who, i);
    DLT_REQUIRE(strides[i] != nullptr, "%s: stride argument %d is NULL", who, i);
  }
  return DLT_OK;
}

int swa_problem(const char* who, const dlt_swa_shape_t* s, const dlt_rope_t* rope, AttnProblem& p) {
  DLT_REQUIRE(s != nullptr, "%s: shape is NULL", who);
  DLT_REQUIRE(is_dtype(s->dtype), "%s: bad dtype %d", who, s->dtype);
  DLT_REQUIRE(s->B > 0 && s->H > 0, "%s: B=%d H=%d must be positive", who, s->B, s->H);
  DLT_REQUIRE(s->b_size > 0 && s->t_height > 0 && s->t_width > 0, "%s: b_size=%d t_height=%d t_width=%d must be positive",
              who, s->b_size, s->t_height, s->t_width);
  DLT_REQUIRE(s->row_size >= 0 && s->col_size >= 0, "%s: negative window (%d, %d)", who, s->row_size, s->col_size);
  DLT_REQUIRE(s->dk > 0 && s->dv > 0, "%s: dk=%d dv=%d must be positive", who, s->dk, s->dv);
  DLT_REQUIRE((int64_t)s->t_height * s->t_width * s->b_size <= 0x3fffffff, "%s: too many tokens", who);
  DLT_REQUIRE(std::isfinite(s->sm_scale), "%s: sm_scale is not finite", who);
  p.g.mode = DLT_GEOM_SWA;
  p.g.TR = s->t_height;
  p.g.TC = s->t_width;
  p.g.S = s->b_size;
  p.g.XLq = p.g.XLk = s->t_width * s->b_size;
  p.g.WR = dlt_imin(s->row_size, s->t_height);
  p.g.WC = dlt_imin(s->col_size, s->t_width);
  p.B = s->B; p.H = s->H; p.dk = s->dk; p.dv = s->dv; p.sm_scale = s->sm_scale; p.dtype = s->dtype;
  if (rope != nullptr) {
    int rc = dlt_validate_rope(rope, s->dk);
    if (rc != DLT_OK) return rc;
  }
  p.rope = dlt_make_rope_dev(rope, 0);
  p.rope_prerot = 0;
  p.tm = dlt_tokmap_none();
  return DLT_OK;
}

int flash_problem(const char* who, const dlt_flash_shape_t* s, AttnProblem& p) {
  DLT_REQUIRE(s != nullptr, "%s: shape is NULL", who);
  DLT_REQUIRE(is_dtype(s->dtype), "%s: bad dtype %d", who, s->dtype);
  DLT_REQUIRE(s->B > 0 && s->H > 0 && s->Lq > 0 && s->Lk > 0, "%s: B=%d H=%d Lq=%d Lk=%d must be positive", who, s->B, s->H, s->Lq, s->Lk);
  DLT_REQUIRE(s->dk > 0 && s->dv > 0, "%s: dk=%d dv=%d must be positive", who, s->dk, s->dv);
  DLT_REQUIRE(!s->causal || s->Lq == s->Lk, "%s: causal attention needs Lq == Lk (got %d, %d)", who, s->Lq, s->Lk);
  DLT_REQUIRE(std::isfinite(s->sm_scale), "%s: sm_scale is not finite", who);
  p.g.mode = s->causal ? DLT_GEOM_CAUSAL : DLT_GEOM_DENSE;
  p.g.TR = 1; p.g.TC = 1; p.g.S = 1; p.g.WR = 0; p.g.WC = 0;
  p.g.XLq = s->Lq; p.g.XLk = s->Lk;
  p.B = s->B; p.H = s->H; p.dk = s->dk; p.dv = s->dv; p.sm_scale = s->sm_scale; p.dtype = s->dtype;
  p.rope = dlt_make_rope_dev(nullptr, 0);
  p.rope_prerot = 0;
  p.tm = dlt_tokmap_none();
  return DLT_OK;
}

void cp4(int64_t* d, const int64_t* s) { for (int i = 0; i < 4; i++) d[i] = s[i]; }
void cp3(int64_t* d, const int64_t* s) { for (int i = 0; i < 3; i++) d[i] = s[i]; }

int fill_fwd(const char* who, AttnTensors& t, const void* q, const int64_t* qs, const void* k, const int64_t* ks,
             const void* v, const int64_t* vs, void* o, const int64_t* os, float* lse, const int64_t* ls) {
  const void* const ptrs[] = {q, k, v, o, lse};
  const int64_t* const st[] = {qs, ks, vs, os, ls};
  int rc = check_ptrs(who, ptrs, st, 5);
  if (rc != DLT_OK) return rc;
  memset(&t, 0, sizeof(t));
  t.q = q; t.k = k; t.v = v; t.out_o = o; t.lse = lse;
  cp4(t.qs, qs); cp4(t.ks, ks); cp4(t.vs, vs); cp4(t.os, os); cp3(t.ls, ls);
  return DLT_OK;
}

int fill_bwd(const char* who, AttnTensors& t, const void* q, const int64_t* qs, const void* k, const int64_t* ks,
             const void* v, const int64_t* vs, const void* o, const int64_t* os, const void* d_o, const int64_t* dos,
             const float* lse, float* delta, const int64_t* ls, void* dq, const int64_t* dqs, void* dk,
             const int64_t* dks, void* dv, const int64_t* dvs) {
  const void* const ptrs[] = {q, k, v, o, d_o, lse, delta, dq, dk, dv};
  const int64_t* const st[] = {qs, ks, vs, os, dos, ls, ls, dqs, dks, dvs};
  int rc = check_ptrs(who, ptrs, st, 10);
  if (rc != DLT_OK) return rc;
  memset(&t, 0, sizeof(t));
  t.q = q; t.k = k; t.v = v; t.o = o; t.d_o = d_o; t.lse = const_cast<float*>(lse); t.delta = delta;
  t.dq = dq; t.dk = dk; t.dv = dv;
  cp4(t.qs, qs); cp4(t.ks, ks); cp4(t.vs, vs); cp4(t.os, os); cp4(t.dos, dos);
  cp4(t.dqs, dqs); cp4(t.dks, dks); cp4(t.dvs, dvs); cp3(t.ls, ls);
  return DLT_OK;
}

// ---- image layout: [B, IH, IW, heads, D] strides -> internal [B, heads, pixel x, D, pixel y] -------
int image_tile(const char* who, const dlt_swa_shape_t* s, const dlt_swa_tile_t* tile) {
  DLT_REQUIRE(s != nullptr && tile != nullptr, "%s: shape / tile is NULL", who);
  DLT_REQUIRE(tile->bh > 0 && tile->bw > 0, "%s: tile of %d x %d pixels", who, tile->bh, tile->bw);
  DLT_REQUIRE((int64_t)tile->bh * tile->bw == s->b_size, "%s: b_size=%d is not the tile of %d x %d pixels", who,
              s->b_size, tile->bh, tile->bw);
  return DLT_OK;
}

int image_strides(const char* who, int which, const int64_t* in, int64_t* out) {
  DLT_REQUIRE(in != nullptr, "%s: stride argument %d is NULL", who, which);
  for (int i = 0; i < 5; i++) DLT_REQUIRE(in[i] >= 0, "%s: image tensor %d has a negative stride", who, which);
  out[0] = in[0]; out[1] = in[3]; out[2] = in[2]; out[3] = in[4]; out[4] = in[1];
  return DLT_OK;
}

// Every tensor of a call whose pixel rows are TC * bw pixel columns apart with single-pixel tiles is
// a plain [B, H, N, D] view: the token map is dropped and every kernel family stays available.
void image_finish(AttnProblem& p, const dlt_swa_tile_t* tile, int64_t* const* st, int n) {
  bool linear = tile->bh == 1 && tile->bw == 1;
  for (int i = 0; i < n && linear; i++) linear = st[i][4] == (int64_t)p.g.TC * st[i][2];
  if (linear) {
    for (int i = 0; i < n; i++) st[i][4] = 0;
    return;
  }
  p.tm = dlt_tokmap_image((uint32_t)tile->bh, (uint32_t)tile->bw, (uint32_t)p.g.TC);
}

}  // namespace

namespace {
__global__ __launch_bounds__(256) void debug_copy_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst, int64_t n) {
  int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (; i < n; i += stride) dst[i] = src[i];
}

}  // namespace

extern "C" int dlt_debug_copy(void* dst, const void* src, int64_t bytes, void* stream) {
  DLT_REQUIRE(bytes >= 0 && bytes % 16 == 0, "debug_copy: size must be a multiple of 16");
  DLT_REQUIRE(((uintptr_t)dst | (uintptr_t)src) % 16 == 0, "debug_copy: pointers must be 16-byte aligned");
  if (bytes == 0) return DLT_OK;
  DLT_REQUIRE(dst != nullptr && src != nullptr, "debug_copy: NULL pointer");
  const int64_t n = bytes / 16;
  int64_t blocks = (n + 255) / 256;
  if (blocks > 256 * 32) blocks = 256 * 32;
  hipLaunchKernelGGL(debug_copy_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                     reinterpret_cast<const uint4*>(src), reinterpret_cast<uint4*>(dst), n);
  DLT_CHECK_LAUNCH("debug_copy launch");
  return DLT_OK;
}

extern "C" int dlt_swa_neighbors(int32_t t_height, int32_t t_width, int32_t row_size, int32_t col_size,
                                 uint8_t* mask, void* stream) {
  DLT_REQUIRE(t_height > 0 && t_width > 0 && row_size >= 0 && col_size >= 0, "swa_neighbors: bad grid/window");
  DLT_REQUIRE(mask != nullptr, "swa_neighbors: mask is NULL");
  const int64_t T = (int64_t)t_height * t_width;
  DLT_REQUIRE(T * T <= ((int64_t)1 << 36), "swa_neighbors: grid too large for a dense mask");
  DltGeom g;
  g.mode = DLT_GEOM_SWA; g.TR = t_height; g.TC = t_width; g.S = 1; g.XLq = g.XLk = t_width;
  g.WR = dlt_imin(row_size, t_height); g.WC = dlt_imin(col_size, t_width);
  hipLaunchKernelGGL(swa_neighbors_kernel, dim3((unsigned)((T * T + 255) / 256)), dim3(256), 0, (hipStream_t)stream, g, mask);
  DLT_CHECK_LAUNCH("swa_neighbors launch");
  return DLT_OK;
}

extern "C" int dlt_swa_fwd(const void* q, const int64_t q_strides[4], const void* k, const int64_t k_strides[4],
                           const void* v, const int64_t v_strides[4], void* o, const int64_t o_strides[4],
                           float* lse2, const int64_t lse_strides[3],
                           const dlt_swa_shape_t* shape, const dlt_rope_t* rope, void* stream) {
  AttnProblem p;
  int rc = swa_problem("swa_fwd", shape, rope, p);
  if (rc != DLT_OK) return rc;
  AttnTensors t;
  rc = fill_fwd("swa_fwd", t, q, q_strides, k, k_strides, v, v_strides, o, o_strides, lse2, lse_strides);
  if (rc != DLT_OK) return rc;
  return dlt_attn_forward(p, t, (hipStream_t)stream);
}

extern "C" int dlt_swa_bwd(const void* q, const int64_t q_strides[4], const void* k, const int64_t k_strides[4],
                           const void* v, const int64_t v_strides[4], const void* o, const int64_t o_strides[4],
                           const void* d_o, const int64_t do_strides[4],
                           const float* lse2, float* delta, const int64_t lse_strides[3],
                           void* dq, const int64_t dq_strides[4], void* dk, const int64_t dk_strides[4],
                           void* dv, const int64_t dv_strides[4],
                           const dlt_swa_shape_t* shape, const dlt_rope_t* rope, void* stream) {
  AttnProblem p;
  int rc = swa_problem("swa_bwd", shape, rope, p);
  if (rc != DLT_OK) return rc;
  AttnTensors t;
  rc = fill_bwd("swa_bwd", t, q, q_strides, k, k_strides, v, v_strides, o, o_strides, d_o, do_strides, lse2, delta,
                lse_strides, dq, dq_strides, dk, dk_strides, dv, dv_strides);
  if (rc != DLT_OK) return rc;
  return dlt_attn_backward(p, t, (hipStream_t)stream);
}

// ---- backward without a caller-provided scratch buffer ------------------------------------------
// The array's name is a host-side stand-in, not a device address: host code uses the pointer that
// hipGetSymbolAddress returns for the current device (each GPU holds its own copy at its own address).
int dlt_ensure_lds(const void* kern, int bytes) {
  if (bytes <= 48 * 1024) return DLT_OK;   // within the default limit
  struct Entry { const void* kern; int dev; int bytes; };
  static std::mutex mu;
  static std::vector<Entry> seen;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return dlt_set_error(DLT_ERR_LAUNCH, "hipGetDevice: %s", hipGetErrorString(e));
  std::lock_guard<std::mutex> lock(mu);
  Entry* hit = nullptr;
  for (Entry& en : seen)
    if (en.kern == kern && en.dev == dev) { hit = &en; break; }
  if (hit != nullptr && hit->bytes >= bytes) return DLT_OK;
  e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e != hipSuccess) return dlt_set_error(DLT_ERR_LAUNCH, "hipFuncSetAttribute(%d bytes of LDS): %s", bytes, hipGetErrorString(e));
  if (hit != nullptr) hit->bytes = bytes;
  else seen.push_back(Entry{kern, dev, bytes});
  return DLT_OK;
}

namespace {
thread_local int g_family = DLT_FAMILY_NONE;
thread_local bool g_dry = false;
}  // namespace
bool dlt_route_note(int family) { g_family = family; return g_dry; }
bool dlt_route_dry() { return g_dry; }
void dlt_route_reset() { g_family = DLT_FAMILY_NONE; }
extern "C" int dlt_dry_run(int on) { g_dry = on != 0; return DLT_OK; }
extern "C" int dlt_last_kernel_family(void) { return g_family; }

int dlt_device_cus() {
  constexpr int MAXDEV = 64;
  static std::mutex mu;
  static int cus[MAXDEV] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAXDEV) return 256;
  std::lock_guard<std::mutex> lock(mu);
  if (cus[dev] == 0) {
    int n = 0;
    cus[dev] = (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0) ? n : 256;
  }
  return cus[dev];
}

static __device__ __align__(256) float g_delta_scratch[DLT_NOALLOC_MAX_DELTA];

namespace {
constexpr int MAX_DEVICES = 64;
std::mutex g_scratch_mutex;
float* g_scratch_ptr[MAX_DEVICES] = {};

// device address of the scratch array on the CURRENT device, looked up once per device
int delta_scratch(const char* who, float** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return dlt_set_error(DLT_ERR_LAUNCH, "%s: hipGetDevice: %s", who, hipGetErrorString(e));
  if (dev < 0 || dev >= MAX_DEVICES) return dlt_set_error(DLT_ERR_UNSUPPORTED, "%s: device %d is out of range", who, dev);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(g_delta_scratch));
    if (e != hipSuccess || p == nullptr)
      return dlt_set_error(DLT_ERR_LAUNCH, "%s: hipGetSymbolAddress(scratch) on device %d: %s", who, dev, hipGetErrorString(e));
    g_scratch_ptr[dev] = static_cast<float*>(p);
  }
  *out = g_scratch_ptr[dev];
  return DLT_OK;
}
}  // namespace

extern "C" int dlt_swa_bwd_noalloc(const void* q, const int64_t q_strides[4], const void* k, const int64_t k_strides[4],
                                   const void* v, const int64_t v_strides[4], const void* o, const int64_t o_strides[4],
                                   const void* d_o, const int64_t do_strides[4],
                                   const float* lse2, const int64_t lse_strides[3],
                                   void* dq, const int64_t dq_strides[4], void* dk, const int64_t dk_strides[4],
                                   void* dv, const int64_t dv_strides[4],
                                   const dlt_swa_shape_t* shape, const dlt_rope_t* rope, void* stream) {
  const char* who = "swa_bwd_noalloc";
  AttnProblem p;
  int rc = swa_problem(who, shape, rope, p);
  if (rc != DLT_OK) return rc;
  DLT_REQUIRE(lse_strides != nullptr, "%s: lse_strides is NULL", who);
  DLT_REQUIRE(lse_strides[0] >= 0 && lse_strides[1] >= 0 && lse_strides[2] >= 0, "%s: negative lse2 stride", who);
  const int64_t n_tok = (int64_t)shape->t_height * shape->t_width * shape->b_size;
  const int64_t last = (shape->B - 1) * lse_strides[0] + (shape->H - 1) * lse_strides[1] + (n_tok - 1) * lse_strides[2];
  DLT_REQUIRE(last < DLT_NOALLOC_MAX_DELTA,
              "%s: the scratch for delta holds %d floats, this call needs %lld (B * H * N with the strides of lse2); "
              "use dlt_swa_bwd with a caller-provided buffer", who, DLT_NOALLOC_MAX_DELTA, (long long)(last + 1));
  float* delta = nullptr;
  rc = delta_scratch(who, &delta);
  if (rc != DLT_OK) return rc;
  AttnTensors t;
  rc = fill_bwd(who, t, q, q_strides, k, k_strides, v, v_strides, o, o_strides, d_o, do_strides, lse2, delta,
                lse_strides, dq, dq_strides, dk, dk_strides, dv, dv_strides);
  if (rc != DLT_OK) return rc;
  return dlt_attn_backward(p, t, (hipStream_t)stream);
}

extern "C" int dlt_flash_fwd(const void* q, const int64_t q_strides[4], const void* k, const int64_t k_strides[4],
                             const void* v, const int64_t v_strides[4], void* o, const int64_t o_strides[4],
                             float* lse2, const int64_t lse_strides[3],
                             const dlt_flash_shape_t* shape, void* stream) {
  AttnProblem p;
  int rc = flash_problem("flash_fwd", shape, p);
  if (rc != DLT_OK) return rc;
  AttnTensors t;
  rc = fill_fwd("flash_fwd", t, q, q_strides, k, k_strides, v, v_strides, o, o_strides, lse2, lse_strides);
  if (rc != DLT_OK) return rc;
  return dlt_attn_forward(p, t, (hipStream_t)stream);
}

extern "C" int dlt_flash_bwd(const void* q, const int64_t q_strides[4], const void* k, const int64_t k_strides[4],
                             const void* v, const int64_t v_strides[4], const void* o, const int64_t o_strides[4],
                             const void* d_o, const int64_t do_strides[4],
                             const float* lse2, float* delta, const int64_t lse_strides[3],
                             void* dq, const int64_t dq_strides[4], void* dk, const int64_t dk_strides[4],
                             void* dv, const int64_t dv_strides[4],
                             const dlt_flash_shape_t* shape, void* stream) {
  AttnProblem p;
  int rc = flash_problem("flash_bwd", shape, p);
  if (rc != DLT_OK) return rc;
  AttnTensors t;
  rc = fill_bwd("flash_bwd", t, q, q_strides, k, k_strides, v, v_strides, o, o_strides, d_o, do_strides, lse2, delta,
                lse_strides, dq, dq_strides, dk, dk_strides, dv, dv_strides);
  if (rc != DLT_OK) return rc;
  return dlt_attn_backward(p, t, (hipStream_t)stream);
}

// ---- image-layout entry points ------------------------------------------------------------------
extern "C" int dlt_swa_image_offsets(int32_t t_height, int32_t t_width, int32_t bh, int32_t bw, int64_t stride_y,
                                     int64_t stride_x, int64_t* offsets, void* stream) {
  DLT_REQUIRE(t_height > 0 && t_width > 0 && bh > 0 && bw > 0, "swa_image_offsets: bad grid / tile");
  DLT_REQUIRE(offsets != nullptr, "swa_image_offsets: offsets is NULL");
  const int64_t n = (int64_t)t_height * t_width * bh * bw;
  DLT_REQUIRE(n <= 0x3fffffff, "swa_image_offsets: too many tokens");
  const DltTokMap tm = dlt_tokmap_image((uint32_t)bh, (uint32_t)bw, (uint32_t)t_width);
  hipLaunchKernelGGL(swa_image_offsets_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, tm,
                     stride_y, stride_x, n, offsets);
  DLT_CHECK_LAUNCH("swa_image_offsets launch");
  return DLT_OK;
}

extern "C" int dlt_swa_fwd_image(const void* q, const int64_t q_strides[5], const void* k, const int64_t k_strides[5],
                                 const void* v, const int64_t v_strides[5], void* o, const int64_t o_strides[5],
                                 float* lse2, const int64_t lse_strides[3], const dlt_swa_shape_t* shape,
                                 const dlt_swa_tile_t* tile, const dlt_rope_t* rope, void* stream) {
  const char* who = "swa_fwd_image";
  int rc = image_tile(who, shape, tile);
  if (rc != DLT_OK) return rc;
  AttnProblem p;
  rc = swa_problem(who, shape, rope, p);
  if (rc != DLT_OK) return rc;
  const void* const ptrs[] = {q, k, v, o, lse2};
  const int64_t* const st[] = {q_strides, k_strides, v_strides, o_strides, lse_strides};
  rc = check_ptrs(who, ptrs, st, 5);
  if (rc != DLT_OK) return rc;
  AttnTensors t;
  memset(&t, 0, sizeof(t));
  t.q = q; t.k = k; t.v = v; t.out_o = o; t.lse = lse2;
  cp3(t.ls, lse_strides);
  int64_t* const mine[] = {t.qs, t.ks, t.vs, t.os};
  for (int i = 0; i < 4; i++) {
    rc = image_strides(who, i, st[i], mine[i]);
    if (rc != DLT_OK) return rc;
  }
  image_finish(p, tile, mine, 4);
  return dlt_attn_forward(p, t, (hipStream_t)stream);
}

extern "C" int dlt_swa_bwd_image(const void* q, const int64_t q_strides[5], const void* k, const int64_t k_strides[5],
                                 const void* v, const int64_t v_strides[5], const void* o, const int64_t o_strides[5],
                                 const void* d_o, const int64_t do_strides[5],
                                 const float* lse2, float* delta, const int64_t lse_strides[3],
                                 void* dq, const int64_t dq_strides[5], void* dk, const int64_t dk_strides[5],
                                 void* dv, const int64_t dv_strides[5], const dlt_swa_shape_t* shape,
                                 const dlt_swa_tile_t* tile, const dlt_rope_t* rope, void* stream) {
  const char* who = "swa_bwd_image";
  int rc = image_tile(who, shape, tile);
  if (rc != DLT_OK) return rc;
  AttnProblem p;
  rc = swa_problem(who, shape, rope, p);
  if (rc != DLT_OK) return rc;
  const void* const ptrs[] = {q, k, v, o, d_o, dq, dk, dv, lse2, delta};
  const int64_t* const st[] = {q_strides, k_strides, v_strides, o_strides, do_strides, dq_strides, dk_strides, dv_strides,
                               lse_strides, lse_strides};
  rc = check_ptrs(who, ptrs, st, 10);
  if (rc != DLT_OK) return rc;
  AttnTensors t;
  memset(&t, 0, sizeof(t));
  t.q = q; t.k = k; t.v = v; t.o = o; t.d_o = d_o; t.lse = const_cast<float*>(lse2); t.delta = delta;
  t.dq = dq; t.dk = dk; t.dv = dv;
  cp3(t.ls, lse_strides);
  int64_t* const mine[] = {t.qs, t.ks, t.vs, t.os, t.dos, t.dqs, t.dks, t.dvs};
  for (int i = 0; i < 8; i++) {
    rc = image_strides(who, i, st[i], mine[i]);
    if (rc != DLT_OK) return rc;
  }
  image_finish(p, tile, mine, 8);
  return dlt_attn_backward(p, t, (hipStream_t)stream);
}

// ---- fused rotation with the rotated q, k kept for the backward pass -------------------------------
extern "C" int dlt_swa_fwd_rot(const void* q, const int64_t q_strides[4], const void* k, const int64_t k_strides[4],
                               const void* v, const int64_t v_strides[4], void* o, const int64_t o_strides[4],
                               float* lse2, const int64_t lse_strides[3],
                               void* q_rot, const int64_t q_rot_strides[4], void* k_rot, const int64_t k_rot_strides[4],
                               const dlt_swa_shape_t* shape, const dlt_rope_t* rope, void* stream) {
  const char* who = "swa_fwd_rot";
  DLT_REQUIRE(rope != nullptr, "%s: rope is NULL", who);
  AttnProblem p;
  int rc = swa_problem(who, shape, rope, p);
  if (rc != DLT_OK) return rc;
  AttnTensors t;
  rc = fill_fwd(who, t, q, q_strides, k, k_strides, v, v_strides, o, o_strides, lse2, lse_strides);
  if (rc != DLT_OK) return rc;
  DLT_REQUIRE(q_rot != nullptr && k_rot != nullptr && q_rot_strides != nullptr && k_rot_strides != nullptr,
              "%s: q_rot / k_rot is NULL", who);
  // other workgroups still read q and k while a workgroup stores its rotated tokens
  DLT_REQUIRE(q_rot != q && k_rot != k && q_rot != k && k_rot != q && q_rot != k_rot,
              "%s: q_rot and k_rot must be distinct buffers that do not alias q or k", who);
  t.q_rot = q_rot; t.k_rot = k_rot;
  cp4(t.qrs, q_rot_strides); cp4(t.krs, k_rot_strides);
  return dlt_attn_forward(p, t, (hipStream_t)stream);
}

extern "C" int dlt_swa_bwd_rot(const void* q_rot, const int64_t q_rot_strides[4], const void* k_rot,
                               const int64_t k_rot_strides[4], const void* v, const int64_t v_strides[4], const void* o,
                               const int64_t o_strides[4], const void* d_o, const int64_t do_strides[4],
                               const float* lse2, float* delta, const int64_t lse_strides[3],
                               void* dq, const int64_t dq_strides[4], void* dk, const int64_t dk_strides[4],
                               void* dv, const int64_t dv_strides[4],
                               const dlt_swa_shape_t* shape, const dlt_rope_t* rope, void* stream) {
  const char* who = "swa_bwd_rot";
  DLT_REQUIRE(rope != nullptr, "%s: rope is NULL", who);
  AttnProblem p;
  int rc = swa_problem(who, shape, rope, p);
  if (rc != DLT_OK) return rc;
  p.rope_prerot = 1;
  AttnTensors t;
  rc = fill_bwd(who, t, q_rot, q_rot_strides, k_rot, k_rot_strides, v, v_strides, o, o_strides, d_o, do_strides, lse2, delta,
                lse_strides, dq, dq_strides, dk, dk_strides, dv, dv_strides);
  if (rc != DLT_OK) return rc;
  return dlt_attn_backward(p, t, (hipStream_t)stream);
}
