// Standalone in-place 2D rotary encoding for gfx950: a pure HBM-streaming kernel.
//
// Replaces rope2d_fwd_kernel / rope2d_bwd_kernel (src/fused_rope2d.py:24-122) with the
// semantics of rope2d_ref (:204-225): an axis whose 16-bit index is negative is left
// untouched (the Triton kernel's `other=1` / `other=0` fills, :53-54, are not reproduced).
//
// Data movement: only the 4R rotated dims of tokens with at least one rotated axis are
// read and written (R + W of 2 * elt * 4R bytes per token row); pass-through dims and
// no-PE tokens generate no traffic.  One thread owns one (token, 8-wide pair chunk) and
// keeps its 8 (cos, sin) pairs in registers while it walks over the batch rows, so the
// table is read once per thread and the x traffic is 16-byte vector loads/stores.
#include "dlt_internal.hpp"

namespace {

struct RopeKArgs {
  void* x[2];
  int64_t s[2][3];
  int32_t nb[2];
  int32_t N, C;
  RopeDev r;
  int32_t bb;  // batch rows handled by one block in y
};

typedef __bf16 bf16_t;
typedef _Float16 f16_t;

template <typename T> struct alignas(8 * sizeof(T) > 16 ? 16 : 8 * sizeof(T)) Vec8 { T v[8]; };  // 16 bytes for 2-byte T, 32 for float

template <typename T> __device__ inline float to_f(T v) { return (float)v; }
template <typename T> __device__ inline T from_f(float v) { return (T)v; }

// y0 = x0*c - x1*s ; y1 = x0*s + x1*c, each product rounded before the add: the evaluation
// order of the eager reference (src/fused_rope2d.py:221-222), so fp32 results are bit-equal.
__device__ inline void rotate(float x0, float x1, float c, float s, float& y0, float& y1) {
#pragma clang fp contract(off)
  const float a = x0 * c, b = x1 * s, d = x0 * s, e = x1 * c;
  y0 = a - b;
  y1 = d + e;
}

constexpr int UNR = 4;

// Fast path: unit last stride, 16-byte aligned rows, R % 8 == 0, aligned tables.
template <typename T>
__global__ __launch_bounds__(256) void rope2d_vec_kernel(RopeKArgs a) {
  const int z = blockIdx.z;
  const int cpa = a.r.R >> 3;          // 8-wide chunks per half axis
  const int items = 2 * cpa;           // (axis, chunk) work items per token
  const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t n = gid / items;
  if (n >= a.N) return;
  const int pc = (int)(gid - n * items);
  const int ax = pc / cpa, ci = pc - ax * cpa;

  // The x loads do not depend on idx: they are issued first so that the idx -> table chain and
  // the first batch of data travel together (tokens with an unrotated axis cost a read only).
  const int32_t id = a.r.idx[n];
  const int d0 = ax * 2 * a.r.R + 8 * ci, d1 = d0 + a.r.R;
  T* xb = reinterpret_cast<T*>(a.x[z]) + n * a.s[z][1];
  const int64_t sb = a.s[z][0];
  const int b_begin = blockIdx.y * a.bb;
  const int b_end = dlt_imin(b_begin + a.bb, a.nb[z]);
  Vec8<T> v0[UNR], v1[UNR];
#pragma unroll
  for (int u = 0; u < UNR; u++) {
    if (b_begin + u < b_end) {
      T* px = xb + (int64_t)(b_begin + u) * sb;
      v0[u] = *reinterpret_cast<const Vec8<T>*>(px + d0);
      v1[u] = *reinterpret_cast<const Vec8<T>*>(px + d1);
    }
  }
  int p = ax == 0 ? dlt_rope_row(id) : dlt_rope_col(id);
  if (p < 0) return;  // this axis is not rotated for this token: nothing is written
  p = dlt_imin(p, (ax == 0 ? a.r.row_len : a.r.col_len) - 1);
  const float* tab = (ax == 0 ? a.r.row_cs + (int64_t)p * a.r.rs0 : a.r.col_cs + (int64_t)p * a.r.cs0) + 16 * ci;
  float cs[16];
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const float4 t = reinterpret_cast<const float4*>(tab)[j];
    cs[4 * j] = t.x; cs[4 * j + 1] = t.y; cs[4 * j + 2] = t.z; cs[4 * j + 3] = t.w;
  }
  if (a.r.inverse) {
#pragma unroll
    for (int j = 0; j < 8; j++) cs[2 * j + 1] = -cs[2 * j + 1];
  }
  for (int b0 = b_begin; b0 < b_end; b0 += UNR) {
    if (b0 != b_begin) {
#pragma unroll
      for (int u = 0; u < UNR; u++) {
        if (b0 + u < b_end) {
          T* px = xb + (int64_t)(b0 + u) * sb;
          v0[u] = *reinterpret_cast<const Vec8<T>*>(px + d0);
          v1[u] = *reinterpret_cast<const Vec8<T>*>(px + d1);
        }
      }
    }
#pragma unroll
    for (int u = 0; u < UNR; u++) {
      if (b0 + u < b_end) {
        Vec8<T> y0, y1;
#pragma unroll
        for (int j = 0; j < 8; j++) {
          float r0, r1;
          rotate(to_f(v0[u].v[j]), to_f(v1[u].v[j]), cs[2 * j], cs[2 * j + 1], r0, r1);
          y0.v[j] = from_f<T>(r0);
          y1.v[j] = from_f<T>(r1);
        }
        T* px = xb + (int64_t)(b0 + u) * sb;
        *reinterpret_cast<Vec8<T>*>(px + d0) = y0;
        *reinterpret_cast<Vec8<T>*>(px + d1) = y1;
      }
    }
  }
}

// Generic path: any strides, any R, any alignment; one thread per (token, axis, i).
template <typename T>
__global__ __launch_bounds__(256) void rope2d_generic_kernel(RopeKArgs a) {
  const int z = blockIdx.z;
  const int items = 2 * a.r.R;
  const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t n = gid / items;
  if (n >= a.N) return;
  const int pc = (int)(gid - n * items);
  const int ax = pc / a.r.R, i = pc - ax * a.r.R;
  const int32_t id = a.r.idx[n];
  int p = ax == 0 ? dlt_rope_row(id) : dlt_rope_col(id);
  if (p < 0) return;
  p = dlt_imin(p, (ax == 0 ? a.r.row_len : a.r.col_len) - 1);
  const float* tab = (ax == 0 ? a.r.row_cs + (int64_t)p * a.r.rs0 : a.r.col_cs + (int64_t)p * a.r.cs0) + 2 * i;
  const float c = tab[0];
  const float s = a.r.inverse ? -tab[1] : tab[1];
  const int d0 = ax * 2 * a.r.R + i, d1 = d0 + a.r.R;
  T* xb = reinterpret_cast<T*>(a.x[z]) + n * a.s[z][1];
  const int b_begin = blockIdx.y * a.bb;
  const int b_end = dlt_imin(b_begin + a.bb, a.nb[z]);
  for (int b = b_begin; b < b_end; b++) {
    T* px = xb + (int64_t)b * a.s[z][0];
    float y0, y1;
    rotate(to_f(px[d0 * a.s[z][2]]), to_f(px[d1 * a.s[z][2]]), c, s, y0, y1);
    px[d0 * a.s[z][2]] = from_f<T>(y0);
    px[d1 * a.s[z][2]] = from_f<T>(y1);
  }
}

// Out-of-place rotation of a [B, H, N, C] tensor with any strides: dst = rotate(src), every element
// copied (pass-through dims and unrotated tokens included).  One thread per element; the slow,
// layout-agnostic companion of the in-place kernels, used when a caller wants the rotated tensor
// next to the original and the attention kernels cannot produce it themselves.
struct RopeCopyArgs {
  const void* src;
  void* dst;
  int64_t ss[4], ds[4];
  int32_t B, H, N, C;
  RopeDev r;
};

template <typename T>
__global__ __launch_bounds__(256) void rope2d_copy_kernel(RopeCopyArgs a) {
  const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t per_bh = (int64_t)a.N * a.C;
  const int64_t bh = gid / per_bh;
  if (bh >= (int64_t)a.B * a.H) return;
  const int64_t rem = gid - bh * per_bh;
  const int n = (int)(rem / a.C), d = (int)(rem - (int64_t)n * a.C);
  const int b = (int)(bh / a.H), h = (int)(bh - (int64_t)b * a.H);
  const T* ps = reinterpret_cast<const T*>(a.src) + b * a.ss[0] + h * a.ss[1] + n * a.ss[2];
  T* pd = reinterpret_cast<T*>(a.dst) + b * a.ds[0] + h * a.ds[1] + n * a.ds[2];
  const T self = ps[d * a.ss[3]];
  T out = self;
  if (d < 4 * a.r.R) {
    const int region = d / a.r.R, i = d - region * a.r.R, ax = region >> 1;
    const int32_t id = a.r.idx[n];
    int p = ax == 0 ? dlt_rope_row(id) : dlt_rope_col(id);
    if (p >= 0) {
      p = dlt_imin(p, (ax == 0 ? a.r.row_len : a.r.col_len) - 1);
      const float* tab = (ax == 0 ? a.r.row_cs + (int64_t)p * a.r.rs0 : a.r.col_cs + (int64_t)p * a.r.cs0) + 2 * i;
      const float c = tab[0];
      const float s = a.r.inverse ? -tab[1] : tab[1];
      const bool is_x0 = (region & 1) == 0;
      const float other = to_f(ps[(is_x0 ? d + a.r.R : d - a.r.R) * a.ss[3]]);
      float y0, y1;
      rotate(is_x0 ? to_f(self) : other, is_x0 ? other : to_f(self), c, s, y0, y1);
      out = from_f<T>(is_x0 ? y0 : y1);
    }
  }
  pd[d * a.ds[3]] = out;
}

// The same for rows of element stride 1 whose 8-element chunks are 16-byte (32-byte for fp32) aligned and
// R % 8 == 0: one thread per chunk, the partner chunk is read a second time (from L1).
template <typename T>
__global__ __launch_bounds__(256) void rope2d_copy_vec_kernel(RopeCopyArgs a) {
  const int nch = a.C >> 3;
  const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t per_bh = (int64_t)a.N * nch;
  const int64_t bh = gid / per_bh;
  if (bh >= (int64_t)a.B * a.H) return;
  const int64_t rem = gid - bh * per_bh;
  const int n = (int)(rem / nch), c = (int)(rem - (int64_t)n * nch);
  const int b = (int)(bh / a.H), h = (int)(bh - (int64_t)b * a.H);
  const T* ps = reinterpret_cast<const T*>(a.src) + b * a.ss[0] + h * a.ss[1] + n * a.ss[2];
  T* pd = reinterpret_cast<T*>(a.dst) + b * a.ds[0] + h * a.ds[1] + n * a.ds[2];
  Vec8<T> self = *reinterpret_cast<const Vec8<T>*>(ps + 8 * c);
  const int r8 = a.r.R >> 3;
  if (c < 4 * r8) {
    const int region = c / r8, ci = c - region * r8, ax = region >> 1;
    const bool is_x0 = (region & 1) == 0;
    const Vec8<T> other = *reinterpret_cast<const Vec8<T>*>(ps + 8 * (is_x0 ? c + r8 : c - r8));
    const int32_t id = a.r.idx[n];
    int p = ax == 0 ? dlt_rope_row(id) : dlt_rope_col(id);
    if (p >= 0) {
      p = dlt_imin(p, (ax == 0 ? a.r.row_len : a.r.col_len) - 1);
      const float* tab = (ax == 0 ? a.r.row_cs + (int64_t)p * a.r.rs0 : a.r.col_cs + (int64_t)p * a.r.cs0) + 16 * ci;
#pragma unroll
      for (int j = 0; j < 8; j++) {
        const float cs = tab[2 * j], sn = a.r.inverse ? -tab[2 * j + 1] : tab[2 * j + 1];
        float y0, y1;
        rotate(is_x0 ? to_f(self.v[j]) : to_f(other.v[j]), is_x0 ? to_f(other.v[j]) : to_f(self.v[j]), cs, sn, y0, y1);
        self.v[j] = from_f<T>(is_x0 ? y0 : y1);
      }
    }
  }
  *reinterpret_cast<Vec8<T>*>(pd + 8 * c) = self;
}

__global__ void rope_pe_mask_kernel(const int32_t* idx, int64_t n_tokens, uint8_t* bits) {
  const int64_t n = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (n >= n_tokens) return;
  const int32_t id = idx[n];
  bits[n] = (uint8_t)((dlt_rope_row(id) >= 0 ? 1 : 0) | (dlt_rope_col(id) >= 0 ? 2 : 0));
}

template <typename T>
int launch_rope(const RopeKArgs& a, bool vec, hipStream_t stream, int ntens) {
  const int items = vec ? 2 * (a.r.R / 8) : 2 * a.r.R;
  const int64_t threads = (int64_t)a.N * items;
  const int64_t gx = (threads + 255) / 256;
  if (gx > 0x7fffffff) return dlt_set_error(DLT_ERR_UNSUPPORTED, "rope2d: too many tokens (%lld)", (long long)a.N);
  const int maxb = dlt_imax(a.nb[0], ntens > 1 ? a.nb[1] : 0);
  dim3 grid((unsigned)gx, (unsigned)((maxb + a.bb - 1) / a.bb), (unsigned)ntens);
  dlt_timing_before(DLT_K_ROPE, stream);
  if (vec) hipLaunchKernelGGL(rope2d_vec_kernel<T>, grid, dim3(256), 0, stream, a);
  else hipLaunchKernelGGL(rope2d_generic_kernel<T>, grid, dim3(256), 0, stream, a);
  dlt_timing_after(stream);
  DLT_CHECK_LAUNCH("rope2d launch");
  return DLT_OK;
}

int rope_impl(void* const x[2], const int64_t* const st[2], const int64_t nb[2], int ntens, int64_t N, int64_t C,
              const dlt_rope_t* rope, int inverse, int dtype, void* stream) {
  DLT_REQUIRE(dtype == DLT_BF16 || dtype == DLT_FP16 || dtype == DLT_FP32, "rope2d: bad dtype %d", dtype);
  DLT_REQUIRE(N >= 0 && C >= 0 && N <= 0x7fffffff && C <= 0x7fffffff, "rope2d: bad shape N=%lld C=%lld", (long long)N, (long long)C);
  int rc = dlt_validate_rope(rope, C);
  if (rc != DLT_OK) return rc;
  RopeKArgs a;
  a.N = (int32_t)N; a.C = (int32_t)C;
  a.r = dlt_make_rope_dev(rope, inverse);
  const int es = dlt_elem_size(dtype);
  const int vec_bytes = 8 * es;
  bool vec = (a.r.R % 8 == 0) && ((uintptr_t)a.r.row_cs % 16 == 0) && ((uintptr_t)a.r.col_cs % 16 == 0) &&
             (a.r.rs0 % 4 == 0) && (a.r.cs0 % 4 == 0);
  int64_t maxb = 0;
  for (int z = 0; z < 2; z++) {
    a.x[z] = z < ntens ? x[z] : nullptr;
    a.nb[z] = 0;
    for (int j = 0; j < 3; j++) a.s[z][j] = 0;
    if (z >= ntens) continue;
    DLT_REQUIRE(nb[z] >= 0 && nb[z] <= 0x7fffffff, "rope2d: bad batch %lld", (long long)nb[z]);
    DLT_REQUIRE(x[z] != nullptr || nb[z] * N == 0, "rope2d: x is NULL");
    a.nb[z] = (int32_t)nb[z];
    for (int j = 0; j < 3; j++) a.s[z][j] = st[z][j];
    vec = vec && st[z][2] == 1 && ((uintptr_t)x[z] % vec_bytes == 0) && (st[z][0] * es % vec_bytes == 0) &&
          (st[z][1] * es % vec_bytes == 0);
    if (nb[z] > maxb) maxb = nb[z];
  }
  if (N == 0 || maxb == 0 || a.r.R == 0) return DLT_OK;
  const int items = vec ? 2 * (a.r.R / 8) : 2 * a.r.R;
  const int64_t bx = ((int64_t)N * items + 255) / 256;
  int bb = (int)maxb;
  // two workgroups per CU: measured optimum on the benchmark shape (a thread's token index -> table row chain is paid once
  // per workgroup, so more, shorter workgroups re-read the tables more often: 1024 blocks +2 %, 2048 blocks +16 %, 256 +10 %)
  while (bb > 1 && bx * ((maxb + bb - 1) / bb) * ntens < 512) bb = (bb + 1) / 2;
  a.bb = bb < 1 ? 1 : bb;
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case DLT_BF16: return launch_rope<bf16_t>(a, vec, s, ntens);
    case DLT_FP16: return launch_rope<f16_t>(a, vec, s, ntens);
    default: return launch_rope<float>(a, vec, s, ntens);
  }
}

}  // namespace

int dlt_rope_rotate_copy(const void* src, const int64_t* ss, void* dst, const int64_t* ds, int B, int H, int64_t N, int C,
                         const RopeDev& rope, int dtype, hipStream_t stream) {
  if (dlt_route_dry()) return DLT_OK;
  RopeCopyArgs a;
  a.src = src; a.dst = dst;
  for (int i = 0; i < 4; i++) { a.ss[i] = ss[i]; a.ds[i] = ds[i]; }
  a.B = B; a.H = H; a.N = (int32_t)N; a.C = C;
  a.r = rope;
  const int es = dlt_elem_size(dtype), vb = 8 * es;
  bool vec = C % 8 == 0 && rope.R % 8 == 0 && ss[3] == 1 && ds[3] == 1 && (uintptr_t)src % vb == 0 && (uintptr_t)dst % vb == 0;
  for (int i = 0; i < 3; i++) vec = vec && (ss[i] * es) % vb == 0 && (ds[i] * es) % vb == 0;
  const int64_t total = (int64_t)B * H * N * (vec ? C / 8 : C);
  if (total == 0) return DLT_OK;
  const int64_t gx = (total + 255) / 256;
  if (gx > 0x7fffffff) return dlt_set_error(DLT_ERR_UNSUPPORTED, "rope rotate-copy: tensor too large");
  dlt_timing_before(DLT_K_ROPE, stream);
  const dim3 grid((unsigned)gx), block(256);
  if (vec) {
    switch (dtype) {
      case DLT_BF16: hipLaunchKernelGGL(rope2d_copy_vec_kernel<bf16_t>, grid, block, 0, stream, a); break;
      case DLT_FP16: hipLaunchKernelGGL(rope2d_copy_vec_kernel<f16_t>, grid, block, 0, stream, a); break;
      default: hipLaunchKernelGGL(rope2d_copy_vec_kernel<float>, grid, block, 0, stream, a); break;
    }
  } else {
    switch (dtype) {
      case DLT_BF16: hipLaunchKernelGGL(rope2d_copy_kernel<bf16_t>, grid, block, 0, stream, a); break;
      case DLT_FP16: hipLaunchKernelGGL(rope2d_copy_kernel<f16_t>, grid, block, 0, stream, a); break;
      default: hipLaunchKernelGGL(rope2d_copy_kernel<float>, grid, block, 0, stream, a); break;
    }
  }
  dlt_timing_after(stream);
  DLT_CHECK_LAUNCH("rope rotate-copy launch");
  return DLT_OK;
}

// In-place rotation of a [B, H, N, C] tensor with any strides through the standalone kernels: one launch
// when (B, H) collapses into one batch stride, else one per b.
int dlt_rope_inplace_4d(void* x, const int64_t* st, int B, int H, int64_t N, int C, const dlt_rope_t* rope, int inverse,
                        int dtype, hipStream_t stream) {
  if (dlt_route_dry()) return DLT_OK;
  const bool flat = B == 1 || st[0] == (int64_t)H * st[1];
  const int64_t s3[3] = {st[1], st[2], st[3]};
  const int es = dlt_elem_size(dtype);
  for (int b = 0; b < (flat ? 1 : B); b++) {
    void* const xs[2] = {static_cast<char*>(x) + (int64_t)b * st[0] * es, nullptr};
    const int64_t* const sts[2] = {s3, nullptr};
    const int64_t nb[2] = {flat ? (int64_t)B * H : H, 0};
    int rc = rope_impl(xs, sts, nb, 1, N, C, rope, inverse, dtype, stream);
    if (rc != DLT_OK) return rc;
  }
  return DLT_OK;
}

int dlt_validate_rope(const dlt_rope_t* rope, int64_t n_dim) {
  DLT_REQUIRE(rope != nullptr, "rope: descriptor is NULL");
  DLT_REQUIRE(rope->n_rdim >= 0, "rope: n_rdim %d < 0", rope->n_rdim);
  DLT_REQUIRE((int64_t)4 * rope->n_rdim <= n_dim, "rope: 4 * n_rdim (%d) exceeds the head dim (%lld)", 4 * rope->n_rdim, (long long)n_dim);
  if (rope->n_rdim == 0) return DLT_OK;  // nothing is rotated; tables may be empty
  DLT_REQUIRE(rope->idx != nullptr, "rope: idx is NULL");
  DLT_REQUIRE(rope->row_cs != nullptr && rope->col_cs != nullptr, "rope: cos/sin table is NULL");
  DLT_REQUIRE(rope->row_len > 0 && rope->col_len > 0, "rope: empty cos/sin table");
  DLT_REQUIRE(rope->row_cs_stride0 >= 2 * rope->n_rdim && rope->col_cs_stride0 >= 2 * rope->n_rdim,
              "rope: table row stride smaller than 2 * n_rdim");
  return DLT_OK;
}

RopeDev dlt_make_rope_dev(const dlt_rope_t* rope, int inverse) {
  RopeDev r;
  if (rope == nullptr) {
    r = RopeDev{};
    return r;
  }
  r.idx = rope->idx; r.row_cs = rope->row_cs; r.col_cs = rope->col_cs;
  r.rs0 = rope->row_cs_stride0; r.cs0 = rope->col_cs_stride0;
  r.R = rope->n_rdim; r.row_len = rope->row_len; r.col_len = rope->col_len;
  r.inverse = inverse ? 1 : 0;
  r.enabled = 1;
  return r;
}

extern "C" int dlt_rope2d(void* x, const int64_t x_strides[3], int64_t n_batch, int64_t n_tokens, int64_t n_dim,
                          const dlt_rope_t* rope, int inverse, int dtype, void* stream) {
  DLT_REQUIRE(x_strides != nullptr, "rope2d: strides is NULL");
  void* const xs[2] = {x, nullptr};
  const int64_t* const st[2] = {x_strides, nullptr};
  const int64_t nb[2] = {n_batch, 0};
  return rope_impl(xs, st, nb, 1, n_tokens, n_dim, rope, inverse, dtype, stream);
}

extern "C" int dlt_rope2d_pair(void* x0, const int64_t x0_strides[3], int64_t n_batch0,
                               void* x1, const int64_t x1_strides[3], int64_t n_batch1,
                               int64_t n_tokens, int64_t n_dim,
                               const dlt_rope_t* rope, int inverse, int dtype, void* stream) {
  DLT_REQUIRE(x0_strides != nullptr && x1_strides != nullptr, "rope2d_pair: strides is NULL");
  void* const xs[2] = {x0, x1};
  const int64_t* const st[2] = {x0_strides, x1_strides};
  const int64_t nb[2] = {n_batch0, n_batch1};
  return rope_impl(xs, st, nb, 2, n_tokens, n_dim, rope, inverse, dtype, stream);
}

extern "C" int dlt_rope_pe_mask(const int32_t* idx, int64_t n_tokens, uint8_t* bits, void* stream) {
  DLT_REQUIRE(n_tokens >= 0, "rope_pe_mask: negative token count");
  if (n_tokens == 0) return DLT_OK;
  DLT_REQUIRE(idx != nullptr && bits != nullptr, "rope_pe_mask: NULL pointer");
  hipLaunchKernelGGL(rope_pe_mask_kernel, dim3((unsigned)((n_tokens + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                     idx, n_tokens, bits);
  DLT_CHECK_LAUNCH("rope_pe_mask launch");
  return DLT_OK;
}
