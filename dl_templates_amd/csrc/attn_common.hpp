// Device helpers shared by the attention kernels (forward, backward dK/dV, backward dQ).
//
// Register layouts (wave64, v_mfma_f32_16x16x32_{bf16,f16}); lane = 16 * g + n:
//   A operand (16 x 32): lane holds row n,   k-slots 8g .. 8g+7
//   B operand (32 x 16): lane holds col n,   k-slots 8g .. 8g+7
//   C result  (16 x 16): lane holds col n,   rows 4g .. 4g+3
// A product only needs A and B to agree on which k-slot means what, so the slot order is
// chosen per use: contiguous head-dim chunks for q.k products, and for products that
// contract over tokens the order in which the C layout of the previous product delivers
// them (slot 8g + 4*mb + i  <->  token 16*mb + 4g + i of a 32-token block), which makes the
// probability tile a B operand without any cross-lane traffic.  The matching A operand
// (a [token][dim] LDS tile read with tokens along k) comes from ds_read_b64_tr_b16.
#pragma once
#include "dlt_internal.hpp"

typedef __bf16 bf16_t;
typedef _Float16 f16_t;
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((__vector_size__(8)));

#define DLT_LDS __attribute__((address_space(3)))
#define DLT_DEV __device__ __forceinline__

// compute type for an I/O element type: fp16 stays fp16, bf16 and fp32 run on bf16 MFMA
template <typename TIO> struct ComputeOf { typedef bf16_t type; };
template <> struct ComputeOf<f16_t> { typedef f16_t type; };

template <typename CT> struct Mma;
template <> struct Mma<bf16_t> {
  static DLT_DEV f32x4 mfma(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
};
template <> struct Mma<f16_t> {
  static DLT_DEV f32x4 mfma(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
};

// two floats -> one dword of two 16-bit values (round to nearest even), converted as a vector so
// that the compiler emits a single packed conversion
template <typename CT> DLT_DEV unsigned int pack2(float lo, float hi) {
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  typedef CT ctx2 __attribute__((ext_vector_type(2)));
  const f32x2 v = {lo, hi};
  return __builtin_bit_cast(unsigned int, __builtin_convertvector(v, ctx2));
}
template <typename CT> DLT_DEV float unpack_lo(unsigned int w) {
  return (float)__builtin_bit_cast(CT, (unsigned short)(w & 0xffffu));
}
template <typename CT> DLT_DEV float unpack_hi(unsigned int w) {
  return (float)__builtin_bit_cast(CT, (unsigned short)(w >> 16));
}

// c + a.lo * b.lo + a.hi * b.hi for dwords of two 16-bit values (one vector instruction, fp32 accumulation)
template <typename CT> DLT_DEV float dot2_acc(unsigned int a, unsigned int b, float c);
template <> DLT_DEV float dot2_acc<bf16_t>(unsigned int a, unsigned int b, float c) {
  typedef __bf16 v2 __attribute__((ext_vector_type(2)));
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(v2, a), __builtin_bit_cast(v2, b), c, false);
}
template <> DLT_DEV float dot2_acc<f16_t>(unsigned int a, unsigned int b, float c) {
  typedef _Float16 v2 __attribute__((ext_vector_type(2)));
  return __builtin_amdgcn_fdot2(__builtin_bit_cast(v2, a), __builtin_bit_cast(v2, b), c, false);
}

DLT_DEV float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
DLT_DEV float fast_log2(float x) { return __builtin_amdgcn_logf(x); }
DLT_DEV float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }

// Values loaded from HBM before a streaming loop and first used inside it (own-token fragments,
// per-token scalars).  Left alone, the compiler places the wait for them at the first use INSIDE
// the loop as `s_waitcnt vmcnt(0)`, which on every iteration also waits for the chunk prefetch that
// was issued just before, i.e. the prefetch never overlaps the products.  Consuming the values here
// moves that wait in front of the loop (loads complete in order).
// Placed at the top of a wave-uniform `if` body whose work is rarely needed (edge masks, the
// accumulator rescale of the online softmax): the compiler otherwise turns the body into
// unconditional select / multiply instructions that every iteration pays for.
DLT_DEV void keep_branch() { asm volatile(""); }

DLT_DEV void pin_loaded(const u32x4& v) { asm volatile("" ::"v"(v)); }
DLT_DEV void pin_loaded(float v) { asm volatile("" ::"v"(v)); }
DLT_DEV void pin_loaded(const f32x4& v) { asm volatile("" ::"v"(v)); }
template <int N>
DLT_DEV void pin_loaded(const u32x4 (&f)[N]) {
#pragma unroll
  for (int i = 0; i < N; i++) pin_loaded(f[i]);
}
template <int M, int N>
DLT_DEV void pin_loaded(const u32x4 (&f)[M][N]) {
#pragma unroll
  for (int i = 0; i < M; i++) pin_loaded(f[i]);
}

DLT_DEV u32x4 lds_read16(const char* p) { return *reinterpret_cast<const u32x4*>(p); }
DLT_DEV void lds_write16(char* p, u32x4 v) { *reinterpret_cast<u32x4*>(p) = v; }

// transpose read: within a 16-lane group lane i receives element (i % 4) of the 8-byte chunk
// addressed by lane 4j + i/4, for j = 0..3 (the four 16-bit results)
DLT_DEV u32x2 lds_read_tr16(const char* p) {
  s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((DLT_LDS s16x4*)(DLT_LDS void*)(p));
  return __builtin_bit_cast(u32x2, v);
}

// A operand with tokens along k for the 32-token block starting at LDS row `row0` of a
// [token][dim] tile: dims dim0 .. dim0+15 become the 16 rows of the operand.
DLT_DEV u32x4 lds_read_tokens_as_k(const char* tile, int pitch, int row0, int dim0, int n, int g) {
  const char* p = tile + (row0 + 4 * g + (n >> 2)) * pitch + (dim0 + 4 * (n & 3)) * 2;
  const u32x2 lo = lds_read_tr16(p);
  const u32x2 hi = lds_read_tr16(p + 16 * pitch);
  u32x4 r;
  r.x = lo.x; r.y = lo.y; r.z = hi.x; r.w = hi.y;
  return r;
}

// Reductions over the 4 lanes that share n (lanes n, n + 16, n + 32, n + 48), every lane receiving the result.  The two
// exchanges are lane-swap VALU instructions (rows 2,3 <-> rows 0,1, then odd rows <-> even rows), not LDS permutes:
// those queue behind the operand reads of every wave on the CU.
DLT_DEV void wave_rows_swap32(float v, float& a, float& b) {
  typedef unsigned pair_t __attribute__((ext_vector_type(2)));
  const unsigned u = __builtin_bit_cast(unsigned, v);
  const pair_t r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  a = __builtin_bit_cast(float, (unsigned)r.x); b = __builtin_bit_cast(float, (unsigned)r.y);
}
DLT_DEV void wave_rows_swap16(float v, float& a, float& b) {
  typedef unsigned pair_t __attribute__((ext_vector_type(2)));
  const unsigned u = __builtin_bit_cast(unsigned, v);
  const pair_t r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  a = __builtin_bit_cast(float, (unsigned)r.x); b = __builtin_bit_cast(float, (unsigned)r.y);
}
DLT_DEV float wave_max4(float v) {
  float a, b;
  wave_rows_swap32(v, a, b);
  v = fmaxf(a, b);
  wave_rows_swap16(v, a, b);
  return fmaxf(a, b);
}
DLT_DEV float wave_sum4(float v) {
  float a, b;
  wave_rows_swap32(v, a, b);
  v = a + b;
  wave_rows_swap16(v, a, b);
  return a + b;
}

// ---- global <-> register moves of 8 consecutive head dims -------------------------------
template <typename TIO, typename CT> struct Io;

// Stores of results that this kernel does not read again are issued as streaming ("nontemporal") stores: they are
// written through towards memory while the kernel still runs.  A plain store leaves its line dirty in the L2 of its XCD
// until the write-back at the end of the kernel, which the next kernel of the stream waits for: measured between two
// kernels of one stream, 1.1 us when the first writes nothing at its end, 5.0 us after 8 MB, 12.7 us after 26 MB.
DLT_DEV void store_stream16(void* p, const u32x4& v) { __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(p)); }
DLT_DEV void store_stream8(void* p, const u32x2& v) { __builtin_nontemporal_store(v, reinterpret_cast<u32x2*>(p)); }
DLT_DEV void store_stream4(float* p, float v) { __builtin_nontemporal_store(v, p); }
DLT_DEV void store_stream16f(float* p, float a, float b, float c, float d) { __builtin_nontemporal_store(f32x4{a, b, c, d}, reinterpret_cast<f32x4*>(p)); }

template <typename T> struct Io<T, T> {  // 2-byte element, same compute type
  static DLT_DEV u32x4 load8(const T* p, bool vec, int64_t sd, int nvalid) {
    if (vec) return *reinterpret_cast<const u32x4*>(p);
    unsigned short e[8];
#pragma unroll
    for (int j = 0; j < 8; j++) e[j] = j < nvalid ? __builtin_bit_cast(unsigned short, p[j * sd]) : (unsigned short)0;
    u32x4 r;
    r.x = e[0] | ((unsigned)e[1] << 16); r.y = e[2] | ((unsigned)e[3] << 16);
    r.z = e[4] | ((unsigned)e[5] << 16); r.w = e[6] | ((unsigned)e[7] << 16);
    return r;
  }
  static DLT_DEV void store8(T* p, const float* v, bool vec, int64_t sd, int nvalid) {
    if (vec) {
      u32x4 r;
      r.x = pack2<T>(v[0], v[1]); r.y = pack2<T>(v[2], v[3]); r.z = pack2<T>(v[4], v[5]); r.w = pack2<T>(v[6], v[7]);
      store_stream16(p, r);
    } else {
#pragma unroll
      for (int j = 0; j < 8; j++) if (j < nvalid) p[j * sd] = (T)v[j];
    }
  }
};

template <> struct Io<float, bf16_t> {  // fp32 in HBM, bf16 arithmetic
  static DLT_DEV u32x4 load8(const float* p, bool vec, int64_t sd, int nvalid) {
    float f[8];
    if (vec) {
      const float4 a = reinterpret_cast<const float4*>(p)[0], b = reinterpret_cast<const float4*>(p)[1];
      f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w; f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
    } else {
#pragma unroll
      for (int j = 0; j < 8; j++) f[j] = j < nvalid ? p[j * sd] : 0.f;
    }
    u32x4 r;
    r.x = pack2<bf16_t>(f[0], f[1]); r.y = pack2<bf16_t>(f[2], f[3]);
    r.z = pack2<bf16_t>(f[4], f[5]); r.w = pack2<bf16_t>(f[6], f[7]);
    return r;
  }
  static DLT_DEV void store8(float* p, const float* v, bool vec, int64_t sd, int nvalid) {
    if (vec) {
      store_stream16f(p, v[0], v[1], v[2], v[3]);
      store_stream16f(p + 4, v[4], v[5], v[6], v[7]);
    } else {
#pragma unroll
      for (int j = 0; j < 8; j++) if (j < nvalid) p[j * sd] = v[j];
    }
  }
};

template <typename CT> DLT_DEV void unpack8(u32x4 r, float* f) {
  f[0] = unpack_lo<CT>(r.x); f[1] = unpack_hi<CT>(r.x); f[2] = unpack_lo<CT>(r.y); f[3] = unpack_hi<CT>(r.y);
  f[4] = unpack_lo<CT>(r.z); f[5] = unpack_hi<CT>(r.z); f[6] = unpack_lo<CT>(r.w); f[7] = unpack_hi<CT>(r.w);
}
template <typename CT> DLT_DEV u32x4 pack8(const float* f) {
  u32x4 r;
  r.x = pack2<CT>(f[0], f[1]); r.y = pack2<CT>(f[2], f[3]); r.z = pack2<CT>(f[4], f[5]); r.w = pack2<CT>(f[6], f[7]);
  return r;
}

// ---- rotary encoding applied to one 8-dim chunk -----------------------------------------
// y = self * cos -/+ partner * sin with each product rounded before the add: the evaluation
// order of the standalone kernel and of the eager reference (src/fused_rope2d.py:221-222).
DLT_DEV float rope_mix(float self, float partner, float c, float s, bool is_x0) {
#pragma clang fp contract(off)
  const float a = self * c, b = partner * s;
  return is_x0 ? a - b : b + a;
}

// The same value with the sign of the sine decided once per chunk instead of once per element:
// a - b == a + (-b) and b + a == a + b bit for bit, and (-s) * x == -(s * x), so
// rope_mix(self, partner, c, s, is_x0) == rope_mix_signed(self, partner, c, is_x0 ? -s : s).
DLT_DEV unsigned rope_sign_mask(bool is_x0, bool inverse) { return is_x0 != inverse ? 0x80000000u : 0u; }
DLT_DEV float rope_mix_signed(float self, float partner, float c, float s_raw, unsigned sign_mask) {
#pragma clang fp contract(off)
  const float s = __uint_as_float(__float_as_uint(s_raw) ^ sign_mask);
  const float a = self * c, b = partner * s;
  return a + b;
}

// Per-thread rotary context for a fixed 8-dim chunk index `c` (dims 8c .. 8c+7).
struct RopeChunk {
  int mode;      // 0: chunk not rotated, 1: whole-chunk fast path (R % 8 == 0), 2: per-element path
  int axis;      // fast path: 0 row, 1 column
  int is_x0;     // fast path: chunk holds the first element of each pair
  int partner_c; // fast path: chunk index holding the pair partners
  int tab_off;   // fast path: float offset of this chunk's (cos, sin) pairs inside a table row
};

DLT_DEV RopeChunk rope_chunk_setup(const RopeDev& r, int c, bool vec) {
  RopeChunk rc;
  rc.mode = 0; rc.axis = 0; rc.is_x0 = 0; rc.partner_c = 0; rc.tab_off = 0;
  if (!r.enabled || r.R == 0 || 8 * c >= 4 * r.R) return rc;
  if (vec && (r.R & 7) == 0) {
    const int r8 = r.R >> 3;
    // r8 is wave-uniform; the usual sizes are powers of two, where a shift replaces the per-lane division
    const int region = (r8 & (r8 - 1)) == 0 ? c >> __builtin_ctz(r8) : c / r8;
    const int ci = c - region * r8;
    rc.mode = 1;
    rc.axis = region >> 1;
    rc.is_x0 = (region & 1) == 0;
    rc.partner_c = rc.is_x0 ? c + r8 : c - r8;
    rc.tab_off = 16 * ci;
  } else {
    rc.mode = 2;
  }
  return rc;
}

DLT_DEV const float* rope_table_row(const RopeDev& r, int axis, int32_t id, bool& rotated) {
  int pos = axis == 0 ? dlt_rope_row(id) : dlt_rope_col(id);
  rotated = pos >= 0;
  pos = dlt_imax(0, dlt_imin(pos, (axis == 0 ? r.row_len : r.col_len) - 1));
  return axis == 0 ? r.row_cs + (int64_t)pos * r.rs0 : r.col_cs + (int64_t)pos * r.cs0;
}

// Rotate the 8 values `self` (dims 8c..8c+7 of one token).  `partner(d)` returns the value
// of dim d of the same token (only called for pair partners).
template <typename PartnerFn>
DLT_DEV void rope_apply8(const RopeDev& r, const RopeChunk& rc, int c, int32_t id, float* self, const float* partner8,
                         PartnerFn partner) {
  if (rc.mode == 1) {
    bool rotated;
    const float* tab = rope_table_row(r, rc.axis, id, rotated) + rc.tab_off;
    if (!rotated) return;
    const unsigned sm = rope_sign_mask(rc.is_x0 != 0, r.inverse != 0);
#pragma unroll
    for (int j = 0; j < 8; j++) self[j] = rope_mix_signed(self[j], partner8[j], tab[2 * j], tab[2 * j + 1], sm);
  } else if (rc.mode == 2) {
#pragma unroll
    for (int j = 0; j < 8; j++) {
      const int d = 8 * c + j;
      if (d >= 4 * r.R) continue;
      const int region = d / r.R, i = d - region * r.R;
      bool rotated;
      const float* tab = rope_table_row(r, region >> 1, id, rotated) + 2 * i;
      if (!rotated) continue;
      const bool is_x0 = (region & 1) == 0;
      const float pv = partner(is_x0 ? d + r.R : d - r.R);
      const float sn = r.inverse ? -tab[1] : tab[1];
      self[j] = rope_mix(self[j], pv, tab[0], sn, is_x0);
    }
  }
}

// ---- token -> element offset inside one (batch, head) slab --------------------------------------
// A plain stride (tokens n * sn apart) or, for image-layout tensors, the pixel map of DltTokMap.
struct TokAddr {
  int64_t sn, sy;
  const DltTokMap* tm;
  DLT_DEV int64_t operator()(int64_t t) const {
    if (!tm->img) return t * sn;
    uint32_t y, x;
    dlt_token_pixel(*tm, (uint32_t)t, y, x);
    return (int64_t)y * sy + (int64_t)x * sn;
  }
};
DLT_DEV TokAddr tok_addr(const int64_t (&s)[5], const DltTokMap& tm) { return TokAddr{s[2], s[4], &tm}; }
DLT_DEV int64_t tok_offset(int64_t sn, int64_t t) { return t * sn; }
DLT_DEV int64_t tok_offset(const TokAddr& a, int64_t t) { return a(t); }

// ---- HBM -> LDS staging of `nrows` token rows of D head dims -------------------------------
// LDS tile: row-major, `pitch` bytes per row, compute-type elements.  tok(row) gives the token
// index inside the [N, D] slab at `base` (or -1: the row is zero-filled).  Dims >= dact are
// zero-filled.  With `rope.enabled` rows are rotated on the way in (q and k of the fused call).
template <typename TIO, typename CT, int D, typename TokFn, typename SN>
DLT_DEV void stage_tile(char* s, int pitch, const TIO* base, const SN& sn, int64_t sd, int dact, bool vec, int nrows,
                        TokFn tok, const RopeDev& rope, int tid) {
  constexpr int CH = D / 8;
  constexpr int RSTEP = 256 / CH;
  const int c = tid % CH;
  const RopeChunk rc = rope_chunk_setup(rope, c, vec);
  const int nvalid = dlt_imin(8, dact - 8 * c);
  for (int row = tid / CH; row < nrows; row += RSTEP) {
    const int64_t t = tok(row);
    u32x4 val = {0u, 0u, 0u, 0u};
    if (t >= 0 && nvalid > 0) {
      const TIO* p = base + tok_offset(sn, t);
      val = Io<TIO, CT>::load8(p + (int64_t)8 * c * sd, vec, sd, nvalid);
      if (rc.mode != 0) {
        float self[8], partner8[8];
        unpack8<CT>(val, self);
        if (rc.mode == 1) {
          const u32x4 pr = Io<TIO, CT>::load8(p + (int64_t)8 * rc.partner_c * sd, vec, sd, 8);
          unpack8<CT>(pr, partner8);
        }
        // operands are rounded to the compute type first, as the standalone op sees them
        rope_apply8(rope, rc, c, rope.idx[t], self, partner8,
                    [&](int d) { return (float)(CT)(float)p[(int64_t)d * sd]; });
        val = pack8<CT>(self);
      }
    }
    lds_write16(s + row * pitch + c * 16, val);
  }
}

// fp32 tensors whose values enter a score product: every value is staged as TWO bf16 numbers, hi = bf16(x) and
// lo = bf16(x - hi), hi at the row's start and lo D * 2 bytes further on (row pitch >= 4 D bytes).  The products
// hi * hi + hi * lo + lo * hi then carry x to about 16 significant bits (the reference casts these operands to fp16, 11
// bits: src/tiled_swa.py:111-112); a single bf16 keeps 8, which shows in the softmax when the logits are large.  The
// rotation, when fused, is applied to the fp32 values before the split.
template <int D, typename TokFn, typename SN>
DLT_DEV void stage_tile_split(char* s, int pitch, const float* base, const SN& sn, int64_t sd, int dact, bool vec, int nrows,
                              TokFn tok, const RopeDev& rope, int tid) {
  constexpr int CH = D / 8;
  constexpr int RSTEP = 256 / CH;
  const int c = tid % CH;
  const RopeChunk rc = rope_chunk_setup(rope, c, vec);
  const int nvalid = dlt_imin(8, dact - 8 * c);
  auto load8f = [&](const float* p, int nv, float* f) {
    if (vec) {
      const float4 a = reinterpret_cast<const float4*>(p)[0], b = reinterpret_cast<const float4*>(p)[1];
      f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w; f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
    } else {
#pragma unroll
      for (int j = 0; j < 8; j++) f[j] = j < nv ? p[j * sd] : 0.f;
    }
  };
  for (int row = tid / CH; row < nrows; row += RSTEP) {
    const int64_t t = tok(row);
    float self[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (t >= 0 && nvalid > 0) {
      const float* p = base + tok_offset(sn, t);
      load8f(p + (int64_t)8 * c * sd, nvalid, self);
      if (rc.mode != 0) {
        float partner8[8];
        if (rc.mode == 1) load8f(p + (int64_t)8 * rc.partner_c * sd, 8, partner8);
        rope_apply8(rope, rc, c, rope.idx[t], self, partner8, [&](int d) { return p[(int64_t)d * sd]; });
      }
    }
    float lo[8];
#pragma unroll
    for (int j = 0; j < 8; j++) lo[j] = self[j] - (float)(bf16_t)self[j];
    lds_write16(s + row * pitch + c * 16, pack8<bf16_t>(self));
    lds_write16(s + row * pitch + D * 2 + c * 16, pack8<bf16_t>(lo));
  }
}

// q / k tiles: plain staging, or the hi + lo pair for fp32 tensors (row pitch DK * 4 + 16 then)
template <typename TIO, typename CT, int D, typename TokFn, typename SN>
DLT_DEV void stage_tile_qk(char* s, int pitch, const TIO* base, const SN& sn, int64_t sd, int dact, bool vec, int nrows,
                           TokFn tok, const RopeDev& rope, int tid) {
  if constexpr (sizeof(TIO) == 4) stage_tile_split<D>(s, pitch, base, sn, sd, dact, vec, nrows, tok, rope, tid);
  else stage_tile<TIO, CT, D>(s, pitch, base, sn, sd, dact, vec, nrows, tok, rope, tid);
}

// ---- LDS -> HBM store of an output tile ------------------------------------------------------
// TL: element type of the LDS tile (the output type, or float for fp32 outputs).
template <typename TO, typename TL, int D, typename TokFn, typename SN>
DLT_DEV void store_tile(const char* s, int pitch, TO* base, const SN& sn, int64_t sd, int dact, bool vec, int nrows,
                        TokFn tok, const RopeDev& rope, int tid) {
  constexpr int CH = D / 8;
  constexpr int RSTEP = 256 / CH;
  typedef typename ComputeOf<TO>::type CT;
  const int c = tid % CH;
  const RopeChunk rc = rope_chunk_setup(rope, c, true);
  const int nvalid = dlt_imin(8, dact - 8 * c);
  if (nvalid <= 0) return;
  for (int row = tid / CH; row < nrows; row += RSTEP) {
    const int64_t t = tok(row);
    if (t < 0) continue;
    const TL* lrow = reinterpret_cast<const TL*>(s + row * pitch);
    float v[8], partner8[8];
#pragma unroll
    for (int j = 0; j < 8; j++) v[j] = (float)lrow[8 * c + j];
    if (rc.mode != 0) {
      if (rc.mode == 1) {
#pragma unroll
        for (int j = 0; j < 8; j++) partner8[j] = (float)lrow[8 * rc.partner_c + j];
      }
      rope_apply8(rope, rc, c, rope.idx[t], v, partner8, [&](int d) { return (float)lrow[d]; });
    }
    Io<TO, CT>::store8(base + tok_offset(sn, t) + (int64_t)8 * c * sd, v, vec, sd, nvalid);
  }
}

// LDS tile element type used for an output element type
template <typename TO> struct TileOf { typedef TO type; };

// workgroup id -> logical id such that each XCD (8 of them, workgroups are dealt round-robin)
// walks a contiguous range of logical ids: neighbouring tiles of one head share an L2.
DLT_DEV int xcd_remap(int bid, int nblocks) {
  const int per = nblocks >> 3;
  if (per == 0 || bid >= per * 8) return bid;
  return (bid & 7) * per + (bid >> 3);
}

// Per-launch plan computed on the host (attn_launch.hip).
struct AttnPlan {
  int32_t rowfit;      // 1: a chunk holds whole halo rows, each wave walks from its own x origin
  int32_t chunk_rows;  // halo rows per chunk (rowfit) else 1
  int32_t chunk_x;     // tokens staged per halo row (LDS row pitch in tokens)
  int32_t nblk_x;      // workgroups per grid row on the own side
  int32_t off_a, off_b, off_c, off_d;  // LDS byte offsets of the halo buffers
  int32_t lds_bytes;
};

// Which tokens a workgroup / wave / lane owns and which tokens of the other side they touch.
// "Own" tokens are queries for the forward and dQ kernels and keys for the dK/dV kernel
// (TRANSPOSE); the "halo" is the set of tokens of the other side inside the window of any
// own token: grid rows [rlo, rhi] (the same for the whole workgroup, which owns tokens of a
// single grid row) and x in [X0, X1).  Per lane the window of own token n is the x interval
// [xlo, xlo + span); per 16-token patch and per wave the union / intersection of those
// intervals are wave-uniform and steer which 32-token blocks are visited and whether a
// block needs the element mask at all.
template <int NP, bool TRANSPOSE>
struct TileCtx {
  int b, h, r_own, x0, xlast;
  int rlo, rhi, X0, X1;
  int wfirst, wxlo, wxhi;
  int xlo[NP], span[NP];
  int pxlo[NP], pxhi[NP], pin_lo[NP], pin_hi[NP];
  int64_t own_tok0;
  int XL_own, XL_halo;

  static DLT_DEV void range(const DltGeom& G, int r, int x, int& rl, int& rh, int& xl, int& xh) {
    if (TRANSPOSE) dlt_query_range(G, r, x, rl, rh, xl, xh);
    else dlt_key_range(G, r, x, rl, rh, xl, xh);
  }

  DLT_DEV void init(const DltGeom& G, const AttnPlan& plan, int H, int wave, int n) {
    constexpr int OWN = 64 * NP;
    XL_own = TRANSPOSE ? G.XLk : G.XLq;
    XL_halo = TRANSPOSE ? G.XLq : G.XLk;
    const int lin = xcd_remap(blockIdx.x, gridDim.x);
    const int per_bh = G.TR * plan.nblk_x;
    const int bh = lin / per_bh;
    const int rem = lin - bh * per_bh;
    r_own = rem / plan.nblk_x;
    x0 = (rem - r_own * plan.nblk_x) * OWN;
    b = bh / H;
    h = bh - b * H;
    xlast = dlt_imin(x0 + OWN, XL_own) - 1;
    own_tok0 = (int64_t)r_own * XL_own + x0;
    int t0, t1;
    range(G, r_own, x0, rlo, rhi, X0, t0);
    range(G, r_own, xlast, t0, t1, t0, X1);
    wfirst = x0 + wave * 16 * NP;
    wxlo = wxhi = 0;
#pragma unroll
    for (int p = 0; p < NP; p++) {
      const int xq = wfirst + 16 * p + n;
      int a0, a1, lo = 0, hi = 0;
      if (xq <= xlast) range(G, r_own, xq, a0, a1, lo, hi);
      xlo[p] = lo; span[p] = hi - lo;
      const int pf = wfirst + 16 * p, pl = dlt_imin(pf + 15, xlast);
      pxlo[p] = pxhi[p] = 0; pin_lo[p] = 0x7fffffff; pin_hi[p] = 0;
      if (pf <= xlast) {
        int l0, h0, l1, h1;
        range(G, r_own, pf, a0, a1, l0, h0);
        range(G, r_own, pl, a0, a1, l1, h1);
        pxlo[p] = l0; pxhi[p] = h1;
        if (pl == pf + 15) { pin_lo[p] = l1; pin_hi[p] = h0; }
        if (p == 0) wxlo = l0;
        wxhi = h1;
      }
    }
  }
  DLT_DEV int64_t own_token(int row) const { return x0 + row <= xlast ? own_tok0 + row : (int64_t)-1; }
  DLT_DEV bool patch_skips(int p, int kx0) const { return kx0 >= pxhi[p] || kx0 + 32 <= pxlo[p]; }
  DLT_DEV bool patch_needs_mask(int p, int kx0) const { return !(kx0 >= pin_lo[p] && kx0 + 32 <= pin_hi[p]); }
  // element (mb, i) of a 32-token block at kx0, held by lane group g: token x = kx0 + 16 mb + 4 g + i
  DLT_DEV bool valid(int p, int kx0, int g, int mb, int i) const {
    return (unsigned)(kx0 + 16 * mb + 4 * g + i - xlo[p]) < (unsigned)span[p];
  }
};
