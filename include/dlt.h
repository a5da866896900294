/*
 * dlt.h - C ABI of libdlt_hip.so: the MI355X (gfx950) attention hot path of dl_templates.
 *
 * Conventions shared by every entry point
 *   - returns DLT_OK (0) or a DLT_ERR_* code; dlt_last_error() gives the message of the
 *     last failing call made by the calling thread (thread-local, never NULL);
 *   - every data pointer is a DEVICE pointer owned by the caller; the library allocates
 *     no device memory, never synchronises and keeps no state between calls (the optional
 *     timing facility below is the one exception: a thread-local list of host-side event
 *     handles), so calls are re-entrant (forward on the caller thread, backward on the
 *     autograd thread);
 *   - strides are in ELEMENTS (int64), tensors are [B, H, N, D] unless said otherwise;
 *   - `stream` is a hipStream_t (NULL = the default stream); work is only enqueued;
 *   - arguments are validated on the host before anything is launched: a call that
 *     returns an error has launched nothing.
 */
#ifndef DLT_H
#define DLT_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DLT_OK 0
#define DLT_ERR_INVALID 1     /* bad shape / pointer / stride / enum            */
#define DLT_ERR_UNSUPPORTED 2 /* valid request the kernels do not cover (yet)   */
#define DLT_ERR_LAUNCH 3      /* the HIP runtime reported an error on launch    */

/* element type of q/k/v/o and their gradients; arithmetic is bf16 (fp16 for DLT_FP16)
 * MFMA with fp32 accumulation.  fp32 q and k enter the score products as hi + lo bf16 pairs
 * (about 16 significant bits; the reference casts to fp16, src/tiled_swa.py:111-112), fp32 v
 * and dO are rounded to bf16 when staged. */
typedef enum { DLT_BF16 = 0, DLT_FP16 = 1, DLT_FP32 = 2 } dlt_dtype_t;

const char* dlt_last_error(void);
int dlt_version(void);

/* ---- 2D rotary encoding -------------------------------------------------------------
 * Per-token packed index and the two cos/sin tables, exactly the operands of
 * RotaryPE2D.forward (src/fused_rope2d.py:126-141): idx[n] = (row << 16) | col,
 * an axis whose signed 16-bit value is negative is not rotated (:40-45, :215-219);
 * tables are fp32 [len, R, 2] with (cos, sin) innermost (:22-23, :238-240) and
 * `*_stride0` elements between table rows (cs_stride0, :29,141).  Indices are clamped
 * to [0, len-1] instead of reading out of bounds. */
typedef struct {
  const int32_t* idx;
  const float* row_cs;
  const float* col_cs;
  int64_t row_cs_stride0;
  int64_t col_cs_stride0;
  int32_t n_rdim;  /* R: dims [0,R)x[R,2R) use the row angle, [2R,3R)x[3R,4R) the column angle */
  int32_t row_len; /* number of rows of row_cs */
  int32_t col_len;
} dlt_rope_t;

/* In-place rotation of x[B', N, C] (any strides).  Replaces rope2d_fwd_kernel
 * (src/fused_rope2d.py:24-72) when inverse == 0 and rope2d_bwd_kernel (:74-122, the
 * transposed rotation applied to a gradient) when inverse != 0.  No-PE semantics follow
 * rope2d_ref (:204-225): an unrotated axis leaves its dims bit-identical. */
int dlt_rope2d(void* x, const int64_t x_strides[3], int64_t n_batch, int64_t n_tokens, int64_t n_dim,
               const dlt_rope_t* rope, int inverse, int dtype, void* stream);

/* The same rotation applied to two tensors (q and k of one attention call) in ONE launch;
 * both share idx/tables, N and C.  Replaces two back-to-back RotaryPE2D launches
 * (README.md:11 composition; src/fused_rope2d.py:197-201 called once per tensor). */
int dlt_rope2d_pair(void* x0, const int64_t x0_strides[3], int64_t n_batch0,
                    void* x1, const int64_t x1_strides[3], int64_t n_batch1,
                    int64_t n_tokens, int64_t n_dim,
                    const dlt_rope_t* rope, int inverse, int dtype, void* stream);

/* Debug export: bits[n] = (row >= 0) | (col >= 0) << 1, computed by the SAME device code
 * the rotation kernels use to decode idx (src/fused_rope2d.py:40-45). */
int dlt_rope_pe_mask(const int32_t* idx, int64_t n_tokens, uint8_t* bits, void* stream);

/* ---- tiled 2D sliding-window attention -------------------------------------------------
 * Scalars of TiledSwa.forward (src/tiled_swa.py:604): token n = (r * t_width + c) * b_size + s;
 * query tile (r, c) attends kv tile (r', c') iff |r-r'| <= row_size and |c-c'| <= col_size,
 * truncated at the grid border (:701-713). */
typedef struct {
  int32_t B, H;
  int32_t b_size, t_height, t_width, row_size, col_size;
  int32_t dk, dv; /* q/k head dim, v/o head dim: 1..256 each (larger: DLT_ERR_UNSUPPORTED) */
  float sm_scale; /* must be finite (else DLT_ERR_INVALID); any sign is accepted as in the reference, which scales
                     before taking the row max: the tuned kernels keep the max of the raw scores and take positive
                     scales only, zero and negative scales run on the generic kernels */
  int32_t dtype;  /* dlt_dtype_t */
} dlt_swa_shape_t;

/* Forward: o = softmax_window(q k^T * sm_scale) v, lse2 = log2 sum exp2(.) in log2 units.
 * Replaces tiled_swa_fwd_kernel / tiled_swa_fwd_large_kernel (src/tiled_swa.py:15-133,
 * :142-244) and the launch code of TiledSwa.forward (:605-637).  lse2 is fp32 [B, H, N]
 * (the reference stores fp16 `m`, :608).  When `rope` is not NULL the rotation of
 * dlt_rope2d is applied to q and k as they are loaded (q, k in HBM stay untouched);
 * the result equals RotaryPE2D on q and k followed by the plain forward. */
int dlt_swa_fwd(const void* q, const int64_t q_strides[4], const void* k, const int64_t k_strides[4],
                const void* v, const int64_t v_strides[4], void* o, const int64_t o_strides[4],
                float* lse2, const int64_t lse_strides[3],
                const dlt_swa_shape_t* shape, const dlt_rope_t* rope, void* stream);

/* Backward: replaces tiled_swa_bwd_preprocess_kernel (src/tiled_swa.py:253-282) and
 * tiled_swa_bwd_large_kernel_decoupled_q (:407-562) plus TiledSwa.backward (:649-689).
 * `delta` is caller-provided fp32 scratch with the strides of lse2.  dq/dk/dv are written
 * in the element type of q/k/v (the reference accumulates dq in an fp32 tensor, :656).
 * With `rope` the inputs q, k are the UN-rotated tensors and dq, dk are returned with
 * respect to them (transposed rotation applied on store). */
int dlt_swa_bwd(const void* q, const int64_t q_strides[4], const void* k, const int64_t k_strides[4],
                const void* v, const int64_t v_strides[4], const void* o, const int64_t o_strides[4],
                const void* d_o, const int64_t do_strides[4],
                const float* lse2, float* delta, const int64_t lse_strides[3],
                void* dq, const int64_t dq_strides[4], void* dk, const int64_t dk_strides[4],
                void* dv, const int64_t dv_strides[4],
                const dlt_swa_shape_t* shape, const dlt_rope_t* rope, void* stream);

/* dlt_swa_bwd without the `delta` argument: the fp32 scratch lives in a buffer inside the library
 * (one static device array per GPU, DLT_NOALLOC_MAX_DELTA floats = 4 MiB, held until the process
 * ends) and the call allocates nothing: no hipMalloc / hipFree, no allocating library routine.
 * No counterpart in the reference (TiledSwa.backward allocates delta with torch, src/tiled_swa.py:663);
 * it is for callers that cannot allocate: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  The scratch is addressed with `lse_strides`, so the call is
 * rejected (DLT_ERR_INVALID, nothing launched) when a stride is negative or the largest offset
 * (B-1) s0 + (H-1) s1 + (N-1) s2 reaches DLT_NOALLOC_MAX_DELTA.  Every call on a GPU shares that GPU's
 * buffer and overwrites all of it that it reads: calls that overlap in time on one GPU (two streams,
 * two threads) race and must be serialised by the caller; results equal dlt_swa_bwd's bit for bit.
 * The first call on a device with a given kernel also resolves the scratch symbol and raises that kernel's
 * LDS limit (host-side driver calls, no device memory): make one call with the shapes to be used outside any
 * stream capture before recording the call into a HIP graph. */
#define DLT_NOALLOC_MAX_DELTA (1 << 20)
int dlt_swa_bwd_noalloc(const void* q, const int64_t q_strides[4], const void* k, const int64_t k_strides[4],
                        const void* v, const int64_t v_strides[4], const void* o, const int64_t o_strides[4],
                        const void* d_o, const int64_t do_strides[4],
                        const float* lse2, const int64_t lse_strides[3],
                        void* dq, const int64_t dq_strides[4], void* dk, const int64_t dk_strides[4],
                        void* dv, const int64_t dv_strides[4],
                        const dlt_swa_shape_t* shape, const dlt_rope_t* rope, void* stream);

/* The fused call with the rotated tensors kept: forward as dlt_swa_fwd with `rope`, which in addition
 * stores the rotated q and k into q_rot / k_rot (shapes and element type of q / k, own strides; must
 * not alias q, k or each other).  These are the tensors RotaryPE2D leaves behind in the reference's
 * composition (it rotates q and k in place and autograd saves the rotated tensors,
 * src/fused_rope2d.py:143-147).  On token grids the attention kernel itself writes them (each
 * workgroup its own tokens); otherwise q and k are rotated out of place first and the plain operator
 * runs on the result. */
int dlt_swa_fwd_rot(const void* q, const int64_t q_strides[4], const void* k, const int64_t k_strides[4],
                    const void* v, const int64_t v_strides[4], void* o, const int64_t o_strides[4],
                    float* lse2, const int64_t lse_strides[3],
                    void* q_rot, const int64_t q_rot_strides[4], void* k_rot, const int64_t k_rot_strides[4],
                    const dlt_swa_shape_t* shape, const dlt_rope_t* rope, void* stream);

/* Backward of the fused call from the saved rotated tensors: q_rot / k_rot are read as they are (no
 * rotation in the tile loads: every halo token would be rotated again by each workgroup that stages
 * it); dq and dk get the transposed rotation as they are stored (rope2d_bwd_kernel,
 * src/fused_rope2d.py:74-122, folded into the epilogue), so they are gradients with respect to the
 * UN-rotated q and k, exactly as dlt_swa_bwd with `rope` returns them. */
int dlt_swa_bwd_rot(const void* q_rot, const int64_t q_rot_strides[4], const void* k_rot, const int64_t k_rot_strides[4],
                    const void* v, const int64_t v_strides[4], const void* o, const int64_t o_strides[4],
                    const void* d_o, const int64_t do_strides[4],
                    const float* lse2, float* delta, const int64_t lse_strides[3],
                    void* dq, const int64_t dq_strides[4], void* dk, const int64_t dk_strides[4],
                    void* dv, const int64_t dv_strides[4],
                    const dlt_swa_shape_t* shape, const dlt_rope_t* rope, void* stream);

/* Debug export: mask[i * T + j] = 1 iff query tile i attends kv tile j (T = t_height *
 * t_width, row-major tiles), produced on the device by the SAME window routine the
 * attention kernels call (src/tiled_swa.py:76-79, :97-100, :212-214, :701-713). */
int dlt_swa_neighbors(int32_t t_height, int32_t t_width, int32_t row_size, int32_t col_size,
                      uint8_t* mask, void* stream);

/* ---- the same operator on image-layout tensors ----------------------------------------------
 * q, k, v, o and the gradients are images [B, IH, IW, heads, D] (five element strides each, all
 * non-negative) with IH = t_height * bh and IW = t_width * bw; a tile is a block of bh x bw pixels,
 * shape->b_size must equal bh * bw, and pixel (y, x) is token
 *     n = ((y / bh * t_width + x / bw) * bh + y % bh) * bw + x % bw
 * of the tile-major order dlt_swa_fwd uses: exactly the permutation the reference's demo applies
 * around the operator to move between the two layouts (reshape -> permute(0, 2, 4, 3, 5, 1, 6) ->
 * reshape, src/tiled_swa.py:753-755).  The kernels address pixels directly, so that pass over
 * q, k, v (and over o and the three gradients) disappears.  lse2 / delta stay fp32 [B, heads, N] in
 * tile-major token order, and `rope->idx` is indexed by that token number as well.  A call whose
 * tiles are single pixels and whose pixel rows lie t_width pixel columns apart is run as the plain
 * [B, H, N, D] view it is. */
typedef struct {
  int32_t bh, bw; /* pixels per tile, vertically and horizontally */
} dlt_swa_tile_t;

int dlt_swa_fwd_image(const void* q, const int64_t q_strides[5], const void* k, const int64_t k_strides[5],
                      const void* v, const int64_t v_strides[5], void* o, const int64_t o_strides[5],
                      float* lse2, const int64_t lse_strides[3], const dlt_swa_shape_t* shape,
                      const dlt_swa_tile_t* tile, const dlt_rope_t* rope, void* stream);

int dlt_swa_bwd_image(const void* q, const int64_t q_strides[5], const void* k, const int64_t k_strides[5],
                      const void* v, const int64_t v_strides[5], const void* o, const int64_t o_strides[5],
                      const void* d_o, const int64_t do_strides[5],
                      const float* lse2, float* delta, const int64_t lse_strides[3],
                      void* dq, const int64_t dq_strides[5], void* dk, const int64_t dk_strides[5],
                      void* dv, const int64_t dv_strides[5], const dlt_swa_shape_t* shape,
                      const dlt_swa_tile_t* tile, const dlt_rope_t* rope, void* stream);

/* Debug export: offsets[n] = y * stride_y + x * stride_x for the pixel (y, x) of token n, n in
 * [0, t_height * t_width * bh * bw), computed on the device by the SAME token -> pixel routine the
 * attention kernels use (the inverse of the permutation of src/tiled_swa.py:753-755). */
int dlt_swa_image_offsets(int32_t t_height, int32_t t_width, int32_t bh, int32_t bw, int64_t stride_y,
                          int64_t stride_x, int64_t* offsets, void* stream);

/* ---- flash attention with separate qk / vo head dims -----------------------------------
 * q [B,H,Lq,dk], k [B,H,Lk,dk], v [B,H,Lk,dv], o [B,H,Lq,dv], lse2 fp32 [B,H,Lq].
 * Replaces _attn_fwd (src/flash_attn.py:81-172) and _attention.forward (:455-490); unlike
 * the reference (single N_CTX, :479) Lq != Lk is accepted when causal == 0.
 * Every dk, dv in 1..256 is computed; the tuned kernels take 2-byte element types with dk, dv
 * multiples of 8 up to 128 and 16-byte aligned rows of unit last stride, other calls run on
 * generic kernels several times slower (a caller may zero-pad dk and dv to the next multiple
 * of 8: padded dims of q, k add nothing to the scores, padded dims of v give zero outputs). */
typedef struct {
  int32_t B, H, Lq, Lk;
  int32_t dk, dv;
  float sm_scale;
  int32_t causal;
  int32_t dtype;
} dlt_flash_shape_t;

int dlt_flash_fwd(const void* q, const int64_t q_strides[4], const void* k, const int64_t k_strides[4],
                  const void* v, const int64_t v_strides[4], void* o, const int64_t o_strides[4],
                  float* lse2, const int64_t lse_strides[3],
                  const dlt_flash_shape_t* shape, void* stream);

/* Replaces _attn_bwd_preprocess / _attn_bwd (src/flash_attn.py:186-449) and
 * _attention.backward (:493-538); no host-side pre-scaling pass over k (:509-510) and no
 * N_CTX % 128 requirement (:512). */
int dlt_flash_bwd(const void* q, const int64_t q_strides[4], const void* k, const int64_t k_strides[4],
                  const void* v, const int64_t v_strides[4], const void* o, const int64_t o_strides[4],
                  const void* d_o, const int64_t do_strides[4],
                  const float* lse2, float* delta, const int64_t lse_strides[3],
                  void* dq, const int64_t dq_strides[4], void* dk, const int64_t dk_strides[4],
                  void* dv, const int64_t dv_strides[4],
                  const dlt_flash_shape_t* shape, void* stream);

/* ---- per-kernel timing (measurement aid) ---------------------------------------------------
 * Counterpart of the reference's triton.testing.do_bench calls (src/tiled_swa.py:765-774,
 * src/flash_attn.py:592,606), at kernel granularity.  While enabled for the calling thread,
 * every kernel the library launches is bracketed by a pair of hipEvents recorded on the
 * launch stream.  dlt_timing_collect waits for the recorded events, writes up to `max`
 * records in launch order, stores the number available in *n and clears the list.
 * Enabling creates events lazily (host-side handles only, no device allocation). */
enum { DLT_K_ROPE = 0, DLT_K_FWD = 1, DLT_K_DELTA = 2, DLT_K_BWD_KV = 3, DLT_K_BWD_Q = 4, DLT_K_COUNT = 5 };
typedef struct {
  int32_t kernel; /* DLT_K_* */
  float ms;
} dlt_kernel_time_t;
/* Plain device-to-device copy of `bytes` bytes (16-byte aligned, multiple of 16) by a grid-stride
 * kernel: a workload of exactly known traffic, used to calibrate what the profiler's
 * FETCH_SIZE / WRITE_SIZE counters report per byte.  No counterpart in the reference. */
int dlt_debug_copy(void* dst, const void* src, int64_t bytes, void* stream);

/* Which kernel family an attention call runs on.  No counterpart in the reference (Triton picks a configuration by
 * autotuning, src/tiled_swa.py:570-573); here the host routes every call by shape, element type, strides and
 * alignment, and a C caller cannot see from the outside that, say, head dim 80 or a 9-token tile at head dim 96 lands on the
 * generic kernels (several times slower than the tuned ones).  dlt_last_kernel_family() returns the family the calling
 * thread's latest forward / backward call (dlt_swa_*, dlt_flash_*) was routed to.  With dlt_dry_run(1) (per thread) those
 * calls validate their arguments and route, but launch nothing and touch no memory: pointers only need the alignment
 * of the real ones, so the query also works in a process without a GPU.
 *   MARCHING  token grids (b_size 1), head dim 64, windows up to 13 x 13 (rotation: 8 rotary pairs, rotated q / k kept)
 *   STREAMING token grids, head dim 64 / 128, windows up to 93 columns (beyond 21 columns in column passes), no rotation;
 *             tiles of 2 ... 15 tokens at head dim 64 / 128 (the grid of token slots, up to 24 column groups of 4 slots)
 *   TILE      token grids, head dims in multiples of 32 up to 128, windows up to 21 columns (rotation in the tile loads)
 *   FLASH     dense / causal / tiles of 16 k tokens, 2-byte element types, head dims up to 128 (multiples of 8)
 *   GENERIC   everything else */
enum { DLT_FAMILY_NONE = 0, DLT_FAMILY_MARCHING = 1, DLT_FAMILY_STREAMING = 2, DLT_FAMILY_TILE = 3, DLT_FAMILY_FLASH = 4,
       DLT_FAMILY_GENERIC = 5 };
int dlt_dry_run(int on);
int dlt_last_kernel_family(void);

int dlt_timing_enable(int on);
int dlt_timing_collect(dlt_kernel_time_t* out, int max, int* n);

#ifdef __cplusplus
}
#endif
#endif /* DLT_H */
