// Host side of the attention core: validation that depends on the kernels' limits, the
// per-launch LDS / chunking plan, and dispatch to the instantiation for the padded head dims.
#include "attn_fwd_kernel.hpp"
#include "attn_bwd_kernel.hpp"
#include "swa1_fwd_kernel.hpp"
#include "swa1_bwd_kernel.hpp"
#include "flash_kernel.hpp"
#include "swam_bwd_kernel.hpp"
#include "swa2_bwd_kernel.hpp"

int dlt_launch_fwd_32_32(const FwdArgs&, int, int, hipStream_t);
int dlt_launch_fwd_64_64(const FwdArgs&, int, int, hipStream_t);
int dlt_launch_fwd_128_128(const FwdArgs&, int, int, hipStream_t);
int dlt_launch_fwd_64_128(const FwdArgs&, int, int, hipStream_t);
int dlt_launch_fwd_256_256(const FwdArgs&, int, int, hipStream_t);

int dlt_launch_bwd_32_32(const BwdArgs&, int, const BwdArgs&, int, int, hipStream_t);
int dlt_launch_bwd_64_64(const BwdArgs&, int, const BwdArgs&, int, int, hipStream_t);
int dlt_launch_bwd_128_128(const BwdArgs&, int, const BwdArgs&, int, int, hipStream_t);
int dlt_launch_bwd_64_128(const BwdArgs&, int, const BwdArgs&, int, int, hipStream_t);
int dlt_launch_bwd_256_256(const BwdArgs&, int, const BwdArgs&, int, int, hipStream_t);

int dlt_flash_launch_fwd_32_32(const FlashArgs&, int, int, hipStream_t);
int dlt_flash_launch_fwd_64_64(const FlashArgs&, int, int, hipStream_t);
int dlt_flash_launch_fwd_128_128(const FlashArgs&, int, int, hipStream_t);
int dlt_flash_launch_fwd_64_128(const FlashArgs&, int, int, hipStream_t);
int dlt_flash_launch_bwd_32_32(const FlashBwdArgs&, int, int, int, hipStream_t);
int dlt_flash_launch_bwd_64_64(const FlashBwdArgs&, int, int, int, hipStream_t);
int dlt_flash_launch_bwd_128_128(const FlashBwdArgs&, int, int, int, hipStream_t);
int dlt_flash_launch_bwd_64_128(const FlashBwdArgs&, int, int, int, hipStream_t);
int dlt_launch_delta_32_32(const BwdArgs&, hipStream_t);
int dlt_launch_delta_64_64(const BwdArgs&, hipStream_t);
int dlt_launch_delta_128_128(const BwdArgs&, hipStream_t);
int dlt_launch_delta_64_128(const BwdArgs&, hipStream_t);
int dlt_launch_delta_256_256(const BwdArgs&, hipStream_t);
int dlt_swa1_launch_bwd_64(const Swa1BwdArgs&, int, int, int, int, hipStream_t);
int dlt_swa1_launch_bwd_128(const Swa1BwdArgs&, int, int, int, int, hipStream_t);
int dlt_swa1_launch_fwd_64(const Swa1FwdArgs&, int, int, hipStream_t);
int dlt_swa1_launch_fwd_128(const Swa1FwdArgs&, int, int, hipStream_t);
int dlt_swam_launch_fwd(const SwamFwdArgs&, int, int, hipStream_t);
int dlt_swam_launch_bwd(const SwamBwdArgs&, int, int, hipStream_t);
int dlt_swa2_launch_fwd_64(const Swa2FwdArgs&, int, int, hipStream_t);
int dlt_swa2_launch_bwd_64(const Swa2BwdArgs&, int, int, hipStream_t);
int dlt_swa2_launch_fwd_128(const Swa2FwdArgs&, int, int, hipStream_t);
int dlt_swa2_launch_bwd_128(const Swa2BwdArgs&, int, int, hipStream_t);

namespace {

constexpr int LDS_TOTAL = 160 * 1024;

struct DimClass { int DK, DV, id; };

int pick_dims(const AttnProblem& p, DimClass& dc) {
  if (p.dk <= 32 && p.dv <= 32) dc = {32, 32, 3};  // the reference's demo and test head dims (src/tiled_swa.py:741, src/flash_attn.py:653)
  else if (p.dk <= 64 && p.dv <= 64) dc = {64, 64, 0};
  else if (p.dk <= 64 && p.dv <= 128) dc = {64, 128, 2};
  else if (p.dk <= 128 && p.dv <= 128) dc = {128, 128, 1};
  else if (p.dk <= 256 && p.dv <= 256) dc = {256, 256, 4};  // the largest head dim the reference admits (src/flash_attn.py:460-462): generic kernels only
  else return dlt_set_error(DLT_ERR_UNSUPPORTED, "head dims dk=%d dv=%d: at most 256 is supported", p.dk, p.dv);
  return DLT_OK;
}

int roundup(int v, int m) { return (v + m - 1) / m * m; }

// 16-byte vector access is possible when the last stride is 1 and every row start is aligned
bool vec_ok(const void* ptr, const int64_t* st, int nd, int d, int elem) {
  const int vb = 8 * elem;  // bytes of one 8-element chunk
  if (st[nd - 1] != 1 || d % 8 != 0) return false;
  if ((uintptr_t)ptr % (vb > 16 ? 16 : vb) != 0) return false;
  for (int i = 0; i < nd - 1; i++)
    if ((st[i] * elem) % 16 != 0) return false;
  return true;
}

// [B, H, N, D] tensor (entry 4 of the strides: pixel-row stride of an image-layout tensor, else 0)
bool tvec_ok(const void* ptr, const int64_t* st, int d, int elem) {
  return vec_ok(ptr, st, 4, d, elem) && (st[4] * elem) % 16 == 0;
}

// elements between the first and one past the last token of a (batch, head) slab
int64_t slab_span(const AttnProblem& p, const int64_t* st, int64_t ntok) {
  if (!p.tm.img) return ntok * st[2];
  return ((int64_t)p.g.TR * p.tm.bh - 1) * st[4] + ((int64_t)p.g.TC * p.tm.bw - 1) * st[2] + 1;
}

// chunking plan for a kernel whose halo buffers need `per_tok` bytes per staged token and
// whose own-tile region needs `own_bytes`
int make_plan(const AttnProblem& p, int own, int own_bytes, int per_tok, int XL_own, int XL_halo, AttnPlan& plan) {
  const DltGeom& g = p.g;
  plan.nblk_x = (XL_own + own - 1) / own;
  own_bytes = roundup(own_bytes, 16);
  const int budget2 = LDS_TOTAL / 2 - own_bytes;       // two workgroups per CU
  const int budget1 = LDS_TOTAL - own_bytes - 512;     // one workgroup per CU
  plan.rowfit = 0; plan.chunk_rows = 1; plan.chunk_x = 128;
  if (g.mode == DLT_GEOM_SWA) {
    const int whmax = dlt_imin(XL_halo, own + (2 * g.WC + 2) * g.S);
    const int cx = roundup(whmax + 32, 8);
    const int64_t row_bytes = (int64_t)cx * per_tok;
    const int nrows = 2 * g.WR + 1;
    if (row_bytes <= budget2) {
      plan.rowfit = 1; plan.chunk_x = cx; plan.chunk_rows = dlt_imin((int)(budget2 / row_bytes), nrows);
    } else if (row_bytes <= budget1) {
      plan.rowfit = 1; plan.chunk_x = cx; plan.chunk_rows = dlt_imin((int)(budget1 / row_bytes), nrows);
    }
  }
  if (!plan.rowfit) {
    int cx = 128;
    while (cx > 32 && (int64_t)cx * per_tok > budget2) cx -= 32;
    if ((int64_t)cx * per_tok > budget1) return dlt_set_error(DLT_ERR_UNSUPPORTED, "attention: LDS plan does not fit");
    plan.chunk_x = cx;
  }
  plan.off_a = own_bytes;
  plan.lds_bytes = own_bytes + plan.chunk_rows * plan.chunk_x * per_tok;
  return DLT_OK;
}

// ---- token-grid (b_size == 1) fast path ----------------------------------------------------
struct Swa1Class { int D, wclass, pbit, rope_mode; };
constexpr int SWA2_MAX_PASSES = 4;   // column passes of the streaming kernels: windows up to 93 columns

// Can the token-grid kernels take this problem?  They need 16-byte vector access to the
// streamed tensors, both head dims in one padded class, a window of at most 21 columns and,
// with rotation, rotary partners a power-of-two number of 8-dim chunks apart.
bool swa1_eligible(const AttnProblem& p, const bool* streamed_vec, int n_streamed, Swa1Class& c) {
  if (p.g.mode != DLT_GEOM_SWA || p.g.S != 1 || p.tm.img) return false;
  if (p.dtype != DLT_BF16 && p.dtype != DLT_FP16) return false;
  if (!(p.sm_scale > 0.f)) return false;  // the running max is kept on raw scores: needs a positive scale
  if (p.dk % 32 != 0 || p.dv % 32 != 0) return false;  // 64-byte staging pieces
  if (p.dk <= 64 && p.dv <= 64) c.D = 64;
  else if (p.dk <= 128 && p.dv <= 128 && p.dk > 64 && p.dv > 64) c.D = 128;
  else return false;
  for (int i = 0; i < n_streamed; i++)
    if (!streamed_vec[i]) return false;
  if ((int64_t)p.g.TR * p.g.TC >= ((int64_t)1 << 31) / 1024) return false;  // 32-bit element offsets inside a slab
  // column groups of a wave's window: up to 4 / 6 per class; wider windows (class 2) only run on the streaming kernels,
  // which walk them in column passes
  const int ncg = (4 + 2 * p.g.WC + 3) / 4;
  if (ncg > SWA2_MAX_PASSES * 6) return false;
  c.wclass = ncg <= 4 ? 0 : ncg <= 6 ? 1 : 2;
  c.pbit = 1;
  c.rope_mode = 0;
  if (p.rope.enabled && p.rope.R > 0) {
    const int r8 = p.rope.R / 8;
    if (p.rope.R % 8 != 0 || (r8 & (r8 - 1)) != 0 || 4 * p.rope.R > c.D) return false;
    if ((uintptr_t)p.rope.row_cs % 4 != 0) return false;
    c.pbit = r8;
    // balanced staging map: the rotation covers exactly half of a fully used head dim, so there
    // are as many rotary chunk pairs per token as staging threads
    c.rope_mode = (2 * r8 == c.D / 32 && p.dk == c.D && p.dv == c.D) ? 2 : 1;
    // plain staging map: a thread holds 4 neighbouring chunks of a token, so rotary partners must be 1 or 2
    // chunks apart; farther partners (R = 32: 4 chunks) sit in another thread's piece.  Tensors that arrive
    // rotated are staged without rotation and are not affected.
    if (c.rope_mode == 1 && r8 > 2 && !p.rope_prerot) return false;
  }
  return true;
}

// n_regions: [8 rows x HCW tokens] LDS regions the kernel keeps resident
void swa1_make_plan(const AttnProblem& p, const Swa1Class& c, int n_regions, int extra_bytes, Swa1Plan& plan, int cr = 8, bool kv = false) {
  plan.ncg = (4 + 2 * p.g.WC + 3) / 4;
  const int hcw = swa1_hcw(c.wclass == 0 ? 4 : 6);
  plan.HRP = roundup(4 + 2 * p.g.WR, cr);
  plan.nblk_r = (p.g.TR + 3) / 4;
  plan.nblk_c = (p.g.TC + 15) / 16;
  const int ncgmax = c.wclass == 0 ? 4 : 6;
  const bool wide = c.rope_mode == 0 || c.rope_mode == 3;  // must match WIDE in the kernels
  plan.lds_bytes = cr * hcw * (swa1_pitch(c.D, ncgmax, 0, wide, kv) + swa1_pitch(c.D, ncgmax, 1, wide, kv)) + extra_bytes;
  const int own_tile = 64 * (c.D * 2 + 16);  // output tile of the epilogue
  if (plan.lds_bytes < own_tile) plan.lds_bytes = own_tile;
}

// the token-grid kernels address the streamed tensors with 32-bit BYTE offsets inside a (batch, head) slab
bool swa1_strides_fit(const AttnProblem& p, const AttnTensors& t) {
  const int64_t ntok = (int64_t)p.g.TR * p.g.TC, lim = ((int64_t)1 << 31) - 1;
  const int64_t row = 2 * (int64_t)(p.dk > p.dv ? p.dk : p.dv);   // bytes of the last row
  auto fits = [&](const int64_t* st) { return st[2] >= 0 && (ntok - 1) * st[2] * 2 + row <= lim; };
  // lse2 / delta of the halo tokens are fetched with 32-bit element offsets (backward)
  const bool scalars_fit = t.ls[2] >= 0 && (ntok - 1) * t.ls[2] <= lim;
  return fits(t.qs) && fits(t.ks) && fits(t.vs) && (t.d_o == nullptr || (fits(t.dos) && scalars_fit));
}

int swa1_backward(const AttnProblem& p, const AttnTensors& t, const Swa1Class& c_in, hipStream_t stream) {
  if (dlt_route_note(DLT_FAMILY_TILE)) return DLT_OK;
  Swa1Class c = c_in;
  if (p.rope_prerot && c.rope_mode != 0) c.rope_mode = 3;  // rotated q, k: plain tile loads, gradients rotated back on store
  const int es = dlt_elem_size(p.dtype);
  // delta = rowsum(o * dO): folded into the dQ kernel when o can be read in 16-byte pieces like the
  // other operands, else the pre-pass kernel shared with the generic path
  const bool fuse_delta = tvec_ok(t.o, t.os, p.dv, es) && t.os[2] < ((int64_t)1 << 20);
  BwdArgs d;
  d.p = p;
  d.o = t.o; d.d_o = t.d_o; d.delta = t.delta;
  for (int i = 0; i < 5; i++) { d.os[i] = t.os[i]; d.dos[i] = t.dos[i]; }
  for (int i = 0; i < 3; i++) d.ls[i] = t.ls[i];
  d.o_vec = tvec_ok(t.o, t.os, p.dv, es);
  d.do_vec = tvec_ok(t.d_o, t.dos, p.dv, es);
  d.n_tokens_q = (int64_t)p.g.TR * p.g.XLq;
  if (!fuse_delta) {
    int rc = c.D == 64 ? dlt_launch_delta_64_64(d, stream) : dlt_launch_delta_128_128(d, stream);
    if (rc != DLT_OK) return rc;
  }

  Swa1BwdArgs a;
  a.p = p;
  // chunk heights of the two kernels may differ; the plan fields the kernels read (ncg, block
  // counts) do not depend on it
  Swa1Plan plan_q;
  swa1_make_plan(p, c, 2, 0, plan_q, SWA1_FWD_CR);
  const int hcw = swa1_hcw(c.wclass == 0 ? 4 : 6);
  swa1_make_plan(p, c, 2, 2 * SWA1_KV_CR * hcw * 4, a.plan, SWA1_KV_CR, true);
  const int lds_q = plan_q.lds_bytes, lds_kv = a.plan.lds_bytes;
  a.q = t.q; a.k = t.k; a.v = t.v; a.o = t.o; a.d_o = t.d_o; a.lse = t.lse; a.delta = t.delta;
  a.delta_out = t.delta;
  a.fuse_delta = fuse_delta ? 1 : 0;
  a.dq = t.dq; a.dk = t.dk; a.dv = t.dv;
  for (int i = 0; i < 4; i++) {
    a.qs[i] = t.qs[i]; a.ks[i] = t.ks[i]; a.vs[i] = t.vs[i]; a.os[i] = t.os[i]; a.dos[i] = t.dos[i];
    a.dqs[i] = t.dqs[i]; a.dks[i] = t.dks[i]; a.dvs[i] = t.dvs[i];
  }
  for (int i = 0; i < 3; i++) a.ls[i] = t.ls[i];
  a.q_vec = 1; a.k_vec = 1; a.v_vec = 1; a.do_vec = 1;
  a.dq_vec = tvec_ok(t.dq, t.dqs, p.dk, es);
  a.dk_vec = tvec_ok(t.dk, t.dks, p.dk, es);
  a.dv_vec = tvec_ok(t.dv, t.dvs, p.dv, es);
  a.rope_pbit = c.pbit;
  a.rope_mode = c.rope_mode;
  a.scale_log2 = p.sm_scale * 1.4426950408889634f;
  const int64_t grid = (int64_t)p.B * p.H * a.plan.nblk_r * a.plan.nblk_c;
  if (grid > 0x7fffffff) return dlt_set_error(DLT_ERR_UNSUPPORTED, "attention backward: grid too large");
  return c.D == 64 ? dlt_swa1_launch_bwd_64(a, c.wclass, (int)grid, lds_kv, lds_q, stream)
                   : dlt_swa1_launch_bwd_128(a, c.wclass, (int)grid, lds_kv, lds_q, stream);
}

int swa1_forward(const AttnProblem& p, const AttnTensors& t, const Swa1Class& c, hipStream_t stream) {
  if (dlt_route_note(DLT_FAMILY_TILE)) return DLT_OK;
  const int es = dlt_elem_size(p.dtype);
  Swa1FwdArgs a;
  a.p = p;
  swa1_make_plan(p, c, 2, 0, a.plan, SWA1_FWD_CR);
  a.q = t.q; a.k = t.k; a.v = t.v; a.o = t.out_o; a.lse = t.lse;
  for (int i = 0; i < 4; i++) { a.qs[i] = t.qs[i]; a.ks[i] = t.ks[i]; a.vs[i] = t.vs[i]; a.os[i] = t.os[i]; }
  for (int i = 0; i < 3; i++) a.ls[i] = t.ls[i];
  a.q_rot = c.rope_mode != 0 ? t.q_rot : nullptr;
  a.k_rot = c.rope_mode != 0 ? t.k_rot : nullptr;
  for (int i = 0; i < 4; i++) { a.qrs[i] = t.qrs[i]; a.krs[i] = t.krs[i]; }
  a.q_vec = tvec_ok(t.q, t.qs, p.dk, es);
  a.o_vec = tvec_ok(t.out_o, t.os, p.dv, es);
  a.rope_pbit = c.pbit;
  a.rope_mode = c.rope_mode;
  a.scale_log2 = p.sm_scale * 1.4426950408889634f;
  const int64_t grid = (int64_t)p.B * p.H * a.plan.nblk_r * a.plan.nblk_c;
  if (grid > 0x7fffffff) return dlt_set_error(DLT_ERR_UNSUPPORTED, "attention forward: grid too large");
  return c.D == 64 ? dlt_swa1_launch_fwd_64(a, c.wclass, (int)grid, stream)
                   : dlt_swa1_launch_fwd_128(a, c.wclass, (int)grid, stream);
}

// ---- marching token-grid kernels: head dim 64 exactly, windows up to 13 x 13, no rotation or R = 8 ----------
bool swam_eligible(const AttnProblem& p, const Swa1Class& c) {
  if (c.D != 64 || p.dk != 64 || p.dv != 64) return false;
  if (p.g.WR > 6 || p.g.WC > 6) return false;
  if (c.rope_mode != 0 && !(c.rope_mode == 2 && p.rope.R == 8)) return false;
  return true;
}

// rows per workgroup: the longest band (fewest re-fetched halo rows) that still gives every CU a workgroup
void swam_make_plan(const AttnProblem& p, SwamPlan& plan) {
  plan.nstrips = (p.g.TC + 15) / 16;
  const int steps = (p.g.TR + 7) / 8;
  const int64_t cols = (int64_t)p.B * p.H * plan.nstrips;
  const int gpu_cus = dlt_device_cus();
  int ns = 1;
  for (int cand = 2; cand <= 8 && cand <= steps; cand++)
    if (cols * ((steps + cand - 1) / cand) >= gpu_cus) ns = cand;
  plan.band = 8 * ns;
  plan.nbands = (steps + ns - 1) / ns;
  dlt_fastdiv_make((uint32_t)(plan.nbands * plan.nstrips), plan.m_bh, plan.s_bh);
  dlt_fastdiv_make((uint32_t)plan.nstrips, plan.m_st, plan.s_st);
  dlt_fastdiv_make((uint32_t)p.H, plan.m_h, plan.s_h);
}

int swam_forward(const AttnProblem& p, const AttnTensors& t, const Swa1Class& c, hipStream_t stream) {
  if (dlt_route_note(DLT_FAMILY_MARCHING)) return DLT_OK;
  SwamFwdArgs a;
  a.p = p;
  swam_make_plan(p, a.plan);
  a.q = t.q; a.k = t.k; a.v = t.v; a.o = t.out_o; a.lse = t.lse;
  for (int i = 0; i < 4; i++) { a.qs[i] = t.qs[i]; a.ks[i] = t.ks[i]; a.vs[i] = t.vs[i]; a.os[i] = t.os[i]; }
  for (int i = 0; i < 3; i++) a.ls[i] = t.ls[i];
  a.q_rot = c.rope_mode != 0 ? t.q_rot : nullptr;
  a.k_rot = c.rope_mode != 0 ? t.k_rot : nullptr;
  for (int i = 0; i < 4; i++) { a.qrs[i] = t.qrs[i]; a.krs[i] = t.krs[i]; }
  a.scale_log2 = p.sm_scale * 1.4426950408889634f;
  const int64_t grid = (int64_t)p.B * p.H * a.plan.nbands * a.plan.nstrips;
  if (grid > 0x7fffffff) return dlt_set_error(DLT_ERR_UNSUPPORTED, "attention forward: grid too large");
  return dlt_swam_launch_fwd(a, c.rope_mode != 0, (int)grid, stream);
}

// ---- streaming kernels: head dim 64 or 128 exactly, no rotation, windows up to 21 columns ---------------------------
bool swa2_eligible(const AttnProblem& p, const Swa1Class& c) {
  return (c.D == 64 || c.D == 128) && p.dk == c.D && p.dv == c.D && c.rope_mode == 0;
}
// token slots per grid row, and the largest column extent of a window in slots (tiles of S tokens: S WC + S - 1)
int swa2_slots(const AttnProblem& p) { return p.g.TC * p.g.S; }
int swa2_extent(const AttnProblem& p) { return p.g.S * p.g.WC + p.g.S - 1; }
// Kernel class (column groups of a wave's window per pass: 4 x 4 columns cover windows up to 13 columns, 6 x 4 up to 21)
// and number of column passes.  Wider windows take the split that computes the fewest groups (7 groups: 2 passes of 4,
// not 2 of 6), the larger class on a tie (fewer passes).
void swa2_split(const AttnProblem& p, int& ncg_class, int& npass) {
  const int ncg = (4 + 2 * swa2_extent(p) + 3) / 4;
  if (ncg <= 4) { ncg_class = 4; npass = 1; return; }
  const int n4 = (ncg + 3) / 4, n6 = (ncg + 5) / 6;
  if (4 * n4 < 6 * n6 && n4 <= SWA2_MAX_PASSES) { ncg_class = 4; npass = n4; }
  else { ncg_class = 6; npass = n6; }
}
int swa2_ncg(const AttnProblem& p) { int c, n; swa2_split(p, c, n); return c; }
// the problem without its rotation would run on the streaming kernels
// and is large enough that the four extra launches (two out-of-place rotations, two in-place inverse rotations) do not
// cost more than the tile kernels' repeated rotation (measured: a gain from about 10^5 tokens per call on)
bool swa2_compose_ok(const AttnProblem& p, const Swa1Class& c) {
  return (c.D == 64 || c.D == 128) && p.dk == c.D && p.dv == c.D && (int64_t)p.B * p.H * p.g.TR * p.g.TC >= 131072;
}

void swa2_make_plan(const AttnProblem& p, Swa2Plan& plan, int band = 8) {
  { int c; swa2_split(p, c, plan.npass); }
  plan.S = p.g.S; plan.WCt = p.g.WC;
  dlt_fastdiv_make((uint32_t)p.g.S, plan.m_S, plan.s_S);
  plan.band = band;
  plan.nblk_r = (p.g.TR + band - 1) / band;
  plan.nblk_c = (swa2_slots(p) + 15) / 16;
  dlt_fastdiv_make((uint32_t)(plan.nblk_r * plan.nblk_c), plan.m_bh, plan.s_bh);
  dlt_fastdiv_make((uint32_t)plan.nblk_c, plan.m_c, plan.s_c);
  dlt_fastdiv_make((uint32_t)p.H, plan.m_h, plan.s_h);
}

bool swa2_rows_ok(const AttnProblem& p, const void* ptr, const int64_t* st) {
  return tvec_ok(ptr, st, p.dk, 2) && st[2] >= 0 && ((int64_t)p.g.TR * swa2_slots(p) - 1) * st[2] * 2 + 2 * p.dk <= (((int64_t)1 << 31) - 1);
}
bool swa2_scalars_ok(const AttnProblem& p, const AttnTensors& t) {
  return t.ls[2] >= 0 && ((int64_t)p.g.TR * swa2_slots(p) - 1) * t.ls[2] * 4 + 4 <= (((int64_t)1 << 31) - 1);
}

// Tiles of 2 ... 15 tokens (the regime of the reference's small-tile kernel, src/tiled_swa.py:15-133, b_size < 16 at
// :611): the streaming kernels on the grid of token slots, with the window of a token given by its tile
// (csrc/swa2_index.h).  Head dim 64 or 128 exactly, 2-byte types, no rotation, plain token layout.
bool swa2_tiles_eligible(const AttnProblem& p, const AttnTensors& t, bool backward) {
  if (p.g.mode != DLT_GEOM_SWA || p.g.S < 2 || p.g.S > 15 || p.tm.img) return false;
  if (p.dtype != DLT_BF16 && p.dtype != DLT_FP16) return false;
  if (!(p.sm_scale > 0.f)) return false;
  if (!((p.dk == 64 || p.dk == 128) && p.dv == p.dk)) return false;
  if (p.rope.enabled && p.rope.R > 0) return false;
  if ((4 + 2 * swa2_extent(p) + 3) / 4 > SWA2_MAX_PASSES * 6) return false;
  if ((int64_t)p.g.TR * swa2_slots(p) >= ((int64_t)1 << 31) / 1024) return false;
  if (!swa2_rows_ok(p, t.q, t.qs) || !swa2_rows_ok(p, t.k, t.ks) || !swa2_rows_ok(p, t.v, t.vs)) return false;
  if (!backward) return t.q_rot == nullptr && swa2_rows_ok(p, t.out_o, t.os);
  return swa2_rows_ok(p, t.o, t.os) && swa2_rows_ok(p, t.d_o, t.dos) && swa2_rows_ok(p, t.dq, t.dqs) && swa2_rows_ok(p, t.dk, t.dks) &&
         swa2_rows_ok(p, t.dv, t.dvs) && swa2_scalars_ok(p, t);
}

int swa2_forward(const AttnProblem& p, const AttnTensors& t, hipStream_t stream) {
  if (dlt_route_note(DLT_FAMILY_STREAMING)) return DLT_OK;
  Swa2FwdArgs a;
  a.p = p;
  // head dim 128, more than one band of 8 rows: the forward kernel with two stacked patches per wave (bands of 16 rows);
  // DLT_SWA2_SINGLE_PATCH=1 (read once per process) keeps the one-patch kernel for A/B timing and for its tests
  static const bool single_patch = [] { const char* e = getenv("DLT_SWA2_SINGLE_PATCH"); return e != nullptr && e[0] == '1'; }();
  swa2_make_plan(p, a.plan, p.dk == 128 && p.g.TR > 8 && !single_patch ? 16 : 8);
  a.q = t.q; a.k = t.k; a.v = t.v; a.o = t.out_o; a.lse = t.lse;
  for (int i = 0; i < 4; i++) { a.qs[i] = t.qs[i]; a.ks[i] = t.ks[i]; a.vs[i] = t.vs[i]; a.os[i] = t.os[i]; }
  for (int i = 0; i < 3; i++) a.ls[i] = t.ls[i];
  a.scale_log2 = p.sm_scale * 1.4426950408889634f;
  const int64_t grid = (int64_t)p.B * p.H * a.plan.nblk_r * a.plan.nblk_c;
  if (grid > 0x7fffffff) return dlt_set_error(DLT_ERR_UNSUPPORTED, "attention forward: grid too large");
  return p.dk == 64 ? dlt_swa2_launch_fwd_64(a, swa2_ncg(p), (int)grid, stream) : dlt_swa2_launch_fwd_128(a, swa2_ncg(p), (int)grid, stream);
}

int swa2_backward(const AttnProblem& p, const AttnTensors& t, hipStream_t stream) {
  if (dlt_route_note(DLT_FAMILY_STREAMING)) return DLT_OK;
  Swa2BwdArgs a;
  a.p = p;
  swa2_make_plan(p, a.plan);
  a.q = t.q; a.k = t.k; a.v = t.v; a.o = t.o; a.d_o = t.d_o; a.lse = t.lse; a.delta = t.delta;
  a.dq = t.dq; a.dk = t.dk; a.dv = t.dv;
  for (int i = 0; i < 4; i++) {
    a.qs[i] = t.qs[i]; a.ks[i] = t.ks[i]; a.vs[i] = t.vs[i]; a.os[i] = t.os[i]; a.dos[i] = t.dos[i];
    a.dqs[i] = t.dqs[i]; a.dks[i] = t.dks[i]; a.dvs[i] = t.dvs[i];
  }
  for (int i = 0; i < 3; i++) a.ls[i] = t.ls[i];
  a.scale_log2 = p.sm_scale * 1.4426950408889634f;
  const int64_t grid = (int64_t)p.B * p.H * a.plan.nblk_r * a.plan.nblk_c;
  if (grid > 0x7fffffff) return dlt_set_error(DLT_ERR_UNSUPPORTED, "attention backward: grid too large");
  return p.dk == 64 ? dlt_swa2_launch_bwd_64(a, swa2_ncg(p), (int)grid, stream) : dlt_swa2_launch_bwd_128(a, swa2_ncg(p), (int)grid, stream);
}

// backward on the marching kernels: plain inputs, or rotated inputs with the gradients rotated back on store
int swam_backward(const AttnProblem& p, const AttnTensors& t, bool rot, hipStream_t stream) {
  if (dlt_route_note(DLT_FAMILY_MARCHING)) return DLT_OK;
  SwamBwdArgs a;
  a.p = p;
  swam_make_plan(p, a.plan);
  a.q = t.q; a.k = t.k; a.v = t.v; a.o = t.o; a.d_o = t.d_o; a.lse = t.lse; a.delta = t.delta;
  a.dq = t.dq; a.dk = t.dk; a.dv = t.dv;
  for (int i = 0; i < 4; i++) {
    a.qs[i] = t.qs[i]; a.ks[i] = t.ks[i]; a.vs[i] = t.vs[i]; a.os[i] = t.os[i]; a.dos[i] = t.dos[i];
    a.dqs[i] = t.dqs[i]; a.dks[i] = t.dks[i]; a.dvs[i] = t.dvs[i];
  }
  for (int i = 0; i < 3; i++) a.ls[i] = t.ls[i];
  a.scale_log2 = p.sm_scale * 1.4426950408889634f;
  const int64_t grid = (int64_t)p.B * p.H * a.plan.nbands * a.plan.nstrips;
  if (grid > 0x7fffffff) return dlt_set_error(DLT_ERR_UNSUPPORTED, "attention backward: grid too large");
  return dlt_swam_launch_bwd(a, rot, (int)grid, stream);
}

// 16-byte row pieces and 32-bit byte offsets inside a (batch, head) slab of head dim 64
bool swam_rows_ok(const AttnProblem& p, const void* ptr, const int64_t* st) {
  return tvec_ok(ptr, st, 64, 2) && st[2] >= 0 && ((int64_t)p.g.TR * p.g.TC - 1) * st[2] * 2 + 128 <= (((int64_t)1 << 31) - 1);
}

// ---- flash fast path: dense, causal, and sliding windows over tiles of 16 k tokens -----------
// needs 2-byte elements, 16-byte vector access to q, k, v and 32-bit byte offsets inside a slab;
// tile mode takes no fused rotation (those calls use the generic kernels)
bool flash_eligible(const AttnProblem& p, const AttnTensors& t, bool with_do) {
  if (p.g.mode == DLT_GEOM_SWA) {
    if (p.g.S < 16 || p.g.S % 16 != 0) return false;
    if (p.rope.enabled && p.rope.R > 0) return false;
  }
  if (p.dtype != DLT_BF16 && p.dtype != DLT_FP16) return false;
  if (!(p.sm_scale > 0.f)) return false;  // the running max is kept on raw scores: needs a positive scale
  if (p.dk > 128 || p.dv > 128) return false;
  const int es = 2;
  if (!tvec_ok(t.q, t.qs, p.dk, es) || !tvec_ok(t.k, t.ks, p.dk, es) || !tvec_ok(t.v, t.vs, p.dv, es)) return false;
  if (with_do && !tvec_ok(t.d_o, t.dos, p.dv, es)) return false;
  const int64_t lim = ((int64_t)1 << 31) - 1;
  const int64_t nq = (int64_t)p.g.TR * p.g.XLq, nk = (int64_t)p.g.TR * p.g.XLk;  // tokens of one (batch, head)
  if (slab_span(p, t.ks, nk) * es > lim || slab_span(p, t.vs, nk) * es > lim) return false;
  if (slab_span(p, t.qs, nq) * es > lim) return false;
  if (with_do && slab_span(p, t.dos, nq) * es > lim) return false;
  return true;
}

int flash_forward(const AttnProblem& p, const AttnTensors& t, const DimClass& dc, hipStream_t stream) {
  if (dlt_route_note(DLT_FAMILY_FLASH)) return DLT_OK;
  FlashArgs a;
  a.q = t.q; a.k = t.k; a.v = t.v; a.o = t.out_o; a.lse = t.lse;
  for (int i = 0; i < 5; i++) { a.qs[i] = t.qs[i]; a.ks[i] = t.ks[i]; a.vs[i] = t.vs[i]; a.os[i] = t.os[i]; }
  for (int i = 0; i < 3; i++) a.ls[i] = t.ls[i];
  a.tm = p.tm;
  a.B = p.B; a.H = p.H; a.Lq = p.g.XLq; a.Lk = p.g.XLk; a.dk = p.dk; a.dv = p.dv;
  const int own = 64 * FLASH_NP;
  a.nblk = (a.Lq + own - 1) / own;
  a.causal = p.g.mode == DLT_GEOM_CAUSAL;
  a.causal_group = flash_causal_group(a.Lk, p.dk, p.dv);
  a.tile = p.g.mode == DLT_GEOM_SWA;
  a.g = p.g;
  a.o_vec = tvec_ok(t.out_o, t.os, p.dv, 2);
  const int chunk = flash_ck_fwd(dc.DK, dc.DV) * (dc.DK * 2 + FLASH_PAD + dc.DV * 2 + FLASH_PAD), tile = own * (dc.DV * 2 + 16);
  a.lds_bytes = chunk > tile ? chunk : tile;
  a.scale_log2 = p.sm_scale * 1.4426950408889634f;
  const int64_t grid = (int64_t)p.B * p.H * p.g.TR * a.nblk;
  if (grid > 0x7fffffff) return dlt_set_error(DLT_ERR_UNSUPPORTED, "flash forward: grid too large");
  switch (dc.id) {
    case 0: return dlt_flash_launch_fwd_64_64(a, p.dtype, (int)grid, stream);
    case 1: return dlt_flash_launch_fwd_128_128(a, p.dtype, (int)grid, stream);
    case 3: return dlt_flash_launch_fwd_32_32(a, p.dtype, (int)grid, stream);
    default: return dlt_flash_launch_fwd_64_128(a, p.dtype, (int)grid, stream);
  }
}

int flash_backward(const AttnProblem& p, const AttnTensors& t, const DimClass& dc, hipStream_t stream) {
  if (dlt_route_note(DLT_FAMILY_FLASH)) return DLT_OK;
  BwdArgs d;
  d.p = p;
  d.o = t.o; d.d_o = t.d_o; d.delta = t.delta;
  for (int i = 0; i < 5; i++) { d.os[i] = t.os[i]; d.dos[i] = t.dos[i]; }
  for (int i = 0; i < 3; i++) d.ls[i] = t.ls[i];
  d.o_vec = tvec_ok(t.o, t.os, p.dv, 2);
  d.do_vec = 1;
  d.n_tokens_q = (int64_t)p.g.TR * p.g.XLq;
  // delta = rowsum(o * dO): folded into the dQ kernel when o can be read in 16-byte pieces
  const bool fuse_delta = tvec_ok(t.o, t.os, p.dv, 2) && slab_span(p, t.os, (int64_t)p.g.TR * p.g.XLq) * 2 < ((int64_t)1 << 31);
  if (!fuse_delta) {
    int rc = dc.id == 0 ? dlt_launch_delta_64_64(d, stream) : dc.id == 1 ? dlt_launch_delta_128_128(d, stream)
           : dc.id == 3 ? dlt_launch_delta_32_32(d, stream) : dlt_launch_delta_64_128(d, stream);
    if (rc != DLT_OK) return rc;
  }

  FlashBwdArgs a;
  a.q = t.q; a.k = t.k; a.v = t.v; a.o = t.o; a.d_o = t.d_o; a.lse = t.lse; a.delta = t.delta;
  a.delta_out = t.delta;
  a.fuse_delta = fuse_delta ? 1 : 0;
  a.dq = t.dq; a.dk = t.dk; a.dv = t.dv;
  for (int i = 0; i < 5; i++) {
    a.qs[i] = t.qs[i]; a.ks[i] = t.ks[i]; a.vs[i] = t.vs[i]; a.os[i] = t.os[i]; a.dos[i] = t.dos[i];
    a.dqs[i] = t.dqs[i]; a.dks[i] = t.dks[i]; a.dvs[i] = t.dvs[i];
  }
  for (int i = 0; i < 3; i++) a.ls[i] = t.ls[i];
  a.tm = p.tm;
  a.B = p.B; a.H = p.H; a.Lq = p.g.XLq; a.Lk = p.g.XLk; a.dk_ = p.dk; a.dv_ = p.dv;
  const int own = 64 * flash_np_q(dc.DK, dc.DV), own_kv = 64 * flash_np_kv(dc.DK, dc.DV);
  a.nblk_q = (a.Lq + own - 1) / own;
  a.nblk_k = (a.Lk + own_kv - 1) / own_kv;
  a.causal = p.g.mode == DLT_GEOM_CAUSAL;
  a.causal_group = flash_causal_group(a.Lk, p.dk, p.dv);
  a.tile = p.g.mode == DLT_GEOM_SWA;
  a.g = p.g;
  a.dq_vec = tvec_ok(t.dq, t.dqs, p.dk, 2);
  a.dk_vec = tvec_ok(t.dk, t.dks, p.dk, 2);
  a.dv_vec = tvec_ok(t.dv, t.dvs, p.dv, 2);
  const int row = dc.DK * 2 + FLASH_PAD + dc.DV * 2 + FLASH_PAD;   // one streamed token in both LDS regions
  const int chunk_q = flash_ck_q(dc.DK, dc.DV) * row, ck_kv = flash_ck_kv(dc.DK, dc.DV);
  const int tile_q = own * (dc.DK * 2 + 16);
  const int tile_k = own_kv * (dc.DK * 2 + 16), tile_v = own_kv * (dc.DV * 2 + 16);
  a.lds_q = chunk_q > tile_q ? chunk_q : tile_q;
  a.lds_kv = ck_kv * row + 2 * ck_kv * 4;
  if (tile_k > a.lds_kv) a.lds_kv = tile_k;
  if (tile_v > a.lds_kv) a.lds_kv = tile_v;
  a.scale_log2 = p.sm_scale * 1.4426950408889634f;
  a.sm_scale = p.sm_scale;
  const int64_t grid_q = (int64_t)p.B * p.H * p.g.TR * a.nblk_q, grid_kv = (int64_t)p.B * p.H * p.g.TR * a.nblk_k;
  if (grid_q > 0x7fffffff || grid_kv > 0x7fffffff) return dlt_set_error(DLT_ERR_UNSUPPORTED, "flash backward: grid too large");
  switch (dc.id) {
    case 0: return dlt_flash_launch_bwd_64_64(a, p.dtype, (int)grid_kv, (int)grid_q, stream);
    case 1: return dlt_flash_launch_bwd_128_128(a, p.dtype, (int)grid_kv, (int)grid_q, stream);
    case 3: return dlt_flash_launch_bwd_32_32(a, p.dtype, (int)grid_kv, (int)grid_q, stream);
    default: return dlt_flash_launch_bwd_64_128(a, p.dtype, (int)grid_kv, (int)grid_q, stream);
  }
}

}  // namespace

int dlt_attn_forward(const AttnProblem& p, const AttnTensors& t, hipStream_t stream) {
  dlt_route_reset();
  DimClass dc;
  int rc = pick_dims(p, dc);
  if (rc != DLT_OK) return rc;
  const int es = dlt_elem_size(p.dtype);
  {
    // q is not streamed, but its own-token fragments are read as 16-byte pieces too
    const bool streamed[3] = {tvec_ok(t.q, t.qs, p.dk, es), tvec_ok(t.k, t.ks, p.dk, es), tvec_ok(t.v, t.vs, p.dv, es)};
    Swa1Class c;
    if (swa1_eligible(p, streamed, 3, c) && swa1_strides_fit(p, t)) {
      // rotated side outputs come from the fused kernels only (16-byte rows); otherwise see below
      const bool side_ok = t.q_rot == nullptr || (c.rope_mode != 0 && tvec_ok(t.q_rot, t.qrs, p.dk, es) &&
                                                  tvec_ok(t.k_rot, t.krs, p.dk, es));
      if (side_ok) {
        // the marching kernels store o in 16-byte pieces and address every tensor with 32-bit offsets
        const bool rows_fit = swam_rows_ok(p, t.out_o, t.os) &&
                              (t.q_rot == nullptr || (swam_rows_ok(p, t.q_rot, t.qrs) && swam_rows_ok(p, t.k_rot, t.krs)));
        if (swam_eligible(p, c) && rows_fit) return swam_forward(p, t, c, stream);
        if (swa2_eligible(p, c) && t.q_rot == nullptr && swa2_rows_ok(p, t.out_o, t.os)) return swa2_forward(p, t, stream);
        // Rotation the marching kernels do not take, with the rotated q / k wanted by the caller: rotating both out of place
        // first (below) and running the streaming kernels on the result is faster than the tile kernels, which rotate every
        // halo row again in each workgroup that stages it (128 x 128 grid, d = 128, 21 x 21, 16 rotary pairs, fwd+bwd:
        // 0.90 -> 0.64 ms)
        const bool compose = c.rope_mode != 0 && t.q_rot != nullptr && swa2_compose_ok(p, c) && swa2_rows_ok(p, t.out_o, t.os) &&
                             swa2_rows_ok(p, t.q_rot, t.qrs) && swa2_rows_ok(p, t.k_rot, t.krs);
        if (c.wclass < 2 && !compose) return swa1_forward(p, t, c, stream);
      }
    }
  }
  if (t.q_rot != nullptr) {
    // rotate q and k out of place, then run the plain operator on the rotated tensors (any kernel family)
    rc = dlt_rope_rotate_copy(t.q, t.qs, t.q_rot, t.qrs, p.B, p.H, (int64_t)p.g.TR * p.g.XLq, p.dk, p.rope, p.dtype, stream);
    if (rc == DLT_OK)
      rc = dlt_rope_rotate_copy(t.k, t.ks, t.k_rot, t.krs, p.B, p.H, (int64_t)p.g.TR * p.g.XLk, p.dk, p.rope, p.dtype, stream);
    if (rc != DLT_OK) return rc;
    AttnProblem p2 = p;
    p2.rope = dlt_make_rope_dev(nullptr, 0);
    AttnTensors t2 = t;
    t2.q = t.q_rot; t2.k = t.k_rot; t2.q_rot = t2.k_rot = nullptr;
    for (int i = 0; i < 5; i++) { t2.qs[i] = t.qrs[i]; t2.ks[i] = t.krs[i]; }
    return dlt_attn_forward(p2, t2, stream);
  }
  if (flash_eligible(p, t, false)) return flash_forward(p, t, dc, stream);
  if (swa2_tiles_eligible(p, t, false)) return swa2_forward(p, t, stream);
  if (dlt_route_note(DLT_FAMILY_GENERIC)) return DLT_OK;
  const int np = (p.g.mode == DLT_GEOM_SWA || dc.id == 4) ? 1 : 2;
  const int own = 64 * np;
  // fp32 tensors: q and k rows are staged as hi + lo bf16 pairs (must match SPLIT in attn_fwd_kernel.hpp)
  const int PQ = dc.DK * (p.dtype == DLT_FP32 ? 4 : 2) + 16, PK = PQ, PV = dc.DV * 2 + 16, PO = dc.DV * es + 16;
  FwdArgs a;
  a.p = p;
  rc = make_plan(p, own, own * (PQ > PO ? PQ : PO), PK + PV, p.g.XLq, p.g.XLk, a.plan);
  if (rc != DLT_OK) return rc;
  a.plan.off_b = a.plan.off_a + a.plan.chunk_rows * a.plan.chunk_x * PK;
  a.plan.off_c = a.plan.off_d = 0;
  a.q = t.q; a.k = t.k; a.v = t.v; a.o = t.out_o; a.lse = t.lse;
  for (int i = 0; i < 5; i++) { a.qs[i] = t.qs[i]; a.ks[i] = t.ks[i]; a.vs[i] = t.vs[i]; a.os[i] = t.os[i]; }
  for (int i = 0; i < 3; i++) a.ls[i] = t.ls[i];
  a.q_vec = tvec_ok(t.q, t.qs, p.dk, es);
  a.k_vec = tvec_ok(t.k, t.ks, p.dk, es);
  a.v_vec = tvec_ok(t.v, t.vs, p.dv, es);
  a.o_vec = tvec_ok(t.out_o, t.os, p.dv, es);
  a.scale_log2 = p.sm_scale * 1.4426950408889634f;
  const int64_t grid = (int64_t)p.B * p.H * p.g.TR * a.plan.nblk_x;
  if (grid > 0x7fffffff) return dlt_set_error(DLT_ERR_UNSUPPORTED, "attention forward: grid too large");
  switch (dc.id) {
    case 0: return dlt_launch_fwd_64_64(a, np, (int)grid, stream);
    case 1: return dlt_launch_fwd_128_128(a, np, (int)grid, stream);
    case 3: return dlt_launch_fwd_32_32(a, np, (int)grid, stream);
    case 4: return dlt_launch_fwd_256_256(a, np, (int)grid, stream);
    default: return dlt_launch_fwd_64_128(a, np, (int)grid, stream);
  }
}

int dlt_attn_backward(const AttnProblem& p, const AttnTensors& t, hipStream_t stream) {
  dlt_route_reset();
  DimClass dc;
  int rc = pick_dims(p, dc);
  if (rc != DLT_OK) return rc;
  const int es = dlt_elem_size(p.dtype);
  {
    const bool streamed[4] = {tvec_ok(t.q, t.qs, p.dk, es), tvec_ok(t.k, t.ks, p.dk, es),
                              tvec_ok(t.v, t.vs, p.dv, es), tvec_ok(t.d_o, t.dos, p.dv, es)};
    Swa1Class c;
    if (swa1_eligible(p, streamed, 4, c) && swa1_strides_fit(p, t)) {
      Swa1Class cm = c;
      if (p.rope_prerot && cm.rope_mode != 0) cm.rope_mode = 2;   // the marching kernels rotate dq / dk back on store
      const bool plain_or_prerot = c.rope_mode == 0 || p.rope_prerot;
      if (plain_or_prerot && swam_eligible(p, cm) && swam_rows_ok(p, t.o, t.os) && swam_rows_ok(p, t.dq, t.dqs) &&
          swam_rows_ok(p, t.dk, t.dks) && swam_rows_ok(p, t.dv, t.dvs))
        return swam_backward(p, t, c.rope_mode != 0, stream);
      // lse2 / delta rows are copied with 32-bit byte offsets inside a (batch, head) slab
      if (swa2_eligible(p, c) && swa2_rows_ok(p, t.o, t.os) && swa2_rows_ok(p, t.dq, t.dqs) && swa2_rows_ok(p, t.dk, t.dks) &&
          swa2_rows_ok(p, t.dv, t.dvs) && swa2_scalars_ok(p, t))
        return swa2_backward(p, t, stream);
      // rotated q, k that the marching kernels do not take: the streaming kernels on the rotated tensors, then dq / dk
      // rotated back in place (below), instead of the tile kernels (see the forward pass)
      const bool compose = p.rope_prerot && c.rope_mode != 0 && swa2_compose_ok(p, c) && swa2_rows_ok(p, t.o, t.os) &&
                           swa2_rows_ok(p, t.dq, t.dqs) && swa2_rows_ok(p, t.dk, t.dks) && swa2_rows_ok(p, t.dv, t.dvs) && swa2_scalars_ok(p, t);
      if (c.wclass < 2 && !compose) return swa1_backward(p, t, c, stream);
    }
  }
  if (p.rope_prerot && p.rope.enabled && p.rope.R > 0 && !p.tm.img) {
    // rotated q, k and no token-grid kernel: the plain operator (any kernel family) yields the gradients of the
    // rotated tensors; the standalone rotation turns them back in place
    AttnProblem p2 = p;
    p2.rope = dlt_make_rope_dev(nullptr, 0);
    p2.rope_prerot = 0;
    rc = dlt_attn_backward(p2, t, stream);
    if (rc != DLT_OK) return rc;
    dlt_rope_t r;
    r.idx = p.rope.idx; r.row_cs = p.rope.row_cs; r.col_cs = p.rope.col_cs;
    r.row_cs_stride0 = p.rope.rs0; r.col_cs_stride0 = p.rope.cs0;
    r.n_rdim = p.rope.R; r.row_len = p.rope.row_len; r.col_len = p.rope.col_len;
    rc = dlt_rope_inplace_4d(t.dq, t.dqs, p.B, p.H, (int64_t)p.g.TR * p.g.XLq, p.dk, &r, 1, p.dtype, stream);
    if (rc != DLT_OK) return rc;
    return dlt_rope_inplace_4d(t.dk, t.dks, p.B, p.H, (int64_t)p.g.TR * p.g.XLk, p.dk, &r, 1, p.dtype, stream);
  }
  if (flash_eligible(p, t, true)) return flash_backward(p, t, dc, stream);
  if (swa2_tiles_eligible(p, t, true)) return swa2_backward(p, t, stream);
  if (dlt_route_note(DLT_FAMILY_GENERIC)) return DLT_OK;
  const int np = 1;
  const int own = 64 * np;
  // fp32 tensors: q and k rows are staged as hi + lo bf16 pairs (must match SPLIT in attn_bwd_kernel.hpp)
  const int PQ = dc.DK * (p.dtype == DLT_FP32 ? 4 : 2) + 16, PV = dc.DV * 2 + 16;
  const int tile_k = dc.DK * es + 16, tile_v = dc.DV * es + 16;
  int own_bytes = own * (PQ + PV);
  if (own * tile_k > own_bytes) own_bytes = own * tile_k;
  if (own * tile_v > own_bytes) own_bytes = own * tile_v;

  BwdArgs a;
  a.p = p;
  a.q = t.q; a.k = t.k; a.v = t.v; a.o = t.o; a.d_o = t.d_o; a.lse = t.lse; a.delta = t.delta;
  a.dq = t.dq; a.dk = t.dk; a.dv = t.dv;
  for (int i = 0; i < 5; i++) {
    a.qs[i] = t.qs[i]; a.ks[i] = t.ks[i]; a.vs[i] = t.vs[i]; a.os[i] = t.os[i]; a.dos[i] = t.dos[i];
    a.dqs[i] = t.dqs[i]; a.dks[i] = t.dks[i]; a.dvs[i] = t.dvs[i];
  }
  for (int i = 0; i < 3; i++) a.ls[i] = t.ls[i];
  a.q_vec = tvec_ok(t.q, t.qs, p.dk, es);
  a.k_vec = tvec_ok(t.k, t.ks, p.dk, es);
  a.v_vec = tvec_ok(t.v, t.vs, p.dv, es);
  a.o_vec = tvec_ok(t.o, t.os, p.dv, es);
  a.do_vec = tvec_ok(t.d_o, t.dos, p.dv, es);
  a.dq_vec = tvec_ok(t.dq, t.dqs, p.dk, es);
  a.dk_vec = tvec_ok(t.dk, t.dks, p.dk, es);
  a.dv_vec = tvec_ok(t.dv, t.dvs, p.dv, es);
  a.scale_log2 = p.sm_scale * 1.4426950408889634f;
  a.n_tokens_q = (int64_t)p.g.TR * p.g.XLq;

  // dK/dV: keys are the own side, queries (Q, dO, lse2, delta) are streamed
  BwdArgs akv = a;
  rc = make_plan(p, own, own_bytes, PQ + PV + 8, p.g.XLk, p.g.XLq, akv.plan);
  if (rc != DLT_OK) return rc;
  {
    const int toks = akv.plan.chunk_rows * akv.plan.chunk_x;
    akv.plan.off_b = akv.plan.off_a + toks * PQ;
    akv.plan.off_c = akv.plan.off_b + toks * PV;
    akv.plan.off_d = akv.plan.off_c + toks * 4;
  }
  // dQ: queries are the own side, K and V are streamed
  BwdArgs aq = a;
  rc = make_plan(p, own, own_bytes, PQ + PV, p.g.XLq, p.g.XLk, aq.plan);
  if (rc != DLT_OK) return rc;
  aq.plan.off_b = aq.plan.off_a + aq.plan.chunk_rows * aq.plan.chunk_x * PQ;
  aq.plan.off_c = aq.plan.off_d = 0;

  const int64_t grid_kv = (int64_t)p.B * p.H * p.g.TR * akv.plan.nblk_x;
  const int64_t grid_q = (int64_t)p.B * p.H * p.g.TR * aq.plan.nblk_x;
  if (grid_kv > 0x7fffffff || grid_q > 0x7fffffff) return dlt_set_error(DLT_ERR_UNSUPPORTED, "attention backward: grid too large");
  switch (dc.id) {
    case 0: return dlt_launch_bwd_64_64(akv, (int)grid_kv, aq, (int)grid_q, np, stream);
    case 1: return dlt_launch_bwd_128_128(akv, (int)grid_kv, aq, (int)grid_q, np, stream);
    case 3: return dlt_launch_bwd_32_32(akv, (int)grid_kv, aq, (int)grid_q, np, stream);
    case 4: return dlt_launch_bwd_256_256(akv, (int)grid_kv, aq, (int)grid_q, np, stream);
    default: return dlt_launch_bwd_64_128(akv, (int)grid_kv, aq, (int)grid_q, np, stream);
  }
}
