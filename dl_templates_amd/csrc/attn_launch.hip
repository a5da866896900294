// Host side of the attention core: validation that depends on the kernels' limits, the
// per-launch LDS / chunking plan, and dispatch to the instantiation for the padded head dims.
#include "attn_fwd_kernel.hpp"
#include "attn_bwd_kernel.hpp"

int dlt_launch_fwd_64_64(const FwdArgs&, int, int, hipStream_t);
int dlt_launch_fwd_128_128(const FwdArgs&, int, int, hipStream_t);
int dlt_launch_fwd_64_128(const FwdArgs&, int, int, hipStream_t);

int dlt_launch_bwd_64_64(const BwdArgs&, int, const BwdArgs&, int, int, hipStream_t);
int dlt_launch_bwd_128_128(const BwdArgs&, int, const BwdArgs&, int, int, hipStream_t);
int dlt_launch_bwd_64_128(const BwdArgs&, int, const BwdArgs&, int, int, hipStream_t);

namespace {

constexpr int LDS_TOTAL = 160 * 1024;

struct DimClass { int DK, DV, id; };

int pick_dims(const AttnProblem& p, DimClass& dc) {
  if (p.dk <= 64 && p.dv <= 64) dc = {64, 64, 0};
  else if (p.dk <= 64 && p.dv <= 128) dc = {64, 128, 2};
  else if (p.dk <= 128 && p.dv <= 128) dc = {128, 128, 1};
  else return dlt_set_error(DLT_ERR_UNSUPPORTED, "head dims dk=%d dv=%d: at most 128 is supported", p.dk, p.dv);
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

}  // namespace

int dlt_attn_forward(const AttnProblem& p, const AttnTensors& t, hipStream_t stream) {
  DimClass dc;
  int rc = pick_dims(p, dc);
  if (rc != DLT_OK) return rc;
  const int es = dlt_elem_size(p.dtype);
  const int np = p.g.mode == DLT_GEOM_SWA ? 1 : 2;
  const int own = 64 * np;
  const int PQ = dc.DK * 2 + 16, PK = dc.DK * 2 + 16, PV = dc.DV * 2 + 16, PO = dc.DV * es + 16;
  FwdArgs a;
  a.p = p;
  rc = make_plan(p, own, own * (PQ > PO ? PQ : PO), PK + PV, p.g.XLq, p.g.XLk, a.plan);
  if (rc != DLT_OK) return rc;
  a.plan.off_b = a.plan.off_a + a.plan.chunk_rows * a.plan.chunk_x * PK;
  a.plan.off_c = a.plan.off_d = 0;
  a.q = t.q; a.k = t.k; a.v = t.v; a.o = t.out_o; a.lse = t.lse;
  for (int i = 0; i < 4; i++) { a.qs[i] = t.qs[i]; a.ks[i] = t.ks[i]; a.vs[i] = t.vs[i]; a.os[i] = t.os[i]; }
  for (int i = 0; i < 3; i++) a.ls[i] = t.ls[i];
  a.q_vec = vec_ok(t.q, t.qs, 4, p.dk, es);
  a.k_vec = vec_ok(t.k, t.ks, 4, p.dk, es);
  a.v_vec = vec_ok(t.v, t.vs, 4, p.dv, es);
  a.o_vec = vec_ok(t.out_o, t.os, 4, p.dv, es);
  a.scale_log2 = p.sm_scale * 1.4426950408889634f;
  const int64_t grid = (int64_t)p.B * p.H * p.g.TR * a.plan.nblk_x;
  if (grid > 0x7fffffff) return dlt_set_error(DLT_ERR_UNSUPPORTED, "attention forward: grid too large");
  switch (dc.id) {
    case 0: return dlt_launch_fwd_64_64(a, np, (int)grid, stream);
    case 1: return dlt_launch_fwd_128_128(a, np, (int)grid, stream);
    default: return dlt_launch_fwd_64_128(a, np, (int)grid, stream);
  }
}

int dlt_attn_backward(const AttnProblem& p, const AttnTensors& t, hipStream_t stream) {
  DimClass dc;
  int rc = pick_dims(p, dc);
  if (rc != DLT_OK) return rc;
  const int es = dlt_elem_size(p.dtype);
  const int np = 1;
  const int own = 64 * np;
  const int PQ = dc.DK * 2 + 16, PV = dc.DV * 2 + 16;
  const int tile_k = dc.DK * es + 16, tile_v = dc.DV * es + 16;
  int own_bytes = own * (PQ + PV);
  if (own * tile_k > own_bytes) own_bytes = own * tile_k;
  if (own * tile_v > own_bytes) own_bytes = own * tile_v;

  BwdArgs a;
  a.p = p;
  a.q = t.q; a.k = t.k; a.v = t.v; a.o = t.o; a.d_o = t.d_o; a.lse = t.lse; a.delta = t.delta;
  a.dq = t.dq; a.dk = t.dk; a.dv = t.dv;
  for (int i = 0; i < 4; i++) {
    a.qs[i] = t.qs[i]; a.ks[i] = t.ks[i]; a.vs[i] = t.vs[i]; a.os[i] = t.os[i]; a.dos[i] = t.dos[i];
    a.dqs[i] = t.dqs[i]; a.dks[i] = t.dks[i]; a.dvs[i] = t.dvs[i];
  }
  for (int i = 0; i < 3; i++) a.ls[i] = t.ls[i];
  a.q_vec = vec_ok(t.q, t.qs, 4, p.dk, es);
  a.k_vec = vec_ok(t.k, t.ks, 4, p.dk, es);
  a.v_vec = vec_ok(t.v, t.vs, 4, p.dv, es);
  a.o_vec = vec_ok(t.o, t.os, 4, p.dv, es);
  a.do_vec = vec_ok(t.d_o, t.dos, 4, p.dv, es);
  a.dq_vec = vec_ok(t.dq, t.dqs, 4, p.dk, es);
  a.dk_vec = vec_ok(t.dk, t.dks, 4, p.dk, es);
  a.dv_vec = vec_ok(t.dv, t.dvs, 4, p.dv, es);
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
    default: return dlt_launch_bwd_64_128(akv, (int)grid_kv, aq, (int)grid_q, np, stream);
  }
}
