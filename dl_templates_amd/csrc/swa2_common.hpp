// Streaming token-grid kernels (b_size == 1, head dim 64 or 128, windows up to 21 columns, any number of rows):
// shared geometry, asynchronous staging and swizzled operand reads.
//
// A workgroup of 8 waves owns a band of 8 grid rows x 16 grid columns; wave w owns the 4x4 patch at rows
// 4 (w >> 2), columns 4 (w & 3).  The tokens of the other side that any own token can see (8 + 2 WR halo rows x HCW
// halo columns) stream through LDS in chunks of 4 halo rows.  A chunk is copied HBM -> LDS by the DMA path of the
// vector memory unit (16 bytes per lane, no staging registers: at head dim 128 those were a third of the register
// file) into one of two buffers while the other one is consumed, so a chunk costs one workgroup barrier, every
// halo row is fetched once per 8 own rows, and the registers go to operand read-ahead instead.
//
// A wave's window is NCG column groups of 4 halo columns (NCG = 4: windows up to 13 columns, 6: up to 21), so
// HCW = 16 + 4 NCG - 4 halo columns are staged.  LDS rows are 2 D bytes with no padding; the 16-byte piece c of token
// row t is stored at piece c ^ (m (t & 7)), m = D / 64: operand reads of a wave (16 lanes x 16 bytes, or 32 lanes x
// 8 bytes for the transposing read) then fall on distinct banks, and so do the 64 x 16 bytes a copy instruction writes.
#pragma once
#include <type_traits>
#include "swa1_common.hpp"
#include "swa2_index.h"

// compile-time loop: f(std::integral_constant<int, I>) for I = I0 .. N - 1
template <int I, int N, typename F>
DLT_DEV void swa2_for(F&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    swa2_for<I + 1, N>(f);
  }
}

typedef DLT_LDS const char* Swa2Lds;
DLT_DEV u32x4 swa2_lds16(Swa2Lds p) { return *reinterpret_cast<DLT_LDS const u32x4*>(p); }
DLT_DEV u32x2 swa2_lds_tr(Swa2Lds p) {
  s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((DLT_LDS s16x4*)(p));
  return __builtin_bit_cast(u32x2, v);
}

DLT_DEV Swa2Geom swa2_geom(const AttnProblem& p, const Swa2Plan& P) {
  // token slots per grid row and the largest column extent of a window in slots (tiles of P.S tokens)
  return swa2_geom_at(p.g.TR, p.g.TC * P.S, p.g.WR, P.S * P.WCt + P.S - 1, p.H, P, xcd_remap(blockIdx.x, gridDim.x));
}

// One copy instruction as the hardware sees it: 64 lanes x 16 (or 4) bytes from `base + voff` (base wave-uniform)
// to the LDS address `lds` + 16 (4) lane.  It is issued from inline assembly on purpose: the compiler models the
// instruction as a flat access that may touch LDS, and while one is in flight it turns every wait for an LDS read into
// a wait for ALL outstanding LDS reads (lgkmcnt(0)) and for all outstanding copies (vmcnt(0)), which serialises the
// operand read-ahead of the loops that overlap copies with products.  Hidden from its counters, the waits for operand
// reads are exact again; the waits for the copies themselves are explicit (swa2_wait_copies).  M0 (the LDS address of a
// copy) is a reserved register that cannot be named as an operand or a clobber: the statement saves it, sets it, issues
// the copy (which reads M0 at issue) and puts the saved value back, so whatever the compiler itself keeps in M0 (dynamic
// indexing of register arrays, its own LDS-DMA builtin, messages) survives a copy.
DLT_DEV void dlt_copy16_to_lds(const char* base, uint32_t voff, char* lds) {
  const uint32_t m = (uint32_t)(uintptr_t)(DLT_LDS char*)lds;
  uint32_t saved;
  asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %1\n\ts_mov_b32 m0, %0"
               : "=&s"(saved) : "s"(base), "v"(voff), "s"(m) : "memory");
}
DLT_DEV void dlt_copy4_to_lds(const char* base, uint32_t voff, char* lds) {
  const uint32_t m = (uint32_t)(uintptr_t)(DLT_LDS char*)lds;
  uint32_t saved;
  asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %3\n\ts_nop 0\n\tglobal_load_lds_dword %2, %1\n\ts_mov_b32 m0, %0"
               : "=&s"(saved) : "s"(base), "v"(voff), "s"(m) : "memory");
}

// ---- asynchronous staging (maps in swa2_index.h) ----------------------------------------------------------
template <typename C>
struct Swa2Stage {
  uint32_t off[C::NI];   // byte offset of the lane's piece inside a grid row of the tensor, per instruction
  bool last_on;          // the lane takes part in the last instruction
};

template <typename C>
DLT_DEV void swa2_stage_init(Swa2Stage<C>& st, const Swa2Geom& G, int wave, int lane, int sn2) {
#pragma unroll
  for (int i = 0; i < C::NI; i++) st.off[i] = swa2_stage_off<C>(G, wave, lane, sn2, i);
  st.last_on = swa2_stage_last_on<C>(lane);
}

// one of the NI copy instructions of a halo row (to be spread between the products of a chunk: issued together they
// fill the address queue of the memory pipe and stall the wave in front of its first product)
template <typename C, int I>
DLT_DEV void swa2_issue_one(const Swa2Stage<C>& st, const char* row, char* dst) {
  if constexpr (I < C::NI) {
    if (I + 1 < C::NI || C::HCW % C::TPI == 0 || st.last_on)
      dlt_copy16_to_lds(row, st.off[I], dst + 1024 * I);
  }
}
DLT_DEV const char* swa2_issue_row(const Swa2Geom& G, int ch, const char* base, uint32_t rowstride, int wave) {
  return base + (uint32_t)swa2_issue_grid_row(G, ch, wave) * rowstride;   // wave-uniform
}
template <typename C>
DLT_DEV char* swa2_issue_dst(char* buf, int wave) { return buf + swa2_issue_dst_off<C>(wave); }

// copy halo row (wave & 3) of chunk `ch` of the wave's tensor into its place in `buf`
template <typename C>
DLT_DEV void swa2_issue(const Swa2Stage<C>& st, const Swa2Geom& G, int ch, const char* base, uint32_t rowstride, char* buf, int wave) {
  const char* row = swa2_issue_row(G, ch, base, rowstride, wave);
  char* dst = swa2_issue_dst<C>(buf, wave);
  swa2_for<0, C::NI>([&](auto ic) { swa2_issue_one<C, decltype(ic)::value>(st, row, dst); });
}

// every copy this wave issued has landed in LDS (the workgroup barrier that follows makes all of them visible)
DLT_DEV void swa2_wait_copies() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// Groups of instructions in issue order for the scheduler: one matrix instruction, then `nv` vector instructions that
// do not depend on it.  A wave issues in order: vector work placed behind a run of matrix instructions waits for the
// matrix pipe instead of using the issue slots that the pipe leaves free (a matrix instruction holds the pipe for 16
// cycles and the issue port for 8).
#define SWA2_MIX(nm, nv)                                   \
  _Pragma("unroll") for (int i_ = 0; i_ < (nm); i_++) {    \
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);     \
    __builtin_amdgcn_sched_group_barrier(0x002, (nv), 0);  \
  }

// ---- operand reads (lane constants and offsets in swa2_index.h) ------------------------------------------------
// A-operand pieces of the 16 tokens at column group CG of a chunk region: k[c] = head dims 32 c + 8 g .. + 7
template <typename C, int CG>
DLT_DEV void swa2_read_a(Swa2Lds region, const Swa2Lane<C>& L, u32x4 (&k)[C::KC]) {
#pragma unroll
  for (int c = 0; c < C::KC; c++) k[c] = swa2_lds16(region + swa2_read_a_off<C, CG>(L, c));
}

// A operands with tokens along k for the 32 tokens (4 halo rows x 8 columns) at column groups 2 KB, 2 KB + 1 of a chunk
// region: v[i] has head dims 16 (D0 + i) .. + 15 as its rows
template <typename C, int KB, int D0, int ND>
DLT_DEV void swa2_read_tr(Swa2Lds region, const Swa2Lane<C>& L, u32x4 (&v)[ND]) {
#pragma unroll
  for (int i = 0; i < ND; i++) {
    const int d = D0 + i;
    const u32x2 lo = swa2_lds_tr(region + swa2_read_tr_off<C, KB>(L, d, 0));
    const u32x2 hi = swa2_lds_tr(region + swa2_read_tr_off<C, KB>(L, d, 1));
    v[i].x = lo.x; v[i].y = lo.y; v[i].z = hi.x; v[i].w = hi.y;
  }
}

// own-token fragments in B-operand layout: lane (n, g) holds head dims 32 c + 8 g .. + 7 of token n
template <int KC>
DLT_DEV void swa2_own_frags(u32x4 (&f)[KC], const char* base, int sn2, int tok, int g) {
  const char* p = base + ((uint32_t)((tok >= 0 ? tok : 0) * sn2) + 16 * g);
#pragma unroll
  for (int c = 0; c < KC; c++) f[c] = *reinterpret_cast<const u32x4*>(p + 64 * c);
}

// ---- store epilogue: accumulators in C layout (lane (n, g): dims 16 d + 4 g .. + 3 of own token n, times `mul`) -> a
// wave-private LDS tile [16 tokens][2 D bytes] (pieces swizzled with the token index) -> 16-byte pieces -> HBM rows
template <typename C, typename TIO, typename CT>
DLT_DEV void swa2_store_own(char* sW, const f32x4 (&acc)[C::VB], float mul, TIO* base, int64_t sn, const Swa2Geom& G, int r_p, int c_p,
                            int lane) {
  const int n = lane & 15, g = lane >> 4;
#pragma unroll
  for (int d = 0; d < C::VB; d++) {
    u32x2 w;
    w.x = pack2<CT>(acc[d][0] * mul, acc[d][1] * mul);
    w.y = pack2<CT>(acc[d][2] * mul, acc[d][3] * mul);
    *reinterpret_cast<u32x2*>(sW + swa2_tile_write_off<C>(n, g, d)) = w;
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  constexpr int RPI = 64 / C::PIECES;   // tile rows per pass of the wave
  const int c = lane % C::PIECES;
#pragma unroll
  for (int it = 0; it < 16 / RPI; it++) {
    const int row = lane / C::PIECES + RPI * it;
    const u32x4 v = lds_read16(sW + swa2_tile_read_off<C>(row, c));
    const int r = r_p + (row >> 2), col = c_p + (row & 3);
    if (r < G.TR && col < G.TC) store_stream16(base + (int64_t)(r * G.TC + col) * sn + 8 * c, v);
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
}
