// The tail that the one-launch presses share: selection of a column's kept positions from its scores in LDS and the
// in-place compaction of its K and V rows.
#pragma once
#include "fc_rows.h"
#include "fc_select.h"

// Keys per thread that the lean tail's selection keeps in registers; longer rows are selected from LDS.
#define KP_KPT 16

// What the one-launch press kernels end with: the kk best of the column's S scores in LDS (0 < kk <= S, clamped by the
// caller), their positions to the index row and to LDS, and the kept K and V rows moved to the front of the column.
// The last `tail_kept` positions of the column are kept whatever their scores and are not entered in the selection
// (SnapKV's observation window, kk > tail_kept); sc[] need not hold them.  ptbl: 2 * CP_PT words of 8 bytes in LDS.
//
// LEAN picks the forms with the fewest instructions: the selection over keys held in registers and, for a paged
// column, the walk over page addresses precomputed in LDS (about a fifth of the vector instructions of the general
// forms).  That is what counts inside the SnapKV kernel, which runs at the package power limit, where a column's tail
// costs what its instructions and bytes cost however they are scheduled (measured: ordered chunks, free-running
// streams and the general walk all take the same time there; only the instruction count moved it).  The Knorm press
// and the stand-alone selection + compaction are bound by memory latency instead: there the general walk, which has
// the next chunk's loads in flight before the current chunk's stores are issued and never waits for a store, is the
// faster one (cfg1: 0.282 ms against 0.294 to 0.312 ms with the lean forms), so they keep it.
template <int EB, int THREADS, bool LEAN>
__device__ __forceinline__ void kp_select_and_move(const KvView& kv, const KvView& vv, const int* ktbl, bool k_lds,
                                                   const int* vtbl, bool v_lds, const float* sc, int* sel,
                                                   TkArea<THREADS>& sh, unsigned long long* ptbl, int l, int b, int h,
                                                   int S, int kk, int tail_kept, int* __restrict__ idx_row) {
  const int tid = threadIdx.x, sub = tid % (FC_HEAD_DIM * EB / 16);
  if (kk == S) {   // everything stays where it is
    for (int i = tid; i < S; i += THREADS) idx_row[i] = i;
    return;
  }
  const int n = S - tail_kept, want = kk - tail_kept;   // 0 < want < n
  auto key_at = [&](int i) { return tk_key(sc[i]); };
  auto emit = [&](int pos, int i) {
    idx_row[pos] = i;
    sel[pos] = i;
  };
  if (LEAN && n <= THREADS * KP_KPT)
    tk_select_row_regs<THREADS, KP_KPT>(sh.reg_keys, key_at, n, want, emit);
  else
    tk_select_row<THREADS>(sh.lds_keys, key_at, n, want, emit);
  for (int i = tid; i < tail_kept; i += THREADS) emit(want + i, n + i);
  __syncthreads();
  // compaction in place: row j <- row sel[j]
  char* kcol = kv.base + ((long long)l * kv.stride_layer + (long long)h * kv.stride_head) * EB;
  char* vcol = vv.base + ((long long)l * vv.stride_layer + (long long)h * vv.stride_head) * EB;
  bool paged_walk = LEAN && k_lds && v_lds && cp_pages_ok<EB, THREADS>(kv, S) && cp_pages_ok<EB, THREADS>(vv, S);
  if (paged_walk) {
    const bool k_ok = cp_fill_pages<EB, THREADS>(kv, ktbl, kcol, S, ptbl);
    const bool v_ok = cp_fill_pages<EB, THREADS>(vv, vtbl, vcol, S, ptbl + CP_PT);
    paged_walk = k_ok && v_ok;
  }
  if (paged_walk) {
    const CpPages kp = {ptbl, kv.block_shift, (unsigned)(kv.stride_token * EB)};
    const CpPages vp = {ptbl + CP_PT, vv.block_shift, (unsigned)(vv.stride_token * EB)};
    cp_walk_pages<EB, THREADS>(kp, vp, kk, sel);
  } else {   // the general ordered walk, K then V
    cp_walk<EB, 1, THREADS>(kv, kv, ktbl, k_lds, ktbl, k_lds, b, S, kk, kcol + sub * 16, kcol + sub * 16,
                            kv.base + sub * 16, 0, [&](int j) { return sel[j]; });
    cp_walk<EB, 1, THREADS>(vv, vv, vtbl, v_lds, vtbl, v_lds, b, S, kk, vcol + sub * 16, vcol + sub * 16,
                            vv.base + sub * 16, 0, [&](int j) { return sel[j]; });
  }
}

// the sequence's block-table rows of both views into LDS (when they fit); the caller synchronises
template <int THREADS>
__device__ __forceinline__ void kp_tables(const KvView& kv, const KvView& vv, int* ktbl, int* vtbl, int b, int S,
                                          bool& k_lds, bool& v_lds) {
  const int tid = threadIdx.x;
  const int nblk_k = kv.block_shift >= 0 ? ((S - 1) >> kv.block_shift) + 1 : 0;
  const int nblk_v = vv.block_shift >= 0 ? ((S - 1) >> vv.block_shift) + 1 : 0;
  k_lds = kv.block_tables && kv.block_shift >= 0 && nblk_k <= CP_TBL;
  v_lds = vv.block_tables && vv.block_shift >= 0 && nblk_v <= CP_TBL;
  if (k_lds)
    for (int i = tid; i < nblk_k; i += THREADS) ktbl[i] = kv.block_tables[(long long)b * kv.table_stride + i];
  if (v_lds)
    for (int i = tid; i < nblk_v; i += THREADS) vtbl[i] = vv.block_tables[(long long)b * vv.table_stride + i];
}
