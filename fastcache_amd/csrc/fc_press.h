// The tail that the one-launch presses share: selection of a column's kept positions from its scores in LDS and the
// in-place compaction of its K and V rows.
#pragma once
#include "fc_rows.h"
#include "fc_select.h"

// What the one-launch press kernels end with: the kk best of the column's S scores in LDS (0 < kk <= S, clamped by the
// caller), their positions to the index row and to LDS, and the kept K and V rows moved to the front of the column.
template <int EB, int THREADS>
__device__ __forceinline__ void kp_select_and_move(const KvView& kv, const KvView& vv, const int* ktbl, bool k_lds,
                                                   const int* vtbl, bool v_lds, const float* sc, int* sel,
                                                   TkShared<THREADS>& sh, int l, int b, int h, int S, int kk,
                                                   int* __restrict__ idx_row) {
  const int tid = threadIdx.x, sub = tid % (FC_HEAD_DIM * EB / 16);
  if (kk == S) {   // everything stays where it is
    for (int i = tid; i < S; i += THREADS) idx_row[i] = i;
    return;
  }
  tk_select_row<THREADS>(sh, [&](int i) { return tk_key(sc[i]); }, S, kk, [&](int pos, int i) {
    idx_row[pos] = i;
    sel[pos] = i;
  });
  __syncthreads();
  // compaction in place: row j <- row sel[j], K then V
  char* kbase = kv.base + ((long long)l * kv.stride_layer + (long long)h * kv.stride_head) * EB + sub * 16;
  cp_walk<EB, 1, THREADS>(kv, kv, ktbl, k_lds, ktbl, k_lds, b, S, kk, kbase, kbase, kv.base + sub * 16, 0,
                          [&](int j) { return sel[j]; });
  char* vbase = vv.base + ((long long)l * vv.stride_layer + (long long)h * vv.stride_head) * EB + sub * 16;
  cp_walk<EB, 1, THREADS>(vv, vv, vtbl, v_lds, vtbl, v_lds, b, S, kk, vbase, vbase, vv.base + sub * 16, 0,
                          [&](int j) { return sel[j]; });
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
