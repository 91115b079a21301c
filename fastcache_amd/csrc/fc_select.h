// Exact top-k selection of one row by one workgroup, shared by the kernels that select: MSB-first radix select over
// order-preserving 32-bit keys, then an ordered pass that emits the kept positions in ascending order.
#pragma once
#include "fc_common.h"

#define TK_BINS 256

// order-preserving key of a score: larger score, larger key
__device__ __forceinline__ unsigned tk_key(float f) {
  unsigned u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return 0xffffffffu;  // NaN ranks above +inf
  if ((u & 0x7fffffffu) == 0u) u = 0u;                      // -0 == +0
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// LDS words the selection needs beside the keys
template <int THREADS>
struct TkShared {
  unsigned hist[TK_BINS];
  unsigned wave_tot[TK_BINS / FC_WAVE];
  unsigned sel_bin, sel_remaining;
  unsigned w_eq[THREADS / FC_WAVE], w_gt[THREADS / FC_WAVE];
};

// The kk largest of the n keys key_at(0..n-1), 0 < kk < n, ties to the lowest index: emit(position, index) is called
// once per kept index, positions 0..kk-1 in ascending index order.  Every thread of the workgroup (THREADS of them,
// at least 256) calls this; it synchronises the workgroup several times, the first time before it touches `sh`.
template <int THREADS, typename KeyAt, typename Emit>
__device__ __forceinline__ void tk_select_row(TkShared<THREADS>& sh, KeyAt key_at, int n, int kk, Emit emit) {
  constexpr int WAVES = THREADS / FC_WAVE;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  unsigned prefix = 0, mask = 0, remaining = (unsigned)kk;
  for (int shift = 24; shift >= 0; shift -= 8) {
    if (tid < TK_BINS) sh.hist[tid] = 0;
    __syncthreads();
    for (int i0 = 0; i0 < n; i0 += THREADS) {
      const int i = i0 + tid;
      const unsigned u = i < n ? key_at(i) : 0u;
      bool todo = i < n && (u & mask) == prefix;
      const unsigned bin = (u >> shift) & 255u;
      // Scores of one row share their leading bits, so most lanes of a wavefront hit the same bin in the
      // first passes and their atomics would serialise: the two most common bins are counted with a
      // ballot and one atomic each, what is left goes through per-lane atomics.
#pragma unroll
      for (int rep = 0; rep < 2; ++rep) {
        const unsigned long long act = __ballot(todo);
        if (act == 0ull) break;
        const int leader = __ffsll((long long)act) - 1;
        const unsigned lb = __shfl(bin, leader, 64);
        const unsigned long long same = __ballot(todo && bin == lb);
        if (lane == leader) atomicAdd(&sh.hist[lb], (unsigned)__popcll(same));
        todo = todo && bin != lb;
      }
      if (todo) atomicAdd(&sh.hist[bin], 1u);
    }
    __syncthreads();
    // suffix sums over bins: thread t < 256 owns bin 255 - t
    unsigned h = 0, incl = 0;
    if (tid < TK_BINS) {
      h = sh.hist[TK_BINS - 1 - tid];
      incl = h;
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        unsigned up = __shfl_up(incl, o, 64);
        if (lane >= o) incl += up;
      }
      if (lane == 63) sh.wave_tot[wave] = incl;
    }
    __syncthreads();
    if (tid < TK_BINS) {
      unsigned base = 0;
      for (int w = 0; w < wave; ++w) base += sh.wave_tot[w];
      incl += base;
      const unsigned excl = incl - h;  // elements in strictly larger bins
      if (excl < remaining && remaining <= incl) {
        sh.sel_bin = (unsigned)(TK_BINS - 1 - tid);
        sh.sel_remaining = remaining - excl;
      }
    }
    __syncthreads();
    prefix |= sh.sel_bin << shift;
    mask |= 255u << shift;
    remaining = sh.sel_remaining;
    __syncthreads();
  }
  const unsigned T = prefix;
  const unsigned need = remaining;  // how many keys == T to keep (>= 1)

  // each wave owns a contiguous segment, walked 64 keys at a time
  const int seg = (((n + WAVES - 1) / WAVES) + 63) & ~63;
  const int beg = wave * seg;
  const int end = min(n, beg + seg);
  unsigned eq_cnt = 0, gt_cnt = 0;
  for (int i0 = beg; i0 < end; i0 += 64) {
    int i = i0 + lane;
    unsigned u = (i < end) ? key_at(i) : 0u;
    bool live = i < end;
    eq_cnt += __popcll(__ballot(live && u == T));
    gt_cnt += __popcll(__ballot(live && u > T));
  }
  if (lane == 0) { sh.w_eq[wave] = eq_cnt; sh.w_gt[wave] = gt_cnt; }
  __syncthreads();
  unsigned eq_seen = 0, out_pos = 0;
  {
    unsigned eq_run = 0;
    for (int w = 0; w < wave; ++w) {
      unsigned take = need > eq_run ? min(need - eq_run, sh.w_eq[w]) : 0u;
      out_pos += sh.w_gt[w] + take;
      eq_run += sh.w_eq[w];
    }
    eq_seen = eq_run;
  }
  const unsigned long long lt_mask = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
  for (int i0 = beg; i0 < end; i0 += 64) {
    int i = i0 + lane;
    bool live = i < end;
    unsigned u = live ? key_at(i) : 0u;
    bool is_eq = live && u == T;
    unsigned long long eqb = __ballot(is_eq);
    unsigned my_rank = eq_seen + __popcll(eqb & lt_mask);
    bool sel = live && (u > T || (is_eq && my_rank < need));
    unsigned long long sb = __ballot(sel);
    if (sel) emit((int)(out_pos + __popcll(sb & lt_mask)), i);
    eq_seen += __popcll(eqb);
    out_pos += __popcll(sb);
  }
}
