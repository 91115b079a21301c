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

// The same selection with the row's keys held in registers: every wavefront owns a contiguous segment of the row and
// its lane l the keys segment + e * 64 + l, e < KPT, read and converted ONCE (key_at is called once per key), so the
// digit passes and the ordered pass cost a handful of vector instructions per key instead of an LDS read and a
// conversion each.  Needs n <= THREADS * KPT.
// A column's selection is a chain of short steps between workgroup barriers, and inside a kernel whose other
// workgroups keep the compute unit busy every barrier costs about a microsecond, so the passes are arranged for few
// of them: one per digit pass (every wavefront scans the 256 bins for itself instead of sharing a scan through LDS;
// three histograms in rotation, so that clearing the next one needs no barrier of its own) and one before the
// ordered pass.  The digit passes stop as soon as every key left in the threshold bin is kept (then no tie has to
// be ranked): rows of distinct scores end after two or three passes.
// Keys never produced by tk_key (0) stand for "no key here"; they rank below every real key.
template <int THREADS>
struct TkSharedRegs {
  unsigned hist[3][TK_BINS];
  unsigned w_eq[THREADS / FC_WAVE], w_gt[THREADS / FC_WAVE];
};

template <int THREADS, int KPT, typename KeyAt, typename Emit>
__device__ __forceinline__ void tk_select_row_regs(TkSharedRegs<THREADS>& sh, KeyAt key_at, int n, int kk, Emit emit) {
  constexpr int WAVES = THREADS / FC_WAVE;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int seg = (((n + WAVES - 1) / WAVES) + 63) & ~63;   // <= KPT * 64 by the caller's bound
  const int beg = wave * seg;
  const int end = min(n, beg + seg);
  const int live_e = end > beg ? (end - beg + 63) >> 6 : 0;   // wave-uniform: 64-key groups of this wavefront
  unsigned key[KPT];
#pragma unroll
  for (int e = 0; e < KPT; ++e) {
    const int i = beg + e * 64 + lane;
    key[e] = (e < live_e && i < end) ? key_at(i) : 0u;
  }
  for (int i = tid; i < 2 * TK_BINS; i += THREADS) (&sh.hist[0][0])[i] = 0;   // histograms of the first two passes
  __syncthreads();
  unsigned prefix = 0, mask = 0, remaining = (unsigned)kk;
  bool whole_bin = false;   // every key that matches the prefix so far is kept
  int pass = 0;
  for (int shift = 24; shift >= 0 && !whole_bin; shift -= 8, ++pass) {
    unsigned* hist = sh.hist[pass % 3];
    if (pass >= 1)   // the histogram of the pass after this one; its last readers are two barriers back
      for (int i = tid; i < TK_BINS; i += THREADS) sh.hist[(pass + 1) % 3][i] = 0;
#pragma unroll
    for (int e = 0; e < KPT; ++e) {
      if (e < live_e) {
        const unsigned u = key[e];
        if (u != 0u && (u & mask) == prefix) atomicAdd(&hist[(u >> shift) & 255u], 1u);
      }
    }
    __syncthreads();
    // every wavefront for itself: lane t holds bins 255 - 4t .. 252 - 4t (descending), suffix sums over the 256 bins
    unsigned h4[4], incl = 0;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      h4[r] = hist[TK_BINS - 1 - (4 * lane + r)];
      incl += h4[r];
    }
    const unsigned own = incl;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const unsigned up = __shfl_up(incl, o, 64);
      if (lane >= o) incl += up;
    }
    unsigned excl = incl - own;   // keys in bins above this lane's four
    int found = -1;
    unsigned left = 0, size = 0;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      if (found < 0 && excl < remaining && remaining <= excl + h4[r]) {
        found = TK_BINS - 1 - (4 * lane + r);
        left = remaining - excl;
        size = h4[r];
      }
      excl += h4[r];
    }
    const unsigned long long who = __ballot(found >= 0);   // exactly one lane
    const int src = __ffsll((long long)who) - 1;
    const unsigned bin = (unsigned)__shfl(found, src, 64);
    remaining = __shfl(left, src, 64);
    whole_bin = __shfl(size, src, 64) == remaining;
    prefix |= bin << shift;
    mask |= 255u << shift;
  }
  // kept: keys whose masked bits exceed the prefix, and of those that equal it the first `remaining` by index
  // (all of them when whole_bin; after four passes the masked bits are the whole key)
  const unsigned T = prefix;
  const unsigned need = remaining;
  unsigned eq_cnt = 0, gt_cnt = 0;
#pragma unroll
  for (int e = 0; e < KPT; ++e) {
    if (e < live_e) {
      const unsigned u = key[e], m = u & mask;
      eq_cnt += __popcll(__ballot(u != 0u && m == T));
      gt_cnt += __popcll(__ballot(u != 0u && m > T));
    }
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
#pragma unroll
  for (int e = 0; e < KPT; ++e) {
    if (e < live_e) {
      const unsigned u = key[e], m = u & mask;
      const bool is_eq = u != 0u && m == T;
      const unsigned long long eqb = __ballot(is_eq);
      const unsigned my_rank = eq_seen + __popcll(eqb & lt_mask);
      const bool sel = u != 0u && (m > T || (is_eq && my_rank < need));
      const unsigned long long sb = __ballot(sel);
      if (sel) emit((int)(out_pos + __popcll(sb & lt_mask)), beg + e * 64 + lane);
      eq_seen += __popcll(eqb);
      out_pos += __popcll(sb);
    }
  }
}

// LDS of whichever form of the selection a kernel ends up calling
template <int THREADS>
union TkArea {
  TkShared<THREADS> lds_keys;
  TkSharedRegs<THREADS> reg_keys;
};
