// Row-wise top-k selection with lowest-index tie-break and ascending-index output.
//
// One workgroup per score row: 4 wavefronts, or 16 for rows of more than 8192 scores (few such rows make a
// launch, so each has to be walked by more lanes).  The row is mapped to order-preserving 32-bit
// keys and staged in LDS; an MSB-first radix select (4 passes of 8 bits, LDS histogram) finds
// the exact key T of the k-th largest element and how many elements equal to T are still
// needed.  A final ordered pass keeps every key > T plus the first `need` keys == T in index
// order, using wavefront ballots for the running ranks, so the output is ascending and
// deterministic.  Rows too long for LDS are re-read from global memory (L2-resident).
#include "fc_common.h"

#define TK_BINS 256
#define TK_LDS_MAX_KEYS 15360        // 60 KiB of keys: several workgroups of 256 threads per CU
#define TK_LONG_ROW 8192             // rows longer than this take 1024 threads
#define TK_LDS_MAX_KEYS_LONG 36864   // 144 KiB of keys: one workgroup of 1024 threads per CU

__device__ __forceinline__ unsigned tk_key(float f) {
  unsigned u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return 0xffffffffu;  // NaN ranks above +inf
  if ((u & 0x7fffffffu) == 0u) u = 0u;                      // -0 == +0
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

template <bool LDS_KEYS, int TK_THREADS>
__global__ __launch_bounds__(TK_THREADS) void topk_kernel(const float* __restrict__ scores,
                                                          int score_stride, int len,
                                                          const int* __restrict__ row_lens,
                                                          int rows_per_len, int row_lens_mod, int k,
                                                          const int* __restrict__ n_kept,
                                                          int* __restrict__ indices, int index_stride) {
  constexpr int TK_WAVES = TK_THREADS / FC_WAVE;
  extern __shared__ __align__(16) unsigned lds_keys[];
  __shared__ unsigned hist[TK_BINS];
  __shared__ unsigned wave_tot[TK_BINS / FC_WAVE];
  __shared__ unsigned sel_bin, sel_remaining;
  __shared__ unsigned w_eq[TK_WAVES], w_gt[TK_WAVES];

  const int r = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int li = (row_lens || n_kept) ? (r / rows_per_len) % row_lens_mod : 0;
  int n = row_lens ? row_lens[li] : len;
  if (n > len) n = len;
  int kk = n_kept ? n_kept[li] : k;
  if (kk > n) kk = n;
  if (kk > index_stride) kk = index_stride;
  if (n <= 0 || kk <= 0) return;
  const float* row = scores + (long long)r * score_stride;
  int* out = indices + (long long)r * index_stride;

  if (kk == n) {
    for (int i = tid; i < n; i += TK_THREADS) out[i] = i;
    return;
  }

  if (LDS_KEYS) {
    // 16-byte loads, four per thread in flight, when the row starts on a 16-byte boundary
    int done = 0;
    if ((reinterpret_cast<uintptr_t>(row) & 15) == 0) {
      const float4* row4 = reinterpret_cast<const float4*>(row);
      uint4* keys4 = reinterpret_cast<uint4*>(lds_keys);
      const int n4 = n >> 2;
      for (int i0 = 0; i0 < n4; i0 += 4 * TK_THREADS) {
        float4 v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = row4[min(i0 + u * TK_THREADS + tid, n4 - 1)];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int i = i0 + u * TK_THREADS + tid;
          if (i < n4) keys4[i] = make_uint4(tk_key(v[u].x), tk_key(v[u].y), tk_key(v[u].z), tk_key(v[u].w));
        }
      }
      done = n4 << 2;
    }
    for (int i = done + tid; i < n; i += TK_THREADS) lds_keys[i] = tk_key(row[i]);
  }
  auto key_at = [&](int i) -> unsigned { return LDS_KEYS ? lds_keys[i] : tk_key(row[i]); };

  unsigned prefix = 0, mask = 0, remaining = (unsigned)kk;
  for (int shift = 24; shift >= 0; shift -= 8) {
    if (tid < TK_BINS) hist[tid] = 0;
    __syncthreads();
    for (int i0 = 0; i0 < n; i0 += TK_THREADS) {
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
        if (lane == leader) atomicAdd(&hist[lb], (unsigned)__popcll(same));
        todo = todo && bin != lb;
      }
      if (todo) atomicAdd(&hist[bin], 1u);
    }
    __syncthreads();
    // suffix sums over bins: thread t < 256 owns bin 255 - t
    unsigned h = 0, incl = 0;
    if (tid < TK_BINS) {
      h = hist[TK_BINS - 1 - tid];
      incl = h;
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        unsigned up = __shfl_up(incl, o, 64);
        if (lane >= o) incl += up;
      }
      if (lane == 63) wave_tot[wave] = incl;
    }
    __syncthreads();
    if (tid < TK_BINS) {
      unsigned base = 0;
      for (int w = 0; w < wave; ++w) base += wave_tot[w];
      incl += base;
      const unsigned excl = incl - h;  // elements in strictly larger bins
      if (excl < remaining && remaining <= incl) {
        sel_bin = (unsigned)(TK_BINS - 1 - tid);
        sel_remaining = remaining - excl;
      }
    }
    __syncthreads();
    prefix |= sel_bin << shift;
    mask |= 255u << shift;
    remaining = sel_remaining;
    __syncthreads();
  }
  const unsigned T = prefix;
  const unsigned need = remaining;  // how many keys == T to keep (>= 1)

  // each wave owns a contiguous segment, walked 64 keys at a time
  const int seg = (((n + TK_WAVES - 1) / TK_WAVES) + 63) & ~63;
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
  if (lane == 0) { w_eq[wave] = eq_cnt; w_gt[wave] = gt_cnt; }
  __syncthreads();
  unsigned eq_seen = 0, out_pos = 0;
  {
    unsigned eq_run = 0;
    for (int w = 0; w < wave; ++w) {
      unsigned take = need > eq_run ? min(need - eq_run, w_eq[w]) : 0u;
      out_pos += w_gt[w] + take;
      eq_run += w_eq[w];
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
    if (sel) out[out_pos + __popcll(sb & lt_mask)] = i;
    eq_seen += __popcll(eqb);
    out_pos += __popcll(sb);
  }
}

extern "C" int fc_topk_select(const float* scores, int32_t score_stride, int32_t rows, int32_t len,
                              const int32_t* row_lens, int32_t rows_per_len, int32_t row_lens_mod,
                              int32_t k,
                              const int32_t* n_kept, int32_t* indices, int32_t index_stride,
                              void* stream) {
  FC_REQUIRE(scores && indices, FC_EINVAL, "fc_topk_select: null pointer");
  FC_REQUIRE(rows >= 0 && len >= 0 && score_stride >= len && index_stride >= 0, FC_EINVAL,
             "fc_topk_select: bad sizes rows=%d len=%d score_stride=%d index_stride=%d", rows, len,
             score_stride, index_stride);
  FC_REQUIRE(n_kept != nullptr || (k >= 0 && k <= index_stride), FC_EINVAL,
             "fc_topk_select: k=%d does not fit index_stride=%d", k, index_stride);
  FC_REQUIRE((row_lens == nullptr && n_kept == nullptr) || (row_lens_mod > 0 && rows_per_len > 0),
             FC_EINVAL, "fc_topk_select: rows_per_len and row_lens_mod must be positive when per-row sizes are given");
  if (rows == 0 || len == 0) return FC_OK;
  hipStream_t st = (hipStream_t)stream;
#define TK_LAUNCH(LK, TH, LDSB)                                                                                    \
  hipLaunchKernelGGL((topk_kernel<LK, TH>), dim3(rows), dim3(TH), (size_t)(LDSB), st, scores, score_stride, len,  \
                     row_lens, rows_per_len, row_lens_mod, k, n_kept, indices, index_stride)
  if (len <= TK_LONG_ROW) {
    TK_LAUNCH(true, 256, (size_t)len * 4);
  } else if (len <= TK_LDS_MAX_KEYS_LONG) {
    FC_ALLOW_LDS((topk_kernel<true, 1024>), TK_LDS_MAX_KEYS_LONG * 4);
    TK_LAUNCH(true, 1024, (size_t)len * 4);
  } else {
    TK_LAUNCH(false, 1024, 0);
  }
#undef TK_LAUNCH
  FC_CHECK_LAUNCH("fc_topk_select");
  return FC_OK;
}
