// Row-wise top-k selection with lowest-index tie-break and ascending-index output.
//
// One workgroup per score row: 4 wavefronts, or 16 for rows of more than 8192 scores (few such rows make a
// launch, so each has to be walked by more lanes).  The row is mapped to order-preserving 32-bit
// keys and staged in LDS; an MSB-first radix select (4 passes of 8 bits, LDS histogram) finds
// the exact key T of the k-th largest element and how many elements equal to T are still
// needed.  A final ordered pass keeps every key > T plus the first `need` keys == T in index
// order, using wavefront ballots for the running ranks, so the output is ascending and
// deterministic.  Rows too long for LDS are re-read from global memory (L2-resident).
#include "fc_select.h"

#define TK_LDS_MAX_KEYS 15360        // 60 KiB of keys: several workgroups of 256 threads per CU
#define TK_LONG_ROW 8192             // rows longer than this take 1024 threads
#define TK_LDS_MAX_KEYS_LONG 36864   // 144 KiB of keys: one workgroup of 1024 threads per CU

template <bool LDS_KEYS, int TK_THREADS>
__global__ __launch_bounds__(TK_THREADS) void topk_kernel(const float* __restrict__ scores,
                                                          int score_stride, int len,
                                                          const int* __restrict__ row_lens,
                                                          int rows_per_len, int row_lens_mod, int k,
                                                          const int* __restrict__ n_kept,
                                                          int* __restrict__ indices, int index_stride) {
  extern __shared__ __align__(16) unsigned lds_keys[];
  __shared__ TkShared<TK_THREADS> sh;

  const int r = blockIdx.x;
  const int tid = threadIdx.x;
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

  tk_select_row<TK_THREADS>(sh, key_at, n, kk, [&](int pos, int i) { out[pos] = i; });
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
