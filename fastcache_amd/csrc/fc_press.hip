// Knorm press in one launch: score, select and compact a (layer, sequence, kv head) column by one workgroup.
//
// The three-launch form (norms of every key, top-k per row, compaction per column) reads K, writes the scores, reads
// them back, writes the indices, reads them back and reads the kept rows: every launch starts with an empty GPU and
// ends with a draining one.  Here a workgroup owns its column from beginning to end: it streams the column's key rows
// once for the norms (scores kept in LDS and written out for the caller), selects the kept positions in LDS with the
// same radix select as the stand-alone kernel, and moves the kept K and V rows to the front of the column with the
// same ordered walk as the compaction kernel, so scores, indices and cache bytes are those of the three launches.
// Workgroups run through their phases out of step, so one column's selection hides behind other columns' traffic.
#include "fc_norm.h"
#include "fc_press.h"

#define KP_MAX_LDS (144 * 1024)   // the column's scores and kept positions stay in LDS: 4 * (max_seq_len + index_stride) bytes
#define KP_U 4          // key rows per lane in flight while scoring
// 1024 threads per column from this many bytes of key rows per column on, 256 below.  More lanes finish a column sooner
// (more rows in flight per column, fewer columns half done at any time) but idle through a short column's selection.
// The figures behind both constants are in profiles/launch_shape_crossovers.txt (the library built with the
// constants forced to 0 and to 2e9, `python -m fastcache_amd.crossovers knorm select` on each): the Knorm press with
// 1024 against 256 threads 1.07 / 1.31 ms (4096 columns x 2048 bf16 rows), 0.555 / 0.608 (4096 x 1024), 1.30 / 1.08
// (16384 x 512), 3.59 / 1.04 (65536 x 128); selection + compaction alone 0.509 / 0.519 (2304 x 4096), 0.467 / 0.451
// (4096 x 2048), 0.935 / 0.459 (16384 x 512).
#ifndef KP_WIDE_BYTES_PRESS
#define KP_WIDE_BYTES_PRESS (256 * 1024)
#endif
#ifndef KP_WIDE_BYTES_SELECT
#define KP_WIDE_BYTES_SELECT (1024 * 1024)
#endif

// Which column a workgroup takes.  Workgroups go to the eight XCDs round-robin in launch order; columns that follow each
// other in memory (the heads of a sequence, whose rows of one token are adjacent) are given to the same XCD, one after
// the other, when the column count is a multiple of eight (cfg1: -1.5 %; no effect on the 256-byte rows of cfg2).
__device__ __forceinline__ void kp_column(int& h, int& b, int& l, int H, int B, int L) {
  const long long n = (long long)H * B * L;
  const long long id = blockIdx.x + (long long)gridDim.x * (blockIdx.y + (long long)gridDim.y * blockIdx.z);
  const long long col = (n % 8) == 0 ? (id % 8) * (n / 8) + id / 8 : id;
  h = (int)(col % H);
  b = (int)((col / H) % B);
  l = (int)(col / ((long long)H * B));
}

template <int DTYPE, int THREADS>
__global__ __launch_bounds__(THREADS) void knorm_press_kernel(KvView kv, KvView vv, float* __restrict__ scores,
                                                              int score_stride, int k, const int* __restrict__ n_kept,
                                                              int* __restrict__ indices, int index_stride, int smax) {
  constexpr int EB = (DTYPE == FC_F32) ? 4 : 2;
  constexpr int LPR = FC_HEAD_DIM * EB / 16;   // lanes per row
  constexpr int RPP = THREADS / LPR;           // rows per pass
  extern __shared__ __align__(16) float sc[];  // [smax] scores of the column, then the kept positions
  int* sel = reinterpret_cast<int*>(sc + smax);
  __shared__ int ktbl[CP_TBL], vtbl[CP_TBL];
  __shared__ TkArea<THREADS> sh;

  int h, b, l;
  kp_column(h, b, l, kv.num_kv_heads, kv.batch, kv.num_layers);
  const int H = kv.num_kv_heads;
  const int tid = threadIdx.x, sub = tid % LPR, rg = tid / LPR;
  const int S = min(fc_seq_len(kv, b), smax);
  const long long row_id = ((long long)l * kv.batch + b) * H + h;
  float* out_row = scores + row_id * score_stride;
  int* idx_row = indices + row_id * index_stride;

  for (int s = S + tid; s < score_stride; s += THREADS) out_row[s] = -INFINITY;
  if (S <= 0) return;

  bool k_lds, v_lds;
  kp_tables<THREADS>(kv, vv, ktbl, vtbl, b, S, k_lds, v_lds);
  __syncthreads();

  // ---- norms: KP_U rows per lane and pass, all loads issued before the first is reduced --------------------
  char* kbase = kv.base + ((long long)l * kv.stride_layer + (long long)h * kv.stride_head) * EB + sub * 16;
  for (int r0 = 0; r0 < S; r0 += RPP * KP_U) {
    uint4 x[KP_U];
    unsigned live = 0;
#pragma unroll
    for (int u = 0; u < KP_U; ++u) {
      const int r = min(r0 + u * RPP + rg, S - 1);
      long long off = cp_offset(kv, ktbl, k_lds, b, r);
      live |= off >= 0 ? (1u << u) : 0u;
      off = off < 0 ? 0 : off;
      x[u] = *reinterpret_cast<const uint4*>(kbase + off * EB);
    }
#pragma unroll
    for (int u = 0; u < KP_U; ++u) {
      float part = fc_group_sum<16>(row_sumsq_part<DTYPE>(x[u]));
      if (LPR == 32) part += __shfl_xor(part, 16, 64);
      const int r = r0 + u * RPP + rg;
      if (r < S && sub == 0) sc[r] = (live >> u) & 1u ? -sqrtf(part) : -INFINITY;
    }
  }
  __syncthreads();
  for (int s = tid; s < S; s += THREADS) out_row[s] = sc[s];

  // ---- selection: counts read from device memory are clamped to what the host validated ----------------------
  int kk = n_kept ? n_kept[b] : k;
  kk = min(min(kk, S), index_stride);
  if (kk <= 0) return;
  kp_select_and_move<EB, THREADS, false>(kv, vv, ktbl, k_lds, vtbl, v_lds, sc, sel, sh, nullptr, l, b, h, S, kk, 0, idx_row);
}

// Selection and compaction of a column from scores that another kernel wrote (any press whose scores are per
// (layer, sequence, kv head, token)): fc_topk_select and fc_compact of a cache onto itself in one launch.
template <int EB, int THREADS>
__global__ __launch_bounds__(THREADS) void select_compact_kernel(KvView kv, KvView vv, const float* __restrict__ scores,
                                                                 int score_stride, int k,
                                                                 const int* __restrict__ n_kept,
                                                                 int* __restrict__ indices, int index_stride, int smax) {
  extern __shared__ __align__(16) float sc[];  // [smax] scores of the column, then the kept positions
  int* sel = reinterpret_cast<int*>(sc + smax);
  __shared__ int ktbl[CP_TBL], vtbl[CP_TBL];
  __shared__ TkArea<THREADS> sh;
  int h, b, l;
  kp_column(h, b, l, kv.num_kv_heads, kv.batch, kv.num_layers);
  const int tid = threadIdx.x;
  const int S = min(fc_seq_len(kv, b), smax);
  int kk = n_kept ? n_kept[b] : k;
  kk = min(min(kk, S), index_stride);
  if (kk <= 0) return;
  const long long row_id = ((long long)l * kv.batch + b) * kv.num_kv_heads + h;
  const float* row = scores + row_id * score_stride;
  if ((reinterpret_cast<uintptr_t>(row) & 15) == 0) {
    const float4* row4 = reinterpret_cast<const float4*>(row);
    float4* sc4 = reinterpret_cast<float4*>(sc);
    for (int i = tid; i < (S >> 2); i += THREADS) sc4[i] = row4[i];
    for (int i = (S & ~3) + tid; i < S; i += THREADS) sc[i] = row[i];
  } else {
    for (int i = tid; i < S; i += THREADS) sc[i] = row[i];
  }
  bool k_lds, v_lds;
  kp_tables<THREADS>(kv, vv, ktbl, vtbl, b, S, k_lds, v_lds);
  __syncthreads();
  kp_select_and_move<EB, THREADS, false>(kv, vv, ktbl, k_lds, vtbl, v_lds, sc, sel, sh, nullptr, l, b, h, S, kk, 0,
                                  indices + row_id * index_stride);
}

static int kp_check(const char* who, const fc_kv_view* keys, const fc_kv_view* values, const void* scores,
                    int32_t score_stride, int32_t k, const int32_t* n_kept, const void* indices, int32_t index_stride) {
  int rc;
  if ((rc = fc_check_view(keys, who)) || (rc = fc_check_view(values, who))) return rc;
  FC_REQUIRE(keys->dtype == values->dtype && keys->num_layers == values->num_layers && keys->batch == values->batch &&
                 keys->num_kv_heads == values->num_kv_heads && keys->max_seq_len == values->max_seq_len,
             FC_EINVAL, "%s: key and value views disagree on dtype/layers/batch/heads/length", who);
  FC_REQUIRE(scores && indices, FC_EINVAL, "%s: null pointer", who);
  FC_REQUIRE(score_stride >= keys->max_seq_len, FC_EINVAL, "%s: score_stride %d < max_seq_len %d", who, score_stride,
             keys->max_seq_len);
  FC_REQUIRE(index_stride >= 0 && index_stride <= keys->max_seq_len, FC_EINVAL,
             "%s: index_stride %d exceeds max_seq_len %d", who, index_stride, keys->max_seq_len);
  FC_REQUIRE(n_kept != nullptr || (k >= 0 && k <= index_stride), FC_EINVAL, "%s: k=%d vs index_stride=%d", who, k,
             index_stride);
  FC_REQUIRE(4LL * ((long long)keys->max_seq_len + index_stride) <= KP_MAX_LDS, FC_EUNSUPPORTED,
             "%s: 4 * (max_seq_len + index_stride) = 4 * (%d + %d) bytes exceed the %d of LDS a column may take; such "
             "shapes take the separate launches (fc_topk_select, fc_compact)", who, keys->max_seq_len, index_stride,
             KP_MAX_LDS);
  FC_REQUIRE(keys->batch <= 65535 && keys->num_layers <= 65535, FC_EUNSUPPORTED, "%s: grid too large", who);
  return FC_OK;
}

extern "C" int fc_knorm_press(const fc_kv_view* keys, const fc_kv_view* values, float* scores, int32_t score_stride,
                              int32_t k, const int32_t* n_kept, int32_t* indices, int32_t index_stride, void* stream) {
  const char* who = "fc_knorm_press";
  int rc = kp_check(who, keys, values, scores, score_stride, k, n_kept, indices, index_stride);
  if (rc) return rc;
  if (keys->max_seq_len == 0 || score_stride == 0) return FC_OK;
  KvView kv = fc_make_view(keys), vv = fc_make_view(values);
  const int smax = keys->max_seq_len;
  const size_t lds = ((size_t)smax + (size_t)index_stride) * 4;
  dim3 grid(keys->num_kv_heads, keys->batch, keys->num_layers);
  hipStream_t st = (hipStream_t)stream;
#define KP_LAUNCH(DT, TH)                                                                                        \
  do {                                                                                                           \
    FC_ALLOW_LDS((knorm_press_kernel<DT, TH>), KP_MAX_LDS);                                                       \
    hipLaunchKernelGGL((knorm_press_kernel<DT, TH>), grid, dim3(TH), lds, st, kv, vv, scores, score_stride, k,   \
                       n_kept, indices, index_stride, smax);                                                     \
  } while (0)
  const bool wide = (long long)smax * FC_HEAD_DIM * fc_elem_bytes(keys->dtype) >= KP_WIDE_BYTES_PRESS;
#define KP_DISPATCH(DT) \
  if (wide) KP_LAUNCH(DT, 1024); else KP_LAUNCH(DT, 256)
  switch (keys->dtype) {
    case FC_F32: KP_DISPATCH(FC_F32); break;
    case FC_F16: KP_DISPATCH(FC_F16); break;
    default: KP_DISPATCH(FC_BF16); break;
  }
#undef KP_DISPATCH
#undef KP_LAUNCH
  FC_CHECK_LAUNCH(who);
  return FC_OK;
}

extern "C" int fc_select_compact(const fc_kv_view* keys, const fc_kv_view* values, const float* scores,
                                 int32_t score_stride, int32_t k, const int32_t* n_kept, int32_t* indices,
                                 int32_t index_stride, void* stream) {
  const char* who = "fc_select_compact";
  int rc = kp_check(who, keys, values, scores, score_stride, k, n_kept, indices, index_stride);
  if (rc) return rc;
  if (keys->max_seq_len == 0 || (!n_kept && k == 0)) return FC_OK;
  KvView kv = fc_make_view(keys), vv = fc_make_view(values);
  const int smax = keys->max_seq_len;
  const size_t lds = ((size_t)smax + (size_t)index_stride) * 4;
  dim3 grid(keys->num_kv_heads, keys->batch, keys->num_layers);
  hipStream_t st = (hipStream_t)stream;
#define KP_LAUNCH(E, TH)                                                                                          \
  do {                                                                                                           \
    FC_ALLOW_LDS((select_compact_kernel<E, TH>), KP_MAX_LDS);                                                     \
    hipLaunchKernelGGL((select_compact_kernel<E, TH>), grid, dim3(TH), lds, st, kv, vv, scores, score_stride, k, \
                       n_kept, indices, index_stride, smax);                                                     \
  } while (0)
  const bool wide = (long long)smax * FC_HEAD_DIM * fc_elem_bytes(keys->dtype) >= KP_WIDE_BYTES_SELECT;
  if (keys->dtype == FC_F32) {
    if (wide) KP_LAUNCH(4, 1024); else KP_LAUNCH(4, 256);
  } else {
    if (wide) KP_LAUNCH(2, 1024); else KP_LAUNCH(2, 256);
  }
#undef KP_LAUNCH
  FC_CHECK_LAUNCH(who);
  return FC_OK;
}
