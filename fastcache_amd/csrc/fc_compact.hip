// Gather/compaction of kept K/V rows, and plain ordered token copies.
//
// One workgroup per (K|V, layer, sequence, kv head) column (per pair of heads for 512-byte fp32 rows), walked by
// cp_walk in ascending chunks, which makes the in-place case (dst aliases src) safe.  Different heads, layers and
// K/V planes touch disjoint bytes, so columns need no ordering between each other.
#include "fc_rows.h"

#define CP_THREADS 256

// GATHER: src token = indices[j]; otherwise src token = src_start + j.
// The column is walked in chunks of CH rows with two register buffers: the loads of chunk c+1 are
// issued right after the barrier that releases the stores of chunk c, so loads and stores overlap.
// HG = consecutive kv heads handled by one workgroup (divides num_kv_heads)
template <int EB, bool GATHER, int HG>
__global__ __launch_bounds__(CP_THREADS) void compact_kernel(KvView sk, KvView sv, KvView dk, KvView dv,
                                                             const int* __restrict__ indices,
                                                             int index_stride, int heads_in_index,
                                                             int k, const int* __restrict__ n_kept,
                                                             int src_start, int dst_start,
                                                             const char* const* __restrict__ src_layers,
                                                             int rows_per_piece) {
  constexpr int LPR = FC_HEAD_DIM * EB / 16;
  __shared__ int stbl[CP_TBL], dtbl[CP_TBL];
  // rows_per_piece > 0 (plain copies between buffers that cannot overlap): a column is cut into pieces of that many
  // rows, one workgroup each, so that a few long columns still fill the GPU; blockIdx.x = piece * head groups + head group
  const int head_groups = sk.num_kv_heads / HG;
  const int piece = rows_per_piece > 0 ? (int)blockIdx.x / head_groups : 0;
  const int h0 = (rows_per_piece > 0 ? (int)blockIdx.x % head_groups : (int)blockIdx.x) * HG, b = blockIdx.y;
  const int L = sk.num_layers;
  const int l = (int)blockIdx.z % L;
  const bool is_v = (int)blockIdx.z >= L;
  const KvView& src = is_v ? sv : sk;
  const KvView& dst = is_v ? dv : dk;
  const int tid = threadIdx.x, sub = tid % LPR, rg = tid / LPR;
  const int S = fc_seq_len(src, b);
  // A count read from device memory is never trusted beyond what the host validated: the index row holds
  // index_stride entries, and the destination (its block table included) max_seq_len tokens.
  int n = n_kept ? n_kept[b] : k;
  if (GATHER) n = min(n, index_stride);
  else n = min(n, S - src_start);
  n = min(n, dst.max_seq_len - dst_start);
  if (!GATHER && rows_per_piece > 0) {     // this workgroup's piece of the range
    const int first = piece * rows_per_piece;
    src_start += first;
    dst_start += first;
    n = min(n - first, rows_per_piece);
  }
  if (n <= 0) return;

  // block-table rows of this sequence (source and destination views may differ)
  const bool s_lds = src.block_tables && src.block_shift >= 0 && S > 0 && ((S - 1) >> src.block_shift) < CP_TBL;
  const int dlast = dst_start + n - 1;
  const bool d_lds = dst.block_tables && dst.block_shift >= 0 && (dlast >> dst.block_shift) < CP_TBL;
  if (s_lds)
    for (int i = tid; i <= ((S - 1) >> src.block_shift); i += CP_THREADS)
      stbl[i] = src.block_tables[(long long)b * src.table_stride + i];
  if (d_lds)
    for (int i = tid; i <= (dlast >> dst.block_shift); i += CP_THREADS)
      dtbl[i] = dst.block_tables[(long long)b * dst.table_stride + i];
  __syncthreads();

  const int hh = rg % HG, h = h0 + hh;
  const int* idx = GATHER ? indices + (((long long)l * sk.batch + b) * heads_in_index + (h % heads_in_index)) *
                                          (long long)index_stride
                          : nullptr;
  // the source's layers may be tensors of their own (a list of per-layer tensors): their addresses then come from a table
  const char* slayer = src_layers ? src_layers[l] : src.base + (long long)l * src.stride_layer * EB;
  const char* sbase = slayer + (long long)h * src.stride_head * EB + sub * 16;
  char* dbase = dst.base + ((long long)l * dst.stride_layer + (long long)h * dst.stride_head) * EB + sub * 16;
  cp_walk<EB, HG, CP_THREADS>(src, dst, stbl, s_lds, dtbl, d_lds, b, S, n, sbase, dbase, src.base + sub * 16, dst_start,
                              [&](int j) { return GATHER ? idx[j] : src_start + j; });
}

// Copies and gathers between buffers that cannot overlap need no order among their rows, and a copy is fastest on
// this part as many short-lived workgroups that each load a few rows and store them: a workgroup moves CR_V passes of
// 256 / LPR token rows of one head of one plane and ends (no loop, no barrier, no table in LDS).  Such a workgroup
// lives a few microseconds, so what it computes before its first load counts: one plane per launch (no choice between
// views), blockIdx.x / blockIdx.y = head and chunk of rows in the order the host picked (heads_fast: consecutive
// workgroups take consecutive heads of the same tokens, for a destination that keeps a token's heads together;
// otherwise consecutive chunks of one head), blockIdx.z = layer * sequences + sequence (the layer is the slowest index
// of every layout this library meets), split with a multiplier the host precomputed (exact for every z below 2^16).
// GATHER: source token = indices[j].
#ifndef CR_V
#define CR_V 1
#endif
template <int EB, bool GATHER>
__global__ __launch_bounds__(CP_THREADS) void copy_rows_kernel(KvView src, KvView dst, const int* __restrict__ indices,
                                                               int index_stride, int heads_in_index, int k,
                                                               const int* __restrict__ n_kept, int src_start,
                                                               int dst_start, const char* const* __restrict__ src_layers,
                                                               int heads_fast, unsigned long long inv_batch) {
  constexpr int LPR = FC_HEAD_DIM * EB / 16, RPP = CP_THREADS / LPR;
  const int h = heads_fast ? blockIdx.x : blockIdx.y;
  const int chunk = heads_fast ? blockIdx.y : blockIdx.x;
  const int l = (int)((blockIdx.z * inv_batch) >> 32);
  const int b = (int)blockIdx.z - l * src.batch;
  const int S = fc_seq_len(src, b);
  // a count read from device memory is never trusted beyond what the host validated
  int n = n_kept ? n_kept[b] : k;
  n = GATHER ? min(n, index_stride) : min(n, S - src_start);
  n = min(n, dst.max_seq_len - dst_start);
  const int tid = threadIdx.x, sub = tid % LPR, tg = tid / LPR;
  const int j0 = chunk * (RPP * CR_V);
  if (j0 >= n) return;
  const int* idx = GATHER ? indices + (((long long)l * src.batch + b) * heads_in_index + (h % heads_in_index)) *
                                          (long long)index_stride
                          : nullptr;
  const char* slayer = src_layers ? src_layers[l] : src.base + (long long)l * src.stride_layer * EB;
  const char* sbase = slayer + (long long)h * src.stride_head * EB + sub * 16;
  char* dbase = dst.base + ((long long)l * dst.stride_layer + (long long)h * dst.stride_head) * EB + sub * 16;
  const char* safe = slayer + sub * 16;      // the first 16-byte pieces of the layer: readable whatever the view
  cp_u32x4 buf[CR_V];
  long long doff[CR_V];
  // every lane always loads (rows that do not exist read `safe`), so that all CR_V loads are in flight together
#pragma unroll
  for (int u = 0; u < CR_V; ++u) {
    const int j = j0 + u * RPP + tg;
    long long so = -1;
    doff[u] = -1;
    if (j < n) {
      const int st = GATHER ? idx[j] : src_start + j;
      if (st >= 0 && st < S) so = fc_token_offset(src, b, st);
    }
    if (so >= 0) doff[u] = fc_token_offset(dst, b, dst_start + j);
    buf[u] = *reinterpret_cast<const cp_u32x4*>(doff[u] >= 0 ? sbase + so * EB : safe);
  }
#pragma unroll
  for (int u = 0; u < CR_V; ++u)
    if (doff[u] >= 0) *reinterpret_cast<cp_u32x4*>(dbase + doff[u] * EB) = buf[u];
}

// Whether the bytes two views can reach cannot overlap: a pool and a dense tensor never do (different tensors by
// construction of the callers), two dense tensors do not when the byte ranges they span are disjoint.  Two views of
// one pool are never taken as apart.
static bool cp_views_apart(const fc_kv_view* a, const fc_kv_view* b) {
  if ((a->block_tables == nullptr) != (b->block_tables == nullptr)) return true;
  if (a->block_tables) return false;
  const auto span = [](const fc_kv_view* v, const char*& lo, const char*& hi) {
    const int eb = v->dtype == FC_F32 ? 4 : 2;
    const long long last = (long long)(v->num_layers - 1) * v->stride_layer + (long long)(v->batch - 1) * v->stride_batch +
                           (long long)(v->num_kv_heads - 1) * v->stride_head +
                           (long long)(v->max_seq_len - 1) * v->stride_token + FC_HEAD_DIM;
    lo = (const char*)v->base;
    hi = lo + last * eb;
  };
  const char *alo, *ahi, *blo, *bhi;
  span(a, alo, ahi);
  span(b, blo, bhi);
  return ahi <= blo || bhi <= alo;
}

#ifndef CR_ONESHOT
#define CR_ONESHOT 1
#endif
// grid of the one-shot kernel for `rows` rows per column of one plane; false when the shape does not fit one launch
static bool cp_oneshot_grid(const fc_kv_view* v, int rows, bool heads_fast, dim3& grid, unsigned long long& inv_batch) {
  const int eb = v->dtype == FC_F32 ? 4 : 2;
  const int per_wg = (CP_THREADS / (FC_HEAD_DIM * eb / 16)) * CR_V;
  const long long chunks = ((long long)rows + per_wg - 1) / per_wg;
  const long long z = (long long)v->batch * v->num_layers;
  const long long x = heads_fast ? v->num_kv_heads : chunks, y = heads_fast ? chunks : v->num_kv_heads;
  if (x > 0x7fffffffLL || y > 65535 || z > 65535 || chunks < 1) return false;
  grid = dim3((unsigned)x, (unsigned)y, (unsigned)z);
  inv_batch = (0x100000000ULL + (unsigned)v->batch - 1) / (unsigned)v->batch;   // ceil(2^32 / sequences)
  return true;
}

static int check_pair(const fc_kv_view* a, const fc_kv_view* b, const char* who) {
  FC_REQUIRE(a->dtype == b->dtype && a->num_layers == b->num_layers && a->batch == b->batch &&
                 a->num_kv_heads == b->num_kv_heads,
             FC_EINVAL, "%s: views disagree on dtype/layers/batch/heads", who);
  return FC_OK;
}

extern "C" int fc_compact(const fc_kv_view* src_k, const fc_kv_view* src_v, const fc_kv_view* dst_k,
                          const fc_kv_view* dst_v, const int32_t* indices, int32_t index_stride,
                          int32_t heads_in_index, int32_t k, const int32_t* n_kept, void* stream) {
  const char* who = "fc_compact";
  int rc;
  if ((rc = fc_check_view(src_k, who)) || (rc = fc_check_view(src_v, who)) ||
      (rc = fc_check_view(dst_k, who)) || (rc = fc_check_view(dst_v, who)))
    return rc;
  if ((rc = check_pair(src_k, src_v, who)) || (rc = check_pair(src_k, dst_k, who)) ||
      (rc = check_pair(src_k, dst_v, who)))
    return rc;
  FC_REQUIRE(indices != nullptr, FC_EINVAL, "%s: null indices", who);
  FC_REQUIRE(heads_in_index == 1 || heads_in_index == src_k->num_kv_heads, FC_EINVAL,
             "%s: heads_in_index must be 1 or num_kv_heads", who);
  FC_REQUIRE(n_kept != nullptr || (k >= 0 && k <= index_stride), FC_EINVAL, "%s: k=%d vs index_stride=%d", who,
             k, index_stride);
  FC_REQUIRE((n_kept ? index_stride : k) <= dst_k->max_seq_len && (n_kept ? index_stride : k) <= dst_v->max_seq_len,
             FC_EINVAL, "%s: kept count exceeds the destination view's max_seq_len", who);
  FC_REQUIRE(src_k->num_layers * 2 <= 65535, FC_EUNSUPPORTED, "%s: too many layers", who);
  if (!n_kept && k == 0) return FC_OK;
  KvView sk = fc_make_view(src_k), sv = fc_make_view(src_v), dk = fc_make_view(dst_k), dv = fc_make_view(dst_v);
  hipStream_t st = (hipStream_t)stream;
  {  // no destination can overlap a source: rows in any order, short-lived workgroups, one launch per plane
    dim3 grid;
    unsigned long long inv;
    const bool heads_fast = dk.stride_head < dk.stride_token;
    if (CR_ONESHOT && cp_views_apart(src_k, dst_k) && cp_views_apart(src_k, dst_v) && cp_views_apart(src_v, dst_k) &&
        cp_views_apart(src_v, dst_v) && cp_oneshot_grid(src_k, n_kept ? index_stride : k, heads_fast, grid, inv)) {
      for (int plane = 0; plane < 2; ++plane) {
        const KvView& s1 = plane ? sv : sk;
        const KvView& d1 = plane ? dv : dk;
        if (src_k->dtype == FC_F32)
          hipLaunchKernelGGL((copy_rows_kernel<4, true>), grid, dim3(CP_THREADS), 0, st, s1, d1, indices, index_stride,
                             heads_in_index, k, n_kept, 0, 0, nullptr, (int)heads_fast, inv);
        else
          hipLaunchKernelGGL((copy_rows_kernel<2, true>), grid, dim3(CP_THREADS), 0, st, s1, d1, indices, index_stride,
                             heads_in_index, k, n_kept, 0, 0, nullptr, (int)heads_fast, inv);
        FC_CHECK_LAUNCH(who);
      }
      return FC_OK;
    }
  }
  // 512-byte (fp32) rows: two heads per workgroup measured faster, as long as the grid stays large
  const long long cols = 2LL * src_k->num_layers * src_k->batch * src_k->num_kv_heads;
  if (src_k->dtype == FC_F32 && src_k->num_kv_heads % 2 == 0 && cols >= 2048) {
    dim3 grid(src_k->num_kv_heads / 2, src_k->batch, src_k->num_layers * 2);
    hipLaunchKernelGGL((compact_kernel<4, true, 2>), grid, dim3(CP_THREADS), 0, st, sk, sv, dk, dv, indices,
                       index_stride, heads_in_index, k, n_kept, 0, 0, nullptr, 0);
  } else {
    dim3 grid(src_k->num_kv_heads, src_k->batch, src_k->num_layers * 2);
    if (src_k->dtype == FC_F32)
      hipLaunchKernelGGL((compact_kernel<4, true, 1>), grid, dim3(CP_THREADS), 0, st, sk, sv, dk, dv, indices,
                         index_stride, heads_in_index, k, n_kept, 0, 0, nullptr, 0);
    else
      hipLaunchKernelGGL((compact_kernel<2, true, 1>), grid, dim3(CP_THREADS), 0, st, sk, sv, dk, dv, indices,
                         index_stride, heads_in_index, k, n_kept, 0, 0, nullptr, 0);
  }
  FC_CHECK_LAUNCH(who);
  return FC_OK;
}

static int copy_tokens_impl(const char* who, const void* const* src_layers, const fc_kv_view* src, const fc_kv_view* dst,
                            int32_t seg_start, int32_t count, int32_t dst_start, void* stream) {
  int rc;
  if ((rc = fc_check_view(src, who)) || (rc = fc_check_view(dst, who)) || (rc = check_pair(src, dst, who)))
    return rc;
  FC_REQUIRE(seg_start >= 0 && dst_start >= 0 && count >= 0, FC_EINVAL, "%s: negative range", who);
  FC_REQUIRE((int64_t)dst_start + count <= dst->max_seq_len, FC_EINVAL,
             "%s: destination range [%d, %d) exceeds max_seq_len %d", who, dst_start, dst_start + count,
             dst->max_seq_len);
  if (count == 0) return FC_OK;
  KvView s = fc_make_view(src), d = fc_make_view(dst);
  // A pool and a dense tensor (or a list of per-layer tensors) do not overlap, so the order of the rows does not matter
  // and a long column can be cut into pieces: enough of them for about eight workgroups per compute unit, none
  // shorter than 512 rows.
  int rows_per_piece = 0, pieces = 1;
  const bool apart = src_layers || cp_views_apart(src, dst);
  hipStream_t st = (hipStream_t)stream;
  {
    dim3 grid;
    unsigned long long inv;
    const bool heads_fast = d.stride_head < d.stride_token;
    if (CR_ONESHOT && apart && cp_oneshot_grid(src, count, heads_fast, grid, inv)) {
      if (src->dtype == FC_F32)
        hipLaunchKernelGGL((copy_rows_kernel<4, false>), grid, dim3(CP_THREADS), 0, st, s, d, nullptr, 0, 1, count, nullptr,
                           seg_start, dst_start, (const char* const*)src_layers, (int)heads_fast, inv);
      else
        hipLaunchKernelGGL((copy_rows_kernel<2, false>), grid, dim3(CP_THREADS), 0, st, s, d, nullptr, 0, 1, count, nullptr,
                           seg_start, dst_start, (const char* const*)src_layers, (int)heads_fast, inv);
      FC_CHECK_LAUNCH(who);
      return FC_OK;
    }
  }
  if (apart) {
    const long long cols = (long long)src->num_kv_heads * src->batch * src->num_layers;
    const long long want = (2048 + cols - 1) / cols;
    pieces = (int)(want < 1 ? 1 : (want > (count + 511) / 512 ? (count + 511) / 512 : want));
    if (pieces > 1) {
      rows_per_piece = (count + pieces - 1) / pieces;
      pieces = (count + rows_per_piece - 1) / rows_per_piece;
    }
  }
  // one plane per launch: z covers the layers only
  dim3 grid(src->num_kv_heads * pieces, src->batch, src->num_layers);
  if (src->dtype == FC_F32)
    hipLaunchKernelGGL((compact_kernel<4, false, 1>), grid, dim3(CP_THREADS), 0, st, s, s, d, d, nullptr, 0, 1, count,
                       nullptr, seg_start, dst_start, (const char* const*)src_layers, rows_per_piece);
  else
    hipLaunchKernelGGL((compact_kernel<2, false, 1>), grid, dim3(CP_THREADS), 0, st, s, s, d, d, nullptr, 0, 1, count,
                       nullptr, seg_start, dst_start, (const char* const*)src_layers, rows_per_piece);
  FC_CHECK_LAUNCH(who);
  return FC_OK;
}

extern "C" int fc_copy_tokens(const fc_kv_view* src, const fc_kv_view* dst, int32_t seg_start, int32_t count,
                              int32_t dst_start, void* stream) {
  return copy_tokens_impl("fc_copy_tokens", nullptr, src, dst, seg_start, count, dst_start, stream);
}

extern "C" int fc_copy_tokens_from_layers(const void* const* src_layers, const fc_kv_view* src, const fc_kv_view* dst,
                                          int32_t seg_start, int32_t count, int32_t dst_start, void* stream) {
  const char* who = "fc_copy_tokens_from_layers";
  FC_REQUIRE(src_layers, FC_EINVAL, "%s: null layer table", who);
  FC_REQUIRE(src && src->block_tables == nullptr, FC_EINVAL, "%s: the per-layer tensors must be dense", who);
  return copy_tokens_impl(who, src_layers, src, dst, seg_start, count, dst_start, stream);
}
