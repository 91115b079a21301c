// Gather/compaction of kept K/V rows, and plain ordered token copies.
//
// One workgroup per (K|V, layer, sequence, kv head) column (per pair of heads for 512-byte fp32 rows).  A token row of one head is 128
// elements (256 or 512 bytes) and is moved by 16 or 32 lanes with 16-byte accesses.  The column is
// walked in ascending chunks: all source rows of a chunk are loaded into registers, the
// workgroup waits for the loads and synchronises, and only then are the chunk's destination
// rows stored (while the next chunk's loads are already in flight).  With ascending unique indices (dst j <= src idx[j]) this makes the in-place case
// (dst aliases src) safe: a chunk's stores can only hit rows whose reads have already completed,
// and later chunks read rows that no earlier chunk writes.  Different heads, layers and K/V planes
// touch disjoint bytes, so columns need no ordering between each other.
#include "fc_common.h"

typedef unsigned cp_u32x4 __attribute__((ext_vector_type(4)));   // native vector: arrays of it stay in registers

#define CP_THREADS 256
#ifndef CP_R
#define CP_R 8      // 16-byte loads in flight per lane and chunk
#endif
#define CP_TBL 1024 // block-table entries of one sequence cached in LDS (per view)

// The loaded registers are not consumed before the barrier, so wait for them explicitly.  The stores
// of the previous chunk were issued AFTER these loads; when every lane of the wavefront issued all
// CP_R of them (stores_behind), the loads are complete as soon as at most CP_R operations are still
// outstanding, and the stores' completion is not waited for.
__device__ __forceinline__ void cp_wait_then_barrier(bool stores_behind) {
  if (stores_behind)
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(CP_R) : "memory");
  else
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

__device__ __forceinline__ long long cp_offset(const KvView& v, const int* tbl, bool tbl_lds, int b, int s) {
  if (tbl_lds) {
    const int blk = tbl[s >> v.block_shift];
    return blk < 0 ? -1 : (long long)blk * v.stride_block + (long long)(s & (v.block_size - 1)) * v.stride_token;
  }
  return fc_token_offset(v, b, s);
}

// GATHER: src token = indices[j]; otherwise src token = src_start + j.
// The column is walked in chunks of CH rows with two register buffers: the loads of chunk c+1 are
// issued right after the barrier that releases the stores of chunk c, so loads and stores overlap.
// HG = consecutive kv heads handled by one workgroup (divides num_kv_heads)
template <int EB, bool GATHER, int HG>
__global__ __launch_bounds__(CP_THREADS) void compact_kernel(KvView sk, KvView sv, KvView dk, KvView dv,
                                                             const int* __restrict__ indices,
                                                             int index_stride, int heads_in_index,
                                                             int k, const int* __restrict__ n_kept,
                                                             int src_start, int dst_start) {
  constexpr int LPR = FC_HEAD_DIM * EB / 16;
  constexpr int RPP = CP_THREADS / LPR;
  constexpr int CH = RPP * CP_R / HG;   // tokens per chunk
  __shared__ int stbl[CP_TBL], dtbl[CP_TBL];
  const int h0 = blockIdx.x * HG, b = blockIdx.y;
  const int L = sk.num_layers;
  const int l = blockIdx.z % L;
  const bool is_v = blockIdx.z >= L;
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

  // rows of a chunk are (token j, head) pairs with the head fastest, so that the HG head rows of a
  // token (contiguous in memory) are moved by neighbouring lanes
  const int hh = rg % HG, h = h0 + hh;
  const int* idx = GATHER ? indices + (((long long)l * sk.batch + b) * heads_in_index + (h % heads_in_index)) *
                                          (long long)index_stride
                          : nullptr;
  const char* sbase = src.base + ((long long)l * src.stride_layer + (long long)h * src.stride_head) * EB + sub * 16;
  char* dbase = dst.base + ((long long)l * dst.stride_layer + (long long)h * dst.stride_head) * EB + sub * 16;
  constexpr int TPP = RPP / HG;   // tokens per pass
  const int tg = rg / HG;

  auto load_idx = [&](int (&si)[CP_R], int j0) {
#pragma unroll
    for (int u = 0; u < CP_R; ++u) {
      const int j = j0 + u * TPP + tg;
      si[u] = j < n ? (GATHER ? idx[j] : src_start + j) : -1;
    }
  };
  // Every lane always loads (rows that do not exist read the view's first bytes instead) and the validity
  // goes into a bit mask: with no control flow around the buffer elements they stay in registers.
  const char* safe = src.base + sub * 16;
  auto load_rows = [&](cp_u32x4 (&buf)[CP_R], unsigned& ok, const int (&si)[CP_R]) {
    ok = 0;
#pragma unroll
    for (int u = 0; u < CP_R; ++u) {
      const int s = si[u];
      long long off = -1;
      if (s >= 0 && s < S) off = cp_offset(src, stbl, s_lds, b, s);
      const bool valid = off >= 0;
      const char* p = valid ? sbase + off * EB : safe;
      buf[u] = *reinterpret_cast<const cp_u32x4*>(p);
      ok |= valid ? (1u << u) : 0u;
    }
  };
  // returns whether every lane of this wavefront stored all CP_R rows
  auto store_rows = [&](const cp_u32x4 (&buf)[CP_R], unsigned ok, int j0) {
    bool all = true;
#pragma unroll
    for (int u = 0; u < CP_R; ++u) {
      const int j = j0 + u * TPP + tg;
      long long off = -1;
      if (ok & (1u << u)) off = cp_offset(dst, dtbl, d_lds, b, dst_start + j);
      if (off >= 0) *reinterpret_cast<cp_u32x4*>(dbase + off * EB) = buf[u];
      all &= off >= 0;
    }
    return (bool)__all(all);
  };

  cp_u32x4 bufa[CP_R], bufb[CP_R];
  unsigned oka, okb;
  int sia[CP_R], sib[CP_R];
  load_idx(sia, 0);
  load_rows(bufa, oka, sia);
  load_idx(sib, CH);
  bool behind = false;   // the newest operations in flight are exactly CP_R stores of this wavefront
  for (int j0 = 0; j0 < n; j0 += 2 * CH) {
    // chunk j0 is in flight in buffer a; the indices of chunk j0 + CH are in sib
    cp_wait_then_barrier(behind);
    if (j0 + CH < n) load_rows(bufb, okb, sib);
    load_idx(sia, j0 + 2 * CH);
    behind = store_rows(bufa, oka, j0);
    if (j0 + CH >= n) break;
    cp_wait_then_barrier(behind);
    if (j0 + 2 * CH < n) load_rows(bufa, oka, sia);
    load_idx(sib, j0 + 3 * CH);
    behind = store_rows(bufb, okb, j0 + CH);
  }
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
  // 512-byte (fp32) rows: two heads per workgroup measured faster, as long as the grid stays large
  const long long cols = 2LL * src_k->num_layers * src_k->batch * src_k->num_kv_heads;
  if (src_k->dtype == FC_F32 && src_k->num_kv_heads % 2 == 0 && cols >= 2048) {
    dim3 grid(src_k->num_kv_heads / 2, src_k->batch, src_k->num_layers * 2);
    hipLaunchKernelGGL((compact_kernel<4, true, 2>), grid, dim3(CP_THREADS), 0, st, sk, sv, dk, dv, indices,
                       index_stride, heads_in_index, k, n_kept, 0, 0);
  } else {
    dim3 grid(src_k->num_kv_heads, src_k->batch, src_k->num_layers * 2);
    if (src_k->dtype == FC_F32)
      hipLaunchKernelGGL((compact_kernel<4, true, 1>), grid, dim3(CP_THREADS), 0, st, sk, sv, dk, dv, indices,
                         index_stride, heads_in_index, k, n_kept, 0, 0);
    else
      hipLaunchKernelGGL((compact_kernel<2, true, 1>), grid, dim3(CP_THREADS), 0, st, sk, sv, dk, dv, indices,
                         index_stride, heads_in_index, k, n_kept, 0, 0);
  }
  FC_CHECK_LAUNCH(who);
  return FC_OK;
}

extern "C" int fc_copy_tokens(const fc_kv_view* src, const fc_kv_view* dst, int32_t seg_start, int32_t count,
                              int32_t dst_start, void* stream) {
  const char* who = "fc_copy_tokens";
  int rc;
  if ((rc = fc_check_view(src, who)) || (rc = fc_check_view(dst, who)) || (rc = check_pair(src, dst, who)))
    return rc;
  FC_REQUIRE(seg_start >= 0 && dst_start >= 0 && count >= 0, FC_EINVAL, "%s: negative range", who);
  FC_REQUIRE((int64_t)dst_start + count <= dst->max_seq_len, FC_EINVAL,
             "%s: destination range [%d, %d) exceeds max_seq_len %d", who, dst_start, dst_start + count,
             dst->max_seq_len);
  if (count == 0) return FC_OK;
  KvView s = fc_make_view(src), d = fc_make_view(dst);
  // one plane per launch: z covers the layers only
  dim3 grid(src->num_kv_heads, src->batch, src->num_layers);
  hipStream_t st = (hipStream_t)stream;
  if (src->dtype == FC_F32)
    hipLaunchKernelGGL((compact_kernel<4, false, 1>), grid, dim3(CP_THREADS), 0, st, s, s, d, d, nullptr, 0, 1, count,
                       nullptr, seg_start, dst_start);
  else
    hipLaunchKernelGGL((compact_kernel<2, false, 1>), grid, dim3(CP_THREADS), 0, st, s, s, d, d, nullptr, 0, 1, count,
                       nullptr, seg_start, dst_start);
  FC_CHECK_LAUNCH(who);
  return FC_OK;
}
