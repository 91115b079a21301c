// Gather/compaction of kept K/V rows, and plain ordered token copies.
//
// One workgroup per (K|V, layer, sequence, kv head) column.  A token row of one head is 128
// elements (256 or 512 bytes) and is moved by 16 or 32 lanes with 16-byte accesses.  The column is
// walked in ascending chunks: all source rows of a chunk are loaded into registers, the
// workgroup waits for the loads and synchronises, and only then are the chunk's destination
// rows stored.  With ascending unique indices (dst j <= src idx[j]) this makes the in-place case
// (dst aliases src) safe: a chunk's stores can only hit rows whose reads have already completed,
// and later chunks read rows that no earlier chunk writes.  Different heads, layers and K/V planes
// touch disjoint bytes, so columns need no ordering between each other.
#include "fc_common.h"

#define CP_THREADS 256
#define CP_R 8  // 16-byte loads in flight per lane

__device__ __forceinline__ void cp_wait_loads_then_barrier() {
  // the loaded registers are not consumed before the barrier, so wait for them explicitly
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
}

// GATHER: src token = indices[j]; otherwise src token = src_start + j.
template <int EB, bool GATHER>
__global__ __launch_bounds__(CP_THREADS) void compact_kernel(KvView sk, KvView sv, KvView dk, KvView dv,
                                                             const int* __restrict__ indices,
                                                             int index_stride, int heads_in_index,
                                                             int k, const int* __restrict__ n_kept,
                                                             int src_start, int dst_start) {
  constexpr int LPR = FC_HEAD_DIM * EB / 16;
  constexpr int RPP = CP_THREADS / LPR;
  constexpr int CH = RPP * CP_R;
  const int h = blockIdx.x, b = blockIdx.y;
  const int L = sk.num_layers;
  const int l = blockIdx.z % L;
  const bool is_v = blockIdx.z >= L;
  const KvView& src = is_v ? sv : sk;
  const KvView& dst = is_v ? dv : dk;
  const int tid = threadIdx.x, sub = tid % LPR, rg = tid / LPR;
  const int S = fc_seq_len(src, b);
  int n = n_kept ? n_kept[b] : k;
  if (!GATHER) n = min(n, S - src_start);
  if (n <= 0) return;
  const int* idx = GATHER ? indices + (((long long)l * sk.batch + b) * heads_in_index + (h % heads_in_index)) *
                                          (long long)index_stride
                          : nullptr;
  const char* sbase = src.base + ((long long)l * src.stride_layer + (long long)h * src.stride_head) * EB + sub * 16;
  char* dbase = dst.base + ((long long)l * dst.stride_layer + (long long)h * dst.stride_head) * EB + sub * 16;

  for (int j0 = 0; j0 < n; j0 += CH) {
    uint4 buf[CP_R];
    bool ok[CP_R];
#pragma unroll
    for (int u = 0; u < CP_R; ++u) {
      const int j = j0 + u * RPP + rg;
      ok[u] = false;
      if (j < n) {
        const int s = GATHER ? idx[j] : src_start + j;
        if (s >= 0 && s < S) {
          const long long off = fc_token_offset(src, b, s);
          if (off >= 0) {
            buf[u] = *reinterpret_cast<const uint4*>(sbase + off * EB);
            ok[u] = true;
          }
        }
      }
    }
    cp_wait_loads_then_barrier();
#pragma unroll
    for (int u = 0; u < CP_R; ++u) {
      const int j = j0 + u * RPP + rg;
      if (ok[u]) {
        const long long off = fc_token_offset(dst, b, dst_start + j);
        if (off >= 0) *reinterpret_cast<uint4*>(dbase + off * EB) = buf[u];
      }
    }
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
  dim3 grid(src_k->num_kv_heads, src_k->batch, src_k->num_layers * 2);
  hipStream_t st = (hipStream_t)stream;
  if (src_k->dtype == FC_F32)
    hipLaunchKernelGGL((compact_kernel<4, true>), grid, dim3(CP_THREADS), 0, st, sk, sv, dk, dv, indices,
                       index_stride, heads_in_index, k, n_kept, 0, 0);
  else
    hipLaunchKernelGGL((compact_kernel<2, true>), grid, dim3(CP_THREADS), 0, st, sk, sv, dk, dv, indices,
                       index_stride, heads_in_index, k, n_kept, 0, 0);
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
    hipLaunchKernelGGL((compact_kernel<4, false>), grid, dim3(CP_THREADS), 0, st, s, s, d, d, nullptr, 0, 1, count,
                       nullptr, seg_start, dst_start);
  else
    hipLaunchKernelGGL((compact_kernel<2, false>), grid, dim3(CP_THREADS), 0, st, s, s, d, d, nullptr, 0, 1, count,
                       nullptr, seg_start, dst_start);
  FC_CHECK_LAUNCH(who);
  return FC_OK;
}
