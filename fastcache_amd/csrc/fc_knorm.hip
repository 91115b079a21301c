// Knorm token scoring: one pass over K, HBM-bound.
//
// A workgroup owns a tile of TS consecutive tokens of one (layer, sequence) and all KV heads.
// A token-head row is 128 elements = 512 B (fp32) or 256 B (fp16/bf16): it is read by 32 or 16
// lanes with one 16-byte load each, squared and reduced across those lanes in fp32.  The tile's
// scores are staged in LDS so that each head's TS scores leave as one contiguous segment.
#include "fc_norm.h"

#define KN_TS 16   // tokens per workgroup tile: small enough that short caches still give thousands of workgroups
#define KN_THREADS 256
#define KN_U 4     // rows per lane and pass

// MEAN == false: scores[l][b][h][s] = -norm.   MEAN == true: out[l][b][s] = mean_h norm, with the
// per-head norm and the mean each rounded to the storage dtype (torch's keys.norm().mean(1)).
template <int DTYPE, bool MEAN>
__global__ __launch_bounds__(KN_THREADS) void knorm_kernel(KvView kv, float* __restrict__ out,
                                                           int score_stride) {
  constexpr int EB = (DTYPE == FC_F32) ? 4 : 2;
  constexpr int LPR = FC_HEAD_DIM * EB / 16;  // lanes per row
  constexpr int RPP = KN_THREADS / LPR;       // rows per pass
  extern __shared__ float sc[];               // [H][KN_TS + 1]

  const int l = blockIdx.z, b = blockIdx.y;
  const int s0 = blockIdx.x * KN_TS;
  const int H = kv.num_kv_heads;
  const int S = fc_seq_len(kv, b);
  const int tid = threadIdx.x;
  const int sub = tid % LPR, rg = tid / LPR;
  const bool head_fast = kv.stride_head <= kv.stride_token;
  const char* base = kv.base + (long long)l * kv.stride_layer * EB;

  // KN_U rows per lane and pass: all their loads are issued (unconditionally, a dead row re-reads a
  // valid one) before the first is reduced, so that a lane keeps several 16-byte loads in flight.
  const int rows = KN_TS * H;
  for (int r0 = 0; r0 < rows; r0 += RPP * KN_U) {
    uint4 x[KN_U];
    bool live[KN_U];
    int tt[KN_U], hh[KN_U];
#pragma unroll
    for (int u = 0; u < KN_U; ++u) {
      const int r = r0 + u * RPP + rg;
      const int rc = min(r, rows - 1);
      int t, h;
      if (head_fast) { t = rc / H; h = rc - t * H; } else { h = rc / KN_TS; t = rc - h * KN_TS; }
      const int s = s0 + t;
      long long off = fc_token_offset(kv, b, max(min(s, S - 1), 0));
      live[u] = r < rows && s < S && off >= 0;
      off = off < 0 ? 0 : off;
      tt[u] = t;
      hh[u] = h;
      x[u] = *reinterpret_cast<const uint4*>(base + (off + (long long)h * kv.stride_head) * EB + sub * 16);
    }
#pragma unroll
    for (int u = 0; u < KN_U; ++u) {
      float part = fc_group_sum<16>(row_sumsq_part<DTYPE>(x[u]));
      if (LPR == 32) part += __shfl_xor(part, 16, 64);
      if (r0 + u * RPP + rg < rows && sub == 0) {
        float v;
        if (!live[u]) v = -INFINITY;
        else if (MEAN) v = round_to_storage<DTYPE>(sqrtf(part));
        else v = -sqrtf(part);
        sc[hh[u] * (KN_TS + 1) + tt[u]] = v;
      }
    }
  }
  __syncthreads();
  if (!MEAN) {
    for (int i = tid; i < rows; i += KN_THREADS) {
      int h = i / KN_TS, t = i - h * KN_TS;
      int s = s0 + t;
      if (s < score_stride)
        out[(((long long)l * kv.batch + b) * H + h) * score_stride + s] = sc[h * (KN_TS + 1) + t];
    }
  } else {
    if (tid < KN_TS) {
      int s = s0 + tid;
      if (s < score_stride) {
        float v = -INFINITY;
        if (s < S) {
          float acc = 0.f;
          for (int h = 0; h < H; ++h) acc += sc[h * (KN_TS + 1) + tid];
          v = round_to_storage<DTYPE>(acc / (float)H);
        }
        out[((long long)l * kv.batch + b) * score_stride + s] = v;
      }
    }
  }
}

template <bool MEAN>
static int launch_knorm(const fc_kv_view* keys, float* out, int32_t score_stride, void* stream,
                        const char* who) {
  int rc = fc_check_view(keys, who);
  if (rc) return rc;
  FC_REQUIRE(out != nullptr, FC_EINVAL, "%s: null output", who);
  FC_REQUIRE(score_stride >= keys->max_seq_len, FC_EINVAL, "%s: score_stride %d < max_seq_len %d", who,
             score_stride, keys->max_seq_len);
  FC_REQUIRE(keys->num_kv_heads <= 256, FC_EUNSUPPORTED, "%s: more than 256 kv heads", who);
  if (score_stride == 0) return FC_OK;
  KvView kv = fc_make_view(keys);
  dim3 grid((score_stride + KN_TS - 1) / KN_TS, keys->batch, keys->num_layers);
  size_t lds = (size_t)keys->num_kv_heads * (KN_TS + 1) * sizeof(float);
  hipStream_t st = (hipStream_t)stream;
  switch (keys->dtype) {
    case FC_F32: hipLaunchKernelGGL((knorm_kernel<FC_F32, MEAN>), grid, dim3(KN_THREADS), lds, st, kv, out, score_stride); break;
    case FC_F16: hipLaunchKernelGGL((knorm_kernel<FC_F16, MEAN>), grid, dim3(KN_THREADS), lds, st, kv, out, score_stride); break;
    default: hipLaunchKernelGGL((knorm_kernel<FC_BF16, MEAN>), grid, dim3(KN_THREADS), lds, st, kv, out, score_stride); break;
  }
  FC_CHECK_LAUNCH(who);
  return FC_OK;
}

extern "C" int fc_knorm_score(const fc_kv_view* keys, float* scores, int32_t score_stride, void* stream) {
  return launch_knorm<false>(keys, scores, score_stride, stream, "fc_knorm_score");
}

extern "C" int fc_knorm_mean_score(const fc_kv_view* keys, float* out, int32_t score_stride, void* stream) {
  return launch_knorm<true>(keys, out, score_stride, stream, "fc_knorm_mean_score");
}

// ---- observed attention: column sums of a materialised attention matrix -----------------------------
// out[b][hk][s] = mean over the G query heads of the kv group of ( sum over queries q of attn[b][h][q][s] )
//                 / (number of queries that can attend key s under the causal mask = Sk - s).
// One thread per key column, 256 columns per workgroup, rows read coalesced; the query range is split
// over gridDim.z slices that are combined with a fixed-order second pass (deterministic, no atomics).
template <int DTYPE>
__global__ __launch_bounds__(256) void attn_colsum_kernel(const char* __restrict__ attn, int Hq, int G, int Sq, int Sk,
                                                          int qsplit, float* __restrict__ partial) {
  const int s = blockIdx.x * 256 + threadIdx.x;
  const int hk = blockIdx.y % (Hq / G), b = blockIdx.y / (Hq / G);
  const int slice = blockIdx.z;
  if (s >= Sk) return;
  const int q0 = (int)((long long)Sq * slice / qsplit), q1 = (int)((long long)Sq * (slice + 1) / qsplit);
  float acc = 0.f;
  for (int g = 0; g < G; ++g) {
    const long long base = (((long long)b * Hq + hk * G + g) * Sq) * Sk + s;
    float a = 0.f;
    for (int q = q0; q < q1; ++q) {
      const long long i = base + (long long)q * Sk;
      if constexpr (DTYPE == FC_F32) a += reinterpret_cast<const float*>(attn)[i];
      else {
        const unsigned short r = reinterpret_cast<const unsigned short*>(attn)[i];
        a += DTYPE == FC_BF16 ? fc_bf16_to_float(r) : fc_half_to_float(r);
      }
    }
    acc += a;
  }
  partial[(((long long)slice * gridDim.y + blockIdx.y)) * Sk + s] = acc;
}

__global__ __launch_bounds__(256) void attn_colsum_finish_kernel(const float* __restrict__ partial, int rows, int Sk,
                                                                 int qsplit, int G, float* __restrict__ out) {
  const int s = blockIdx.x * 256 + threadIdx.x;
  const int r = blockIdx.y;
  if (s >= Sk) return;
  float acc = 0.f;
  for (int k = 0; k < qsplit; ++k) acc += partial[((long long)k * rows + r) * Sk + s];
  out[(long long)r * Sk + s] = acc / (float)(Sk - s) / (float)G;
}

extern "C" int64_t fc_observed_attention_workspace_bytes(int32_t batch, int32_t num_kv_heads, int32_t sk) {
  if (batch <= 0 || num_kv_heads <= 0 || sk <= 0) return 0;
  return (int64_t)16 * batch * num_kv_heads * sk * 4;
}

extern "C" int fc_observed_attention_score(const void* attn, int32_t batch, int32_t num_q_heads, int32_t num_kv_heads,
                                           int32_t sq, int32_t sk, int32_t dtype, float* scores, void* workspace,
                                           int64_t workspace_bytes, void* stream) {
  const char* who = "fc_observed_attention_score";
  FC_REQUIRE(attn && scores && workspace, FC_EINVAL, "%s: null pointer", who);
  FC_REQUIRE(batch > 0 && num_kv_heads > 0 && num_q_heads > 0 && num_q_heads % num_kv_heads == 0 && sq > 0 && sk > 0,
             FC_EINVAL, "%s: bad sizes", who);
  FC_REQUIRE(dtype == FC_F32 || dtype == FC_F16 || dtype == FC_BF16, FC_EUNSUPPORTED, "%s: dtype %d", who, dtype);
  FC_REQUIRE(workspace_bytes >= fc_observed_attention_workspace_bytes(batch, num_kv_heads, sk), FC_EINVAL,
             "%s: workspace too small", who);
  FC_REQUIRE((long long)batch * num_kv_heads <= 65535, FC_EUNSUPPORTED, "%s: too many (batch, head) rows", who);
  const int rows = batch * num_kv_heads;
  const int col_blocks = (sk + 255) / 256;
  // enough query slices to fill the chip (at most 16, what the workspace holds)
  int qsplit = 1;
  while (qsplit < 16 && (long long)col_blocks * rows * qsplit < 2048 && qsplit * 64 <= sq) qsplit *= 2;
  const int G = num_q_heads / num_kv_heads;
  hipStream_t st = (hipStream_t)stream;
  dim3 grid(col_blocks, rows, qsplit);
  if (dtype == FC_F32)
    hipLaunchKernelGGL((attn_colsum_kernel<FC_F32>), grid, dim3(256), 0, st, (const char*)attn, num_q_heads, G, sq, sk,
                       qsplit, (float*)workspace);
  else if (dtype == FC_F16)
    hipLaunchKernelGGL((attn_colsum_kernel<FC_F16>), grid, dim3(256), 0, st, (const char*)attn, num_q_heads, G, sq, sk,
                       qsplit, (float*)workspace);
  else
    hipLaunchKernelGGL((attn_colsum_kernel<FC_BF16>), grid, dim3(256), 0, st, (const char*)attn, num_q_heads, G, sq, sk,
                       qsplit, (float*)workspace);
  hipLaunchKernelGGL(attn_colsum_finish_kernel, dim3(col_blocks, rows), dim3(256), 0, st, (const float*)workspace, rows,
                     sk, qsplit, G, scores);
  FC_CHECK_LAUNCH(who);
  return FC_OK;
}
