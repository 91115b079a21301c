// Knorm token scoring: one pass over K, HBM-bound.
//
// A workgroup owns a tile of TS consecutive tokens of one (layer, sequence) and all KV heads.
// A token-head row is 128 elements = 512 B (fp32) or 256 B (fp16/bf16): it is read by 32 or 16
// lanes with one 16-byte load each, squared and reduced across those lanes in fp32.  The tile's
// scores are staged in LDS so that each head's TS scores leave as one contiguous segment.
#include "fc_common.h"

#define KN_TS 32
#define KN_THREADS 256

template <int DTYPE>
__device__ __forceinline__ float row_sumsq_part(const char* p) {
  // p points at this lane's 16 bytes of the row
  if (DTYPE == FC_F32) {
    float4 x = *reinterpret_cast<const float4*>(p);
    return x.x * x.x + x.y * x.y + x.z * x.z + x.w * x.w;
  } else {
    uint4 x = *reinterpret_cast<const uint4*>(p);
    unsigned w[4] = {x.x, x.y, x.z, x.w};
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float lo, hi;
      if (DTYPE == FC_BF16) {
        lo = fc_bf16_to_float((unsigned short)(w[i] & 0xffff));
        hi = fc_bf16_to_float((unsigned short)(w[i] >> 16));
      } else {
        lo = fc_half_to_float((unsigned short)(w[i] & 0xffff));
        hi = fc_half_to_float((unsigned short)(w[i] >> 16));
      }
      acc += lo * lo;
      acc += hi * hi;
    }
    return acc;
  }
}

template <int DTYPE>
__device__ __forceinline__ float round_to_storage(float x) {
  if (DTYPE == FC_BF16) return fc_bf16_to_float(fc_float_to_bf16(x));
  if (DTYPE == FC_F16) return fc_half_to_float(fc_float_to_half(x));
  return x;
}

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

  const int rows = KN_TS * H;
  for (int r0 = 0; r0 < rows; r0 += RPP) {
    int r = r0 + rg;
    float part = 0.f;
    int t = 0, h = 0;
    bool live = false;
    if (r < rows) {
      if (head_fast) { t = r / H; h = r - t * H; } else { h = r / KN_TS; t = r - h * KN_TS; }
      int s = s0 + t;
      if (s < S) {
        long long off = fc_token_offset(kv, b, s);
        if (off >= 0) {
          live = true;
          part = row_sumsq_part<DTYPE>(base + (off + (long long)h * kv.stride_head) * EB + sub * 16);
        }
      }
    }
#pragma unroll
    for (int o = LPR / 2; o > 0; o >>= 1) part += __shfl_xor(part, o, 64);
    if (r < rows && sub == 0) {
      float v;
      if (!live) v = -INFINITY;
      else if (MEAN) v = round_to_storage<DTYPE>(sqrtf(part));
      else v = -sqrtf(part);
      sc[h * (KN_TS + 1) + t] = v;
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
