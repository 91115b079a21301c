// Expected-attention scoring for fp16/bf16 caches: how much attention a key can expect from FUTURE
// queries, modelled as Gaussian with mean mu and covariance C per query head.  For key k of head h
//   z[k]     = mu . k / sqrt(d)  +  k^T C k / (2 d)        (log of the expected unnormalised weight)
//   p[k]     = softmax over the keys past the first n_sink
//   score[k] = (mean over the query heads of the group of p[k] + epsilon) * ||v[k]||
// and the first n_sink keys get the largest score of the whole layer, so they are never pruned.
//
// Kernel 1 (logits) holds one head's C in LDS, split into two 16-bit halves (hi + lo, so the products
// carry ~16-22 mantissa bits), and walks the keys 32 per wavefront:
//   U^T = C * K^T          v_mfma_f32_32x32x16, A = rows of C from LDS, B = key rows straight from memory;
//   z   = sum_j K[k][j] * (U^T[j][k] + 2 sqrt(d) mu[j]) / (2 d)
// The accumulators start from the mu term, so the linear part costs nothing extra; a lane owns one key
// (column) and 64 of the 128 j, the two half-waves are added at the end.
// Kernel 2 (finish) is one workgroup per (sequence, kv head): softmax statistics of the group's rows,
// then 16 lanes per key: the value row's norm and the group mean of the probabilities.
// Kernel 3 writes the sink scores once the layer's maximum is known.
#include "fc_common.h"


#define EA_WAVES 8
#define EA_THREADS (EA_WAVES * 64)
#define EA_ROWB 272               // LDS bytes per row of C: 128 elements + 16 bytes of padding
#define EA_CBYTES (128 * EA_ROWB)
#define EA_KEYS_PER_WG 2048       // keys one workgroup walks with its copy of C
#define EA_LDS (2 * EA_CBYTES + 128 * 4)

template <int DTYPE>
__device__ __forceinline__ float ea_to_float(unsigned short h) {
  return DTYPE == FC_BF16 ? fc_bf16_to_float(h) : fc_half_to_float(h);
}
template <int DTYPE>
__device__ __forceinline__ unsigned short ea_from_float(float f) {
  return DTYPE == FC_BF16 ? fc_float_to_bf16(f) : fc_float_to_half(f);
}

template <int DTYPE>
__global__ __launch_bounds__(EA_THREADS) void ea_logits_kernel(KvView kv, const float* __restrict__ mu,
                                                               const float* __restrict__ cov, int Hq, int n_sink,
                                                               float* __restrict__ raw, int raw_stride,
                                                               unsigned* __restrict__ gmax) {
  extern __shared__ __align__(16) char smem[];
  char* chi = smem;
  char* clo = smem + EA_CBYTES;
  float* mus = reinterpret_cast<float*>(smem + 2 * EA_CBYTES);

  const int hq = blockIdx.y;
  const int b = blockIdx.z % kv.batch, l = blockIdx.z / kv.batch;
  const int Hkv = kv.num_kv_heads, G = Hq / Hkv, h = hq / G;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lrow = lane & 31, lhalf = lane >> 5;
  if (blockIdx.x == 0 && hq == 0 && b == 0 && tid == 0) gmax[l] = 0u;   // the finish kernel takes maxima into it

  const int S = fc_seq_len(kv, b);
  const int k0 = n_sink + blockIdx.x * EA_KEYS_PER_WG;
  if (k0 >= S) return;
  const int k1 = min(S, k0 + EA_KEYS_PER_WG);

  const long long head = ((long long)l * kv.batch + b) * Hq + hq;
  const float beta = 2.f * sqrtf((float)FC_HEAD_DIM);
  if (tid < FC_HEAD_DIM) mus[tid] = mu[head * FC_HEAD_DIM + tid] * beta;
  if (cov) {
    const float* c = cov + head * FC_HEAD_DIM * FC_HEAD_DIM;
    for (int i = tid; i < FC_HEAD_DIM * FC_HEAD_DIM / 2; i += EA_THREADS) {
      const int r = i >> 6, cpair = i & 63;
      const float2 v = *reinterpret_cast<const float2*>(c + r * FC_HEAD_DIM + cpair * 2);
      const unsigned short h0 = ea_from_float<DTYPE>(v.x), h1 = ea_from_float<DTYPE>(v.y);
      const unsigned short l0 = ea_from_float<DTYPE>(v.x - ea_to_float<DTYPE>(h0));
      const unsigned short l1 = ea_from_float<DTYPE>(v.y - ea_to_float<DTYPE>(h1));
      *reinterpret_cast<unsigned*>(chi + r * EA_ROWB + cpair * 4) = (unsigned)h0 | ((unsigned)h1 << 16);
      *reinterpret_cast<unsigned*>(clo + r * EA_ROWB + cpair * 4) = (unsigned)l0 | ((unsigned)l1 << 16);
    }
  }
  __syncthreads();

  const char* kbase = kv.base + ((long long)l * kv.stride_layer + (long long)h * kv.stride_head) * 2;
  float* out = raw + head * (long long)raw_stride;
  for (int t = k0 + wave * 32; t < k1; t += EA_WAVES * 32) {
    const int key = t + lrow;
    long long off = fc_token_offset(kv, b, min(key, S - 1));
    if (off < 0) off = 0;
    const char* kp = kbase + off * 2;
    uint4 kf[8];        // B operand: this lane's half of every 16-element k-step of its key row
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) kf[ks] = *reinterpret_cast<const uint4*>(kp + ks * 32 + lhalf * 16);
    uint2 kq[4][4];     // the key's elements at the j this lane's accumulators hold: 4 consecutive per group
#pragma unroll
    for (int jt = 0; jt < 4; ++jt)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4)
        kq[jt][i4] = *reinterpret_cast<const uint2*>(kp + (jt * 32 + i4 * 8 + lhalf * 4) * 2);

    f32x16 acc[4];
#pragma unroll
    for (int jt = 0; jt < 4; ++jt)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        const float4 m = *reinterpret_cast<const float4*>(mus + jt * 32 + i4 * 8 + lhalf * 4);
        acc[jt][i4 * 4 + 0] = m.x;
        acc[jt][i4 * 4 + 1] = m.y;
        acc[jt][i4 * 4 + 2] = m.z;
        acc[jt][i4 * 4 + 3] = m.w;
      }
    if (cov) {
      const char* ahi = chi + lrow * EA_ROWB + lhalf * 16;
      const char* alo = clo + lrow * EA_ROWB + lhalf * 16;
#pragma unroll
      for (int ks = 0; ks < 8; ++ks)
#pragma unroll
        for (int jt = 0; jt < 4; ++jt) {
          const uint4 a = *reinterpret_cast<const uint4*>(ahi + jt * 32 * EA_ROWB + ks * 32);
          const uint4 a2 = *reinterpret_cast<const uint4*>(alo + jt * 32 * EA_ROWB + ks * 32);
          acc[jt] = fc_mfma<DTYPE>(a, kf[ks], acc[jt]);
          acc[jt] = fc_mfma<DTYPE>(a2, kf[ks], acc[jt]);
        }
    }
    float z = 0.f;
#pragma unroll
    for (int jt = 0; jt < 4; ++jt)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        const unsigned w0 = kq[jt][i4].x, w1 = kq[jt][i4].y;
        z = fmaf(acc[jt][i4 * 4 + 0], ea_to_float<DTYPE>((unsigned short)(w0 & 0xffff)), z);
        z = fmaf(acc[jt][i4 * 4 + 1], ea_to_float<DTYPE>((unsigned short)(w0 >> 16)), z);
        z = fmaf(acc[jt][i4 * 4 + 2], ea_to_float<DTYPE>((unsigned short)(w1 & 0xffff)), z);
        z = fmaf(acc[jt][i4 * 4 + 3], ea_to_float<DTYPE>((unsigned short)(w1 >> 16)), z);
      }
    z += __shfl_xor(z, 32, 64);
    if (lhalf == 0 && key < k1) out[key] = z * (1.f / (2.f * FC_HEAD_DIM));
  }
}

#define EA_FIN_THREADS 256
#define EA_MAX_GROUP 64

template <int DTYPE>
__global__ __launch_bounds__(EA_FIN_THREADS) void ea_finish_kernel(KvView vv, const float* __restrict__ raw,
                                                                   int raw_stride, int Hq, int n_sink, int use_vnorm,
                                                                   float epsilon, float* __restrict__ scores,
                                                                   int score_stride, unsigned* __restrict__ gmax) {
  __shared__ float red[EA_FIN_THREADS / 64];
  __shared__ float gm[EA_MAX_GROUP], gl[EA_MAX_GROUP];
  const int h = blockIdx.x, b = blockIdx.y, l = blockIdx.z;
  const int Hkv = vv.num_kv_heads, G = Hq / Hkv;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int S = fc_seq_len(vv, b);
  float* out = scores + (((long long)l * vv.batch + b) * Hkv + h) * (long long)score_stride;
  for (int s = S + tid; s < score_stride; s += EA_FIN_THREADS) out[s] = -INFINITY;   // past the sequence
  if (S <= n_sink) return;   // only sinks: the fill kernel writes them
  const float* rows = raw + (((long long)l * vv.batch + b) * Hq + (long long)h * G) * raw_stride;

  // softmax statistics of every query head of the group over [n_sink, S)
  for (int g = 0; g < G; ++g) {
    const float* r = rows + (long long)g * raw_stride;
    float m = -INFINITY;
    for (int s = n_sink + tid; s < S; s += EA_FIN_THREADS) m = fmaxf(m, r[s]);
    m = fc_wave_max(m);
    if (lane == 0) red[wave] = m;
    __syncthreads();
    m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    __syncthreads();
    float sum = 0.f;
    for (int s = n_sink + tid; s < S; s += EA_FIN_THREADS) sum += __expf(r[s] - m);
    sum = fc_wave_sum(sum);
    if (lane == 0) red[wave] = sum;
    __syncthreads();
    if (tid == 0) {
      gm[g] = m;
      gl[g] = 1.f / ((red[0] + red[1]) + (red[2] + red[3]));
    }
    __syncthreads();
  }

  // 16 lanes per key: value norm and group mean of the probabilities
  const int sub = tid & 15, slot = tid >> 4;
  const char* vbase = vv.base + ((long long)l * vv.stride_layer + (long long)h * vv.stride_head) * 2 + sub * 16;
  const float inv_g = 1.f / (float)G;
  float best = 0.f;
  for (int s0 = n_sink; s0 < S; s0 += EA_FIN_THREADS / 16) {
    const int s = s0 + slot;
    const bool ok = s < S;
    float p = 0.f, sq = 0.f;
    if (ok) {
      for (int g = sub; g < G; g += 16) p += __expf(rows[(long long)g * raw_stride + s] - gm[g]) * gl[g];
      if (use_vnorm) {
        long long off = fc_token_offset(vv, b, s);
        if (off < 0) off = 0;
        const uint4 x = *reinterpret_cast<const uint4*>(vbase + off * 2);
        const unsigned w[4] = {x.x, x.y, x.z, x.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float a = ea_to_float<DTYPE>((unsigned short)(w[i] & 0xffff));
          const float c = ea_to_float<DTYPE>((unsigned short)(w[i] >> 16));
          sq = fmaf(a, a, sq);
          sq = fmaf(c, c, sq);
        }
      }
    }
    p = fc_group_sum<16>(p) * inv_g;
    sq = fc_group_sum<16>(sq);
    if (ok && sub == 0) {
      const float sc = use_vnorm ? (p + epsilon) * sqrtf(sq) : p;
      out[s] = sc;
      best = fmaxf(best, sc);
    }
  }
  best = fc_wave_max(best);
  if (lane == 0 && best > 0.f) atomicMax(gmax + l, __float_as_uint(best));   // non-negative floats order like their bits
}

__global__ void ea_sink_kernel(const int* __restrict__ seq_lens, int max_seq_len, int rows_per_layer, int batch,
                               int Hkv, int n_sink, float* __restrict__ scores, int score_stride,
                               const unsigned* __restrict__ gmax) {
  const int row = blockIdx.x;    // (l, b, h)
  const int l = row / rows_per_layer, b = (row / Hkv) % batch;
  int S = seq_lens ? seq_lens[b] : max_seq_len;
  S = S < max_seq_len ? (S < 0 ? 0 : S) : max_seq_len;
  const float v = __uint_as_float(gmax[l]);
  for (int s = threadIdx.x; s < n_sink && s < S; s += blockDim.x) scores[(long long)row * score_stride + s] = v;
}

extern "C" int64_t fc_expected_attention_workspace_bytes(int32_t num_layers, int32_t batch, int32_t num_q_heads,
                                                         int32_t max_seq_len) {
  if (num_layers <= 0 || batch <= 0 || num_q_heads <= 0 || max_seq_len < 0) return -1;
  return ((int64_t)num_layers * batch * num_q_heads * max_seq_len + num_layers + 64) * (int64_t)sizeof(float);
}

extern "C" int fc_expected_attention_score(const fc_kv_view* keys, const fc_kv_view* values, const float* mean_query,
                                           const float* cov_query, int32_t num_q_heads, int32_t n_sink,
                                           int32_t use_vnorm, float epsilon, float* scores, int32_t score_stride,
                                           void* workspace, int64_t workspace_bytes, void* stream) {
  const char* who = "fc_expected_attention_score";
  int rc;
  if ((rc = fc_check_view(keys, who)) || (rc = fc_check_view(values, who))) return rc;
  FC_REQUIRE(keys->dtype == values->dtype && keys->num_layers == values->num_layers && keys->batch == values->batch &&
                 keys->num_kv_heads == values->num_kv_heads && keys->max_seq_len == values->max_seq_len &&
                 keys->seq_lens == values->seq_lens,
             FC_EINVAL, "%s: key and value views disagree", who);
  FC_REQUIRE(keys->dtype == FC_F16 || keys->dtype == FC_BF16, FC_EUNSUPPORTED, "%s: fp16/bf16 caches only", who);
  FC_REQUIRE(mean_query && scores && workspace, FC_EINVAL, "%s: null pointer", who);
  FC_REQUIRE(num_q_heads > 0 && num_q_heads % keys->num_kv_heads == 0 &&
                 num_q_heads / keys->num_kv_heads <= EA_MAX_GROUP,
             FC_EINVAL, "%s: num_q_heads %d must be a multiple of num_kv_heads %d, at most %d per kv head", who,
             num_q_heads, keys->num_kv_heads, EA_MAX_GROUP);
  FC_REQUIRE(n_sink >= 0 && epsilon >= 0.f, FC_EINVAL, "%s: n_sink and epsilon must not be negative", who);
  FC_REQUIRE(score_stride >= keys->max_seq_len, FC_EINVAL, "%s: score_stride %d < max_seq_len %d", who, score_stride,
             keys->max_seq_len);
  FC_REQUIRE((((uintptr_t)mean_query | (uintptr_t)cov_query) & 7) == 0, FC_EINVAL, "%s: statistics not 8-byte aligned",
             who);
  const int L = keys->num_layers, B = keys->batch, Hkv = keys->num_kv_heads, S = keys->max_seq_len;
  const int64_t need = fc_expected_attention_workspace_bytes(L, B, num_q_heads, S);
  FC_REQUIRE(workspace_bytes >= need, FC_EINVAL, "%s: workspace of %lld bytes, %lld needed", who,
             (long long)workspace_bytes, (long long)need);
  FC_REQUIRE((long long)L * B <= 65535 && num_q_heads <= 65535 && B <= 65535 && L <= 65535, FC_EUNSUPPORTED,
             "%s: grid too large", who);
  if (S == 0) return FC_OK;
  float* raw = (float*)workspace;
  unsigned* gmax = (unsigned*)(raw + (int64_t)L * B * num_q_heads * S);
  KvView k = fc_make_view(keys), v = fc_make_view(values);
  hipStream_t st = (hipStream_t)stream;
  const int chunks = S > n_sink ? (S - n_sink + EA_KEYS_PER_WG - 1) / EA_KEYS_PER_WG : 1;
  const bool bf = keys->dtype == FC_BF16;
#define EA_RUN(DT)                                                                                                   \
  do {                                                                                                               \
    FC_ALLOW_LDS((ea_logits_kernel<DT>), EA_LDS);                                                             \
    hipLaunchKernelGGL((ea_logits_kernel<DT>), dim3(chunks, num_q_heads, L * B), dim3(EA_THREADS), EA_LDS, st, k,    \
                       mean_query, cov_query, num_q_heads, n_sink, raw, S, gmax);                                    \
    hipLaunchKernelGGL((ea_finish_kernel<DT>), dim3(Hkv, B, L), dim3(EA_FIN_THREADS), 0, st, v, (const float*)raw, S, \
                       num_q_heads, n_sink, use_vnorm, epsilon, scores, score_stride, gmax);                         \
  } while (0)
  if (bf) EA_RUN(FC_BF16); else EA_RUN(FC_F16);
#undef EA_RUN
  if (n_sink > 0)
    hipLaunchKernelGGL(ea_sink_kernel, dim3(L * B * Hkv), dim3(64), 0, st, keys->seq_lens, S, B * Hkv, B, Hkv, n_sink,
                       scores, score_stride, (const unsigned*)gmax);
  FC_CHECK_LAUNCH(who);
  return FC_OK;
}
