// Key-channel statistics and pruning for the ThinK press: the energy of every head-dimension channel of a
// (layer, sequence, kv head) column of K, summed over its tokens, and zeroing of the channels a press decided to
// drop.  Both are single passes over K: a token-head row of 128 elements is covered by 16 lanes (32 for fp32) with
// one 16-byte access each, a workgroup walks its column 32 (16) rows at a time.
#include "fc_common.h"

#define TH_THREADS 512
#define TH_U 4            // rows per lane in flight
// tokens per workgroup of the zeroing kernel: one pass of its 16 rows of 256 bytes, so that the workgroup loads, masks,
// stores and ends (measured on 2304 columns of 4096 bf16 rows: 0.867 ms against 0.929 / 0.963 ms with 256 / 2048 tokens)
#ifndef TH_CHUNK
#define TH_CHUNK 16
#endif

// energy[l][b][h][d] = sum over the tokens s < len(b) of k[l][b][h][s][d]^2, fp32, fixed summation order
template <int DTYPE>
__global__ __launch_bounds__(TH_THREADS) void key_channel_energy_kernel(KvView kv, float* __restrict__ out) {
  constexpr int EB = (DTYPE == FC_F32) ? 4 : 2;
  constexpr int EPL = 16 / EB;                 // elements per lane
  constexpr int LPR = FC_HEAD_DIM * EB / 16;   // lanes per row
  constexpr int RPP = TH_THREADS / LPR;        // rows per pass
  __shared__ float part[RPP][FC_HEAD_DIM + 4];
  const int l = blockIdx.z, b = blockIdx.y, h = blockIdx.x;
  const int S = fc_seq_len(kv, b);
  const int tid = threadIdx.x, sub = tid % LPR, rg = tid / LPR;
  const char* base = kv.base + ((long long)l * kv.stride_layer + (long long)h * kv.stride_head) * EB + sub * 16;
  float acc[EPL];
#pragma unroll
  for (int j = 0; j < EPL; ++j) acc[j] = 0.f;
  for (int s0 = 0; s0 < S; s0 += RPP * TH_U) {
    uint4 x[TH_U];
    bool live[TH_U];
#pragma unroll
    for (int u = 0; u < TH_U; ++u) {   // every lane always loads (a dead row re-reads the last one)
      const int s = s0 + u * RPP + rg;
      long long off = fc_token_offset(kv, b, min(s, S - 1));
      live[u] = s < S && off >= 0;
      x[u] = *reinterpret_cast<const uint4*>(base + (off < 0 ? 0 : off) * EB);
    }
#pragma unroll
    for (int u = 0; u < TH_U; ++u) {
      if (!live[u]) continue;
      const unsigned w[4] = {x[u].x, x[u].y, x[u].z, x[u].w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if constexpr (DTYPE == FC_F32) {
          const float v = __uint_as_float(w[i]);
          acc[i] += v * v;
        } else {
          const float lo = DTYPE == FC_BF16 ? fc_bf16_to_float((unsigned short)(w[i] & 0xffff))
                                            : fc_half_to_float((unsigned short)(w[i] & 0xffff));
          const float hi = DTYPE == FC_BF16 ? fc_bf16_to_float((unsigned short)(w[i] >> 16))
                                            : fc_half_to_float((unsigned short)(w[i] >> 16));
          acc[2 * i] += lo * lo;
          acc[2 * i + 1] += hi * hi;
        }
      }
    }
  }
#pragma unroll
  for (int j = 0; j < EPL; ++j) part[rg][sub * EPL + j] = acc[j];
  __syncthreads();
  if (tid < FC_HEAD_DIM) {
    float v = 0.f;
    for (int r = 0; r < RPP; ++r) v += part[r][tid];
    out[(((long long)l * kv.batch + b) * kv.num_kv_heads + h) * FC_HEAD_DIM + tid] = v;
  }
}

// k[l][b][h][s][d] = 0 for every token s < len(b) and every channel d with prune[l][b][h][d] != 0
template <int DTYPE>
__global__ __launch_bounds__(256) void key_channel_zero_kernel(KvView kv, const unsigned char* __restrict__ prune) {
  constexpr int EB = (DTYPE == FC_F32) ? 4 : 2;
  constexpr int EPL = 16 / EB;
  constexpr int LPR = FC_HEAD_DIM * EB / 16;
  constexpr int RPP = 256 / LPR;
  const int H = kv.num_kv_heads;
  const int l = blockIdx.z, b = blockIdx.y / H, h = blockIdx.y % H;
  const int S = fc_seq_len(kv, b);
  const int tid = threadIdx.x, sub = tid % LPR, rg = tid / LPR;
  const unsigned char* pm = prune + (((long long)l * kv.batch + b) * H + h) * FC_HEAD_DIM + sub * EPL;
  unsigned keep[4];
  bool any = false;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if constexpr (DTYPE == FC_F32) {
      keep[i] = pm[i] ? 0u : 0xffffffffu;
    } else {
      keep[i] = (pm[2 * i] ? 0u : 0x0000ffffu) | (pm[2 * i + 1] ? 0u : 0xffff0000u);
    }
    any |= keep[i] != 0xffffffffu;
  }
  if (!any) return;   // this lane's 16 bytes hold no pruned channel: the rows keep them untouched
  char* base = kv.base + ((long long)l * kv.stride_layer + (long long)h * kv.stride_head) * EB + sub * 16;
  const int s_end = min(S, ((int)blockIdx.x + 1) * TH_CHUNK);
  for (int s = blockIdx.x * TH_CHUNK + rg; s < s_end; s += RPP) {
    const long long off = fc_token_offset(kv, b, s);
    if (off < 0) continue;
    uint4* p = reinterpret_cast<uint4*>(base + off * EB);
    uint4 x = *p;
    x.x &= keep[0];
    x.y &= keep[1];
    x.z &= keep[2];
    x.w &= keep[3];
    *p = x;
  }
}

extern "C" int fc_key_channel_energy(const fc_kv_view* keys, float* energy, void* stream) {
  const char* who = "fc_key_channel_energy";
  int rc = fc_check_view(keys, who);
  if (rc) return rc;
  FC_REQUIRE(energy, FC_EINVAL, "%s: null output", who);
  FC_REQUIRE(keys->batch <= 65535 && keys->num_layers <= 65535, FC_EUNSUPPORTED, "%s: grid too large", who);
  KvView kv = fc_make_view(keys);
  dim3 grid(keys->num_kv_heads, keys->batch, keys->num_layers);
  hipStream_t st = (hipStream_t)stream;
  if (keys->dtype == FC_F32) hipLaunchKernelGGL((key_channel_energy_kernel<FC_F32>), grid, dim3(TH_THREADS), 0, st, kv, energy);
  else if (keys->dtype == FC_F16) hipLaunchKernelGGL((key_channel_energy_kernel<FC_F16>), grid, dim3(TH_THREADS), 0, st, kv, energy);
  else hipLaunchKernelGGL((key_channel_energy_kernel<FC_BF16>), grid, dim3(TH_THREADS), 0, st, kv, energy);
  FC_CHECK_LAUNCH(who);
  return FC_OK;
}

extern "C" int fc_key_channel_zero(const fc_kv_view* keys, const uint8_t* prune, void* stream) {
  const char* who = "fc_key_channel_zero";
  int rc = fc_check_view(keys, who);
  if (rc) return rc;
  FC_REQUIRE(prune, FC_EINVAL, "%s: null mask", who);
  const long long cols = (long long)keys->batch * keys->num_kv_heads;
  FC_REQUIRE(cols <= 65535 && keys->num_layers <= 65535, FC_EUNSUPPORTED, "%s: grid too large", who);
  if (keys->max_seq_len == 0) return FC_OK;
  KvView kv = fc_make_view(keys);
  dim3 grid((keys->max_seq_len + TH_CHUNK - 1) / TH_CHUNK, (unsigned)cols, keys->num_layers);
  hipStream_t st = (hipStream_t)stream;
  if (keys->dtype == FC_F32) hipLaunchKernelGGL((key_channel_zero_kernel<FC_F32>), grid, dim3(256), 0, st, kv, prune);
  else if (keys->dtype == FC_F16) hipLaunchKernelGGL((key_channel_zero_kernel<FC_F16>), grid, dim3(256), 0, st, kv, prune);
  else hipLaunchKernelGGL((key_channel_zero_kernel<FC_BF16>), grid, dim3(256), 0, st, kv, prune);
  FC_CHECK_LAUNCH(who);
  return FC_OK;
}
