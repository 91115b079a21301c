// Decode-side kernels over the paged cache: append one K/V row per sequence, advance the lengths,
// and single-query paged attention (split over 256-token chunks, then merged).
//
// Attention is HBM-bound (one pass over K and V, ~1 FLOP per byte per query head), so the kernel is
// organised around the loads: a token row of one kv head is 256 bytes and is read by 16 lanes with
// one 16-byte load each, four rows in flight per lane.  A workgroup owns one (sequence, kv head,
// 256-token chunk) and serves all query heads of the group from the same K/V bytes.
//   phase 1  logits: per lane 8 products per query head, summed across the 16 lanes of a row;
//   phase 2  chunk softmax statistics (max, sum of exp2) per query head;
//   phase 3  sum of p * V rows, 8 output dims per lane, reduced over the 16 row slots of a pass.
// Each chunk writes (max, sum, unnormalised output) to the workspace; a second kernel merges the
// chunks of a sequence.  Grid sizes depend only on the view's max_seq_len, never on the lengths on
// the device, so both launches can be replayed from a graph while the lengths grow.
#include "fc_common.h"

#define DA_THREADS 256
#define DA_CHUNK 256
#define DA_LOG2E 1.4426950408889634f

template <int DTYPE>
__device__ __forceinline__ void da_unpack8(const uint4& x, float (&f)[8]) {
  const unsigned w[4] = {x.x, x.y, x.z, x.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if (DTYPE == FC_BF16) {
      f[2 * i] = __uint_as_float(w[i] << 16);
      f[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    } else {
      f[2 * i] = fc_half_to_float((unsigned short)(w[i] & 0xffff));
      f[2 * i + 1] = fc_half_to_float((unsigned short)(w[i] >> 16));
    }
  }
}

template <int DTYPE>
__device__ __forceinline__ unsigned short da_pack(float f) {
  return DTYPE == FC_BF16 ? fc_float_to_bf16(f) : fc_float_to_half(f);
}

// GT = query heads served per workgroup (a tile of the group)
template <int DTYPE, int GT>
__global__ __launch_bounds__(DA_THREADS) void decode_attn_kernel(KvView kc, KvView vc, int layer,
                                                                 const char* __restrict__ q, int Hq,
                                                                 const int* __restrict__ lens, float c,
                                                                 float* __restrict__ part_o,
                                                                 float* __restrict__ part_ml, int max_splits) {
  __shared__ float sc[GT][DA_CHUNK];
  __shared__ float red[4][GT][FC_HEAD_DIM];
  __shared__ float wred[2][GT][4];

  const int split = blockIdx.x, b = blockIdx.z;
  const int Hkv = kc.num_kv_heads;
  const int G = Hq / Hkv;
  const int gtiles = (G + GT - 1) / GT;
  const int h = blockIdx.y / gtiles, g0 = (blockIdx.y - h * gtiles) * GT;
  int len = lens[b];
  len = min(len, kc.max_seq_len);
  const int t0 = split * DA_CHUNK;
  if (t0 >= len) return;
  const int ntok = min(DA_CHUNK, len - t0);

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int sub = tid & 15, rg = tid >> 4;  // 16 lanes per row, 16 rows per pass

  float qf[GT][8];
#pragma unroll
  for (int g = 0; g < GT; ++g) {
    const int hq = h * G + g0 + g;
    if (g0 + g < G) {
      const uint4 x = *reinterpret_cast<const uint4*>(q + (((long long)b * Hq + hq) * FC_HEAD_DIM + sub * 8) * 2);
      da_unpack8<DTYPE>(x, qf[g]);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) qf[g][e] = 0.f;
    }
  }

  const char* kbase = kc.base + ((long long)layer * kc.stride_layer + (long long)h * kc.stride_head) * 2 + sub * 16;
  const char* vbase = vc.base + ((long long)layer * vc.stride_layer + (long long)h * vc.stride_head) * 2 + sub * 16;

  // ---- phase 1: logits ---------------------------------------------------------------------------
  for (int p0 = 0; p0 < DA_CHUNK / 16; p0 += 4) {
    uint4 kx[4];
    bool ok[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int t = (p0 + u) * 16 + rg;
      ok[u] = t < ntok;
      kx[u] = make_uint4(0, 0, 0, 0);
      if (ok[u]) {
        const long long off = fc_token_offset(kc, b, t0 + t);
        if (off >= 0) kx[u] = *reinterpret_cast<const uint4*>(kbase + off * 2);
      }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      float kf[8];
      da_unpack8<DTYPE>(kx[u], kf);
      const int t = (p0 + u) * 16 + rg;
#pragma unroll
      for (int g = 0; g < GT; ++g) {
        float a = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) a = fmaf(qf[g][e], kf[e], a);
        a += __shfl_xor(a, 8, 64);
        a += __shfl_xor(a, 4, 64);
        a += __shfl_xor(a, 2, 64);
        a += __shfl_xor(a, 1, 64);
        if (sub == 0) sc[g][t] = ok[u] ? a * c : -INFINITY;
      }
    }
  }
  __syncthreads();

  // ---- phase 2: chunk statistics -------------------------------------------------------------------
  float mg[GT], lg[GT];
#pragma unroll
  for (int g = 0; g < GT; ++g) {
    float m = fc_wave_max(sc[g][tid]);
    if (lane == 0) wred[0][g][wave] = m;
  }
  __syncthreads();
#pragma unroll
  for (int g = 0; g < GT; ++g) {
    const float m = fmaxf(fmaxf(wred[0][g][0], wred[0][g][1]), fmaxf(wred[0][g][2], wred[0][g][3]));
    mg[g] = m;
    const float p = __builtin_amdgcn_exp2f(sc[g][tid] - m);  // exp2(-inf) = 0 for the padded slots
    sc[g][tid] = p;
    const float s = fc_wave_sum(p);
    if (lane == 0) wred[1][g][wave] = s;
  }
  __syncthreads();
#pragma unroll
  for (int g = 0; g < GT; ++g) lg[g] = (wred[1][g][0] + wred[1][g][1]) + (wred[1][g][2] + wred[1][g][3]);

  // ---- phase 3: sum of p * V ---------------------------------------------------------------------
  float acc[GT][8];
#pragma unroll
  for (int g = 0; g < GT; ++g)
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[g][e] = 0.f;
  for (int p0 = 0; p0 < DA_CHUNK / 16; p0 += 4) {
    uint4 vx[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int t = (p0 + u) * 16 + rg;
      vx[u] = make_uint4(0, 0, 0, 0);
      if (t < ntok) {
        const long long off = fc_token_offset(vc, b, t0 + t);
        if (off >= 0) vx[u] = *reinterpret_cast<const uint4*>(vbase + off * 2);
      }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      float vf[8];
      da_unpack8<DTYPE>(vx[u], vf);
      const int t = (p0 + u) * 16 + rg;
#pragma unroll
      for (int g = 0; g < GT; ++g) {
        const float p = sc[g][t];
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[g][e] = fmaf(p, vf[e], acc[g][e]);
      }
    }
  }
  // rows of a pass sit 16 lanes apart: fold the 4 row slots of this wavefront, then the 4 wavefronts
#pragma unroll
  for (int g = 0; g < GT; ++g)
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      float a = acc[g][e];
      a += __shfl_xor(a, 16, 64);
      a += __shfl_xor(a, 32, 64);
      if (lane < 16) red[wave][g][sub * 8 + e] = a;
    }
  __syncthreads();
  for (int i = tid; i < GT * FC_HEAD_DIM; i += DA_THREADS) {
    const int g = i / FC_HEAD_DIM, d = i - g * FC_HEAD_DIM;
    if (g0 + g < G) {
      const int hq = h * G + g0 + g;
      const float o = (red[0][g][d] + red[1][g][d]) + (red[2][g][d] + red[3][g][d]);
      part_o[(((long long)b * Hq + hq) * max_splits + split) * FC_HEAD_DIM + d] = o;
    }
  }
#pragma unroll
  for (int g = 0; g < GT; ++g)
    if (tid == g && g0 + g < G) {
      const int hq = h * G + g0 + g;
      float* ml = part_ml + (((long long)b * Hq + hq) * max_splits + split) * 2;
      ml[0] = mg[g];
      ml[1] = lg[g];
    }
}

template <int DTYPE>
__global__ __launch_bounds__(FC_HEAD_DIM) void decode_merge_kernel(const float* __restrict__ part_o,
                                                                   const float* __restrict__ part_ml,
                                                                   const int* __restrict__ lens, int max_seq_len,
                                                                   int Hq, int max_splits, char* __restrict__ out) {
  const int hq = blockIdx.x, b = blockIdx.y, d = threadIdx.x;
  int len = min(lens[b], max_seq_len);
  unsigned short* o = reinterpret_cast<unsigned short*>(out) + ((long long)b * Hq + hq) * FC_HEAD_DIM + d;
  if (len <= 0) {
    *o = 0;
    return;
  }
  const int ns = (len + DA_CHUNK - 1) / DA_CHUNK;
  const float* ml = part_ml + ((long long)b * Hq + hq) * max_splits * 2;
  const float* po = part_o + ((long long)b * Hq + hq) * max_splits * FC_HEAD_DIM + d;
  float M = -INFINITY;
  for (int s = 0; s < ns; ++s) M = fmaxf(M, ml[2 * s]);
  float L = 0.f, acc = 0.f;
  for (int s = 0; s < ns; ++s) {
    const float w = __builtin_amdgcn_exp2f(ml[2 * s] - M);
    L = fmaf(w, ml[2 * s + 1], L);
    acc = fmaf(w, po[(long long)s * FC_HEAD_DIM], acc);
  }
  *o = da_pack<DTYPE>(acc / L);
}

// ---- append / advance ----------------------------------------------------------------------------------
template <int EB>
__global__ __launch_bounds__(256) void store_kv_kernel(KvView kc, KvView vc, const char* __restrict__ k_new,
                                                       const char* __restrict__ v_new,
                                                       const int* __restrict__ lens) {
  const int b = blockIdx.x, l = blockIdx.y;
  const int pos = lens[b];
  if (pos < 0 || pos >= kc.max_seq_len) return;
  const int H = kc.num_kv_heads;
  constexpr int CPR = FC_HEAD_DIM * EB / 16;  // 16-byte chunks per head row
  const long long koff = fc_token_offset(kc, b, pos), voff = fc_token_offset(vc, b, pos);
  if (koff < 0 || voff < 0) return;
  const long long row = ((long long)l * kc.batch + b) * H;
  for (int i = threadIdx.x; i < H * CPR; i += 256) {
    const int h = i / CPR, part = i - h * CPR;
    const long long srcb = ((row + h) * FC_HEAD_DIM) * EB + part * 16;
    *reinterpret_cast<uint4*>(kc.base + ((long long)l * kc.stride_layer + koff + (long long)h * kc.stride_head) * EB +
                              part * 16) = *reinterpret_cast<const uint4*>(k_new + srcb);
    *reinterpret_cast<uint4*>(vc.base + ((long long)l * vc.stride_layer + voff + (long long)h * vc.stride_head) * EB +
                              part * 16) = *reinterpret_cast<const uint4*>(v_new + srcb);
  }
}

// one new row per token i: cache[slot_mapping[i]] <- key[i], value[i]; a row is row_bytes long
__global__ __launch_bounds__(256) void store_slots_kernel(const char* __restrict__ key, long long key_stride_b,
                                                          const char* __restrict__ value, long long value_stride_b,
                                                          char* __restrict__ k_cache, char* __restrict__ v_cache,
                                                          const int* __restrict__ slot_mapping, int row_bytes) {
  const int i = blockIdx.x;
  const long long slot = slot_mapping[i];
  if (slot < 0) return;
  for (int o = threadIdx.x * 16; o < row_bytes; o += 256 * 16) {
    *reinterpret_cast<uint4*>(k_cache + slot * row_bytes + o) = *reinterpret_cast<const uint4*>(key + i * key_stride_b + o);
    *reinterpret_cast<uint4*>(v_cache + slot * row_bytes + o) = *reinterpret_cast<const uint4*>(value + i * value_stride_b + o);
  }
}

__global__ void advance_lens_kernel(int* lens, int n, int delta) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n && lens[i] >= 0) lens[i] += delta;
}

extern "C" int fc_store_kv(const fc_kv_view* k_cache, const fc_kv_view* v_cache, const void* k_new,
                           const void* v_new, const int32_t* context_lens, void* stream) {
  const char* who = "fc_store_kv";
  int rc;
  if ((rc = fc_check_view(k_cache, who)) || (rc = fc_check_view(v_cache, who))) return rc;
  FC_REQUIRE(k_cache->dtype == v_cache->dtype && k_cache->num_layers == v_cache->num_layers &&
                 k_cache->batch == v_cache->batch && k_cache->num_kv_heads == v_cache->num_kv_heads,
             FC_EINVAL, "%s: K and V views disagree", who);
  FC_REQUIRE(k_new && v_new && context_lens, FC_EINVAL, "%s: null pointer", who);
  FC_REQUIRE((((uintptr_t)k_new | (uintptr_t)v_new) & 15) == 0, FC_EINVAL, "%s: new rows not 16-byte aligned", who);
  KvView k = fc_make_view(k_cache), v = fc_make_view(v_cache);
  dim3 grid(k_cache->batch, k_cache->num_layers);
  hipStream_t st = (hipStream_t)stream;
  if (k_cache->dtype == FC_F32)
    hipLaunchKernelGGL((store_kv_kernel<4>), grid, dim3(256), 0, st, k, v, (const char*)k_new, (const char*)v_new,
                       context_lens);
  else
    hipLaunchKernelGGL((store_kv_kernel<2>), grid, dim3(256), 0, st, k, v, (const char*)k_new, (const char*)v_new,
                       context_lens);
  FC_CHECK_LAUNCH(who);
  return FC_OK;
}

extern "C" int fc_store_kv_slots(const void* key, int64_t key_stride, const void* value, int64_t value_stride,
                                 void* k_cache, void* v_cache, const int32_t* slot_mapping, int32_t num_tokens,
                                 int32_t row_elems, int32_t dtype, void* stream) {
  const char* who = "fc_store_kv_slots";
  FC_REQUIRE(key && value && k_cache && v_cache && slot_mapping, FC_EINVAL, "%s: null pointer", who);
  FC_REQUIRE(dtype == FC_F32 || dtype == FC_F16 || dtype == FC_BF16, FC_EINVAL, "%s: unknown dtype %d", who, dtype);
  FC_REQUIRE(num_tokens >= 0 && row_elems > 0, FC_EINVAL, "%s: bad sizes", who);
  const int eb = fc_elem_bytes(dtype);
  FC_REQUIRE(((int64_t)row_elems * eb) % 16 == 0 && (key_stride * eb) % 16 == 0 && (value_stride * eb) % 16 == 0,
             FC_EINVAL, "%s: rows and strides must be multiples of 16 bytes", who);
  FC_REQUIRE((((uintptr_t)key | (uintptr_t)value | (uintptr_t)k_cache | (uintptr_t)v_cache) & 15) == 0, FC_EINVAL,
             "%s: pointers must be 16-byte aligned", who);
  if (num_tokens == 0) return FC_OK;
  hipLaunchKernelGGL(store_slots_kernel, dim3(num_tokens), dim3(256), 0, (hipStream_t)stream, (const char*)key,
                     (long long)key_stride * eb, (const char*)value, (long long)value_stride * eb, (char*)k_cache,
                     (char*)v_cache, slot_mapping, row_elems * eb);
  FC_CHECK_LAUNCH(who);
  return FC_OK;
}

extern "C" int fc_advance_lens(int32_t* context_lens, int32_t batch, int32_t delta, void* stream) {
  FC_REQUIRE(context_lens && batch > 0, FC_EINVAL, "fc_advance_lens: bad arguments");
  hipLaunchKernelGGL(advance_lens_kernel, dim3((batch + 255) / 256), dim3(256), 0, (hipStream_t)stream, context_lens,
                     batch, delta);
  FC_CHECK_LAUNCH("fc_advance_lens");
  return FC_OK;
}

extern "C" int64_t fc_decode_attn_workspace_bytes(int32_t batch, int32_t num_q_heads, int32_t max_seq_len) {
  if (batch <= 0 || num_q_heads <= 0 || max_seq_len < 0) return -1;
  const int64_t splits = (max_seq_len + DA_CHUNK - 1) / DA_CHUNK;
  return (int64_t)batch * num_q_heads * (splits > 0 ? splits : 1) * (FC_HEAD_DIM + 2) * (int64_t)sizeof(float);
}

extern "C" int fc_decode_attn(const fc_kv_view* k_cache, const fc_kv_view* v_cache, int32_t layer, const void* q,
                              void* out, int32_t num_q_heads, const int32_t* context_lens, float scale,
                              void* workspace, int64_t workspace_bytes, void* stream) {
  const char* who = "fc_decode_attn";
  int rc;
  if ((rc = fc_check_view(k_cache, who)) || (rc = fc_check_view(v_cache, who))) return rc;
  FC_REQUIRE(k_cache->dtype == v_cache->dtype && k_cache->num_layers == v_cache->num_layers &&
                 k_cache->batch == v_cache->batch && k_cache->num_kv_heads == v_cache->num_kv_heads &&
                 k_cache->max_seq_len == v_cache->max_seq_len,
             FC_EINVAL, "%s: K and V views disagree", who);
  FC_REQUIRE(k_cache->dtype == FC_F16 || k_cache->dtype == FC_BF16, FC_EUNSUPPORTED, "%s: fp16/bf16 caches only", who);
  FC_REQUIRE(layer >= 0 && layer < k_cache->num_layers, FC_EINVAL, "%s: layer %d out of range", who, layer);
  FC_REQUIRE(q && out && context_lens && workspace, FC_EINVAL, "%s: null pointer", who);
  FC_REQUIRE((((uintptr_t)q | (uintptr_t)workspace) & 15) == 0, FC_EINVAL, "%s: q/workspace not 16-byte aligned", who);
  FC_REQUIRE(num_q_heads > 0 && num_q_heads % k_cache->num_kv_heads == 0, FC_EINVAL,
             "%s: num_q_heads %d not a multiple of num_kv_heads %d", who, num_q_heads, k_cache->num_kv_heads);
  const int64_t need = fc_decode_attn_workspace_bytes(k_cache->batch, num_q_heads, k_cache->max_seq_len);
  FC_REQUIRE(workspace_bytes >= need, FC_EINVAL, "%s: workspace of %lld bytes, %lld needed", who,
             (long long)workspace_bytes, (long long)need);
  const int splits = (k_cache->max_seq_len + DA_CHUNK - 1) / DA_CHUNK;
  const int B = k_cache->batch, Hkv = k_cache->num_kv_heads, G = num_q_heads / Hkv;
  float* part_o = (float*)workspace;
  float* part_ml = part_o + (int64_t)B * num_q_heads * (splits > 0 ? splits : 1) * FC_HEAD_DIM;
  KvView k = fc_make_view(k_cache), v = fc_make_view(v_cache);
  hipStream_t st = (hipStream_t)stream;
  const float c = scale * DA_LOG2E;
  const bool bf = k_cache->dtype == FC_BF16;
  if (splits > 0) {
    const int gt = G >= 8 ? 8 : G >= 4 ? 4 : G >= 2 ? 2 : 1;
    const int gtiles = (G + gt - 1) / gt;
    FC_REQUIRE(Hkv * gtiles <= 65535 && B <= 65535, FC_EUNSUPPORTED, "%s: grid too large", who);
    dim3 grid(splits, Hkv * gtiles, B);
#define DA_LAUNCH(DT, GTV)                                                                                         \
  hipLaunchKernelGGL((decode_attn_kernel<DT, GTV>), grid, dim3(DA_THREADS), 0, st, k, v, layer, (const char*)q,   \
                     num_q_heads, context_lens, c, part_o, part_ml, splits)
#define DA_DISPATCH(DT)                         \
  switch (gt) {                                 \
    case 8: DA_LAUNCH(DT, 8); break;            \
    case 4: DA_LAUNCH(DT, 4); break;            \
    case 2: DA_LAUNCH(DT, 2); break;            \
    default: DA_LAUNCH(DT, 1); break;           \
  }
    if (bf) { DA_DISPATCH(FC_BF16) } else { DA_DISPATCH(FC_F16) }
#undef DA_DISPATCH
#undef DA_LAUNCH
    FC_CHECK_LAUNCH(who);
  }
  dim3 mgrid(num_q_heads, B);
  if (bf)
    hipLaunchKernelGGL((decode_merge_kernel<FC_BF16>), mgrid, dim3(FC_HEAD_DIM), 0, st, part_o, part_ml, context_lens,
                       k_cache->max_seq_len, num_q_heads, splits, (char*)out);
  else
    hipLaunchKernelGGL((decode_merge_kernel<FC_F16>), mgrid, dim3(FC_HEAD_DIM), 0, st, part_o, part_ml, context_lens,
                       k_cache->max_seq_len, num_q_heads, splits, (char*)out);
  FC_CHECK_LAUNCH(who);
  return FC_OK;
}
