// SnapKV observation-window scoring for fp16/bf16 caches.
//
// One workgroup per (layer, sequence, kv head) with one wavefront per 32-row block of window
// queries (group of G query heads x ceil(W/32) blocks, up to 16 wavefronts).  A wavefront keeps
// its 32 query rows as MFMA A-operands in registers for the whole kernel.  Keys stream through
// LDS in tiles of 64 (double buffered, rows padded to 272 bytes so that the 16-byte B-operand
// reads of a half-wave fall on distinct banks) and are multiplied with v_mfma_f32_32x32x16,
// giving each lane 16 logits per 32x32 block: 16 query rows of one key column.
//
// The softmax needs every key of a row before any probability is final, and the [G*W, S] logit
// matrix does not fit on chip, so the keys are swept twice:
//   sweep 1  per-lane (offset, sum of exp2) for each of the lane's 16 query rows.  The first tile
//            fixes the offset with the online-softmax update; later tiles only add
//            exp2(logit - offset).  Should a sum overflow, the sweep is redone with the online
//            update on every tile.  One cross-lane merge per row at the end;
//   sweep 2  logits recomputed, p = exp2(x - m) / l summed over the lane's rows, the two
//            half-waves and the group's wavefronts (fixed order, no atomics) into a 4-tile ring
//            of per-key sums, from which the zero-padded moving average of width `kernel_size`
//            is written two tiles later.
// All arithmetic after the MFMA is fp32.  The second sweep reads K again (a workgroup's column
// does not stay in L2 between the sweeps), so the kernel's memory traffic is about twice the
// algorithmic figure; its run time is set by the exponentials, not by that traffic.
// Optionally the kernel also emits the maximum of each score row for the window fill.
#include "fc_common.h"

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

#ifndef SK_RB
#define SK_RB 1          // 32-row query blocks per wavefront
#endif
#define SK_KT 64          // keys per tile
#define SK_ROWB 272       // LDS bytes per key row (256 + 16 pad)
#define SK_NEG (-1.0e30f) // "minus infinity" that stays finite under subtraction
#define SK_TBL 1024       // block-table entries of one sequence cached in LDS

template <int DTYPE>
__device__ __forceinline__ f32x16 sk_mfma(const uint4& a, const uint4& b, f32x16 c) {
  if constexpr (DTYPE == FC_BF16)
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c,
                                                   0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0,
                                                  0, 0);
}

__device__ __forceinline__ float sk_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

template <int DTYPE, int NW>
__global__ __launch_bounds__(NW * 64, (SK_RB == 2 ? (NW <= 4 ? 2 : 1) : (NW <= 4 ? 4 : NW <= 8 ? 4 : 2))) void snapkv_kernel(
    KvView kv, const char* __restrict__ q, int Hq, int W, int ksz, int causal, float c, float out_mul,
    float* __restrict__ scores, int score_stride, float* __restrict__ row_max) {
  constexpr int THREADS = NW * 64;
  constexpr int CHUNKS = SK_KT * 16;                        // 16-byte chunks per key tile
  constexpr int CH = (CHUNKS + THREADS - 1) / THREADS;      // chunks per thread
  __shared__ __align__(16) char kbuf[2][SK_KT * SK_ROWB];
  __shared__ float vpart[2][NW][SK_KT];
  __shared__ float vraw[4][SK_KT];
  __shared__ int tbl[SK_TBL];

  const int h = blockIdx.x, b = blockIdx.y, l = blockIdx.z;
  const int Hkv = kv.num_kv_heads;
  const int G = Hq / Hkv;
  const int WB = (W + 31) / 32;        // 32-row blocks per query head
  const int RBT = G * WB;              // row blocks of the group
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lrow = lane & 31, lhalf = lane >> 5;
  const int S = fc_seq_len(kv, b);
  float* out_row = scores + (((long long)l * kv.batch + b) * Hkv + h) * (long long)score_stride;

  if (S <= W) {  // nothing outside the window to score
    for (int s = tid; s < score_stride; s += THREADS) out_row[s] = s < S ? 0.f : -INFINITY;
    if (row_max && tid == 0) row_max[((long long)l * kv.batch + b) * Hkv + h] = -INFINITY;
    return;
  }
  const int SW = S - W;                       // scored keys
  const int T = (S + SK_KT - 1) / SK_KT;      // key tiles

  // ---- query fragments ------------------------------------------------------------------
  uint4 qf[SK_RB][8];
  int qi[SK_RB];      // query index (within the window) of this lane's A row
  bool rb_valid[SK_RB];
#pragma unroll
  for (int rb = 0; rb < SK_RB; ++rb) {
    const int blk = wave * SK_RB + rb;
    rb_valid[rb] = blk < RBT;
    const int g = rb_valid[rb] ? blk / WB : 0;
    const int wb = rb_valid[rb] ? blk - g * WB : 0;
    qi[rb] = wb * 32;
    const int qa = wb * 32 + lrow;
    const bool ok = rb_valid[rb] && qa < W;
    const char* qp = q + (((((long long)l * kv.batch + b) * Hq + (h * G + g)) * W + qa) * FC_HEAD_DIM + lhalf * 8) * 2;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks)
      qf[rb][ks] = ok ? *reinterpret_cast<const uint4*>(qp + ks * 32) : make_uint4(0, 0, 0, 0);
  }

  // this sequence's block-table row, so that the tile loads do not wait on a table read each
  const bool paged = kv.block_tables != nullptr;
  const bool tbl_lds = paged && kv.block_shift >= 0 && ((S - 1) >> kv.block_shift) < SK_TBL;
  if (tbl_lds) {
    const int nblk = ((S - 1) >> kv.block_shift) + 1;
    for (int i = tid; i < nblk; i += THREADS) tbl[i] = kv.block_tables[(long long)b * kv.table_stride + i];
  }
  const char* kbase = kv.base + ((long long)l * kv.stride_layer + (long long)h * kv.stride_head) * 2;
  uint4 pre[CH];
  auto load_tile = [&](int t) {
#pragma unroll
    for (int u = 0; u < CH; ++u) {
      const int ch = tid + u * THREADS;
      const int key = ch >> 4, part = ch & 15;
      const int s = t * SK_KT + key;
      pre[u] = make_uint4(0, 0, 0, 0);
      if (ch < CHUNKS && s < S) {
        long long off;
        if (tbl_lds) {
          const int blk = tbl[s >> kv.block_shift];
          off = blk < 0 ? -1 : (long long)blk * kv.stride_block + (long long)(s & (kv.block_size - 1)) * kv.stride_token;
        } else {
          off = fc_token_offset(kv, b, s);
        }
        if (off >= 0) pre[u] = *reinterpret_cast<const uint4*>(kbase + off * 2 + part * 16);
      }
    }
  };
  auto store_tile = [&](int buf) {
#pragma unroll
    for (int u = 0; u < CH; ++u) {
      const int ch = tid + u * THREADS;
      if (ch < CHUNKS) *reinterpret_cast<uint4*>(&kbuf[buf][(ch >> 4) * SK_ROWB + (ch & 15) * 16]) = pre[u];
    }
  };

  // per-lane softmax state for the lane's 2 x 16 query rows: nm = -(offset * c), ls = sum of
  // exp2(logit * c + nm) over the keys this lane has seen
  float nm[SK_RB][16], ls[SK_RB][16];
#pragma unroll
  for (int rb = 0; rb < SK_RB; ++rb)
#pragma unroll
    for (int i = 0; i < 16; ++i) { nm[rb][i] = -SK_NEG; ls[rb][i] = 0.f; }

  __syncthreads();  // tbl
  load_tile(0);
  store_tile(0);
  __syncthreads();

  const bool always_general = SW < SK_KT;

  auto logits = [&](int cur, int cb, f32x16 (&acc)[SK_RB]) {
#pragma unroll
    for (int rb = 0; rb < SK_RB; ++rb)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[rb][i] = 0.f;
    const char* kb = &kbuf[cur][(cb * 32 + lrow) * SK_ROWB + lhalf * 16];
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      const uint4 bf = *reinterpret_cast<const uint4*>(kb + ks * 32);
#pragma unroll
      for (int rb = 0; rb < SK_RB; ++rb) acc[rb] = sk_mfma<DTYPE>(qf[rb][ks], bf, acc[rb]);
    }
  };

  // ================= sweep 1: per-lane softmax statistics ======================================
  // Tile 0 sets every lane-row's offset with the general (online-softmax) update.  Later tiles only
  // add exp2(logit * c + nm): any fixed offset is mathematically valid, it merely has to keep the
  // sums inside the fp32 range.  A sum that overflows (logits rising by more than ~2^7 in log2
  // units above the first tile's) is detected afterwards and the sweep is redone with the general
  // update on every tile.
  int pb = 0;   // LDS buffer parity of tile 0 of the current sweep
  auto sweep1 = [&](bool general) {
    for (int t = 0; t < T; ++t) {
      const int cur = (pb + t) & 1;
      load_tile(t + 1 < T ? t + 1 : 0);   // the tile after the last one is tile 0 of the next sweep
      const int tile_end = (t + 1) * SK_KT;
      const bool masked_tile = tile_end > S || (causal && tile_end > SW + 1);
      const bool slow = general || t == 0;
#pragma unroll
      for (int cb = 0; cb < 2; ++cb) {
        f32x16 acc[SK_RB];
        logits(cur, cb, acc);
        // keys past the sequence end, and (causal) window keys later than the query, are masked
        if (masked_tile) {
          const int s = t * SK_KT + cb * 32 + lrow;
#pragma unroll
          for (int rb = 0; rb < SK_RB; ++rb) {
            // query index of register i is qi[rb] + lhalf*4 + (i/4)*8 + i%4: compare against constants
            const int d = causal ? s - SW - qi[rb] - lhalf * 4 : -1;
#pragma unroll
            for (int i = 0; i < 16; ++i)
              if (s >= S || d > ((i >> 2) * 8 + (i & 3))) acc[rb][i] = SK_NEG;
          }
        }
        if (slow) {
          // differences are formed before scaling: (-1e30) - (-1e30) = 0 exactly for still-masked rows
#pragma unroll
          for (int rb = 0; rb < SK_RB; ++rb)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
              const float tt = -acc[rb][i] * c;
              const float mn = fminf(nm[rb][i], tt);
              ls[rb][i] = ls[rb][i] * sk_exp2(mn - nm[rb][i]) + sk_exp2(mn - tt);
              nm[rb][i] = mn;
            }
        } else {
#pragma unroll
          for (int rb = 0; rb < SK_RB; ++rb)
#pragma unroll
            for (int i = 0; i < 16; ++i) ls[rb][i] += sk_exp2(fmaf(acc[rb][i], c, nm[rb][i]));
        }
      }
      store_tile(cur ^ 1);
      __syncthreads();
    }
    pb += T;
  };
  for (int attempt = 0; attempt < 2; ++attempt) {   // one inlined copy of the sweep
    sweep1(always_general || attempt == 1);
    bool bad = false;
#pragma unroll
    for (int rb = 0; rb < SK_RB; ++rb)
#pragma unroll
      for (int i = 0; i < 16; ++i) bad |= !(ls[rb][i] <= 3.0e38f);   // inf or NaN
    if (attempt == 1 || !__syncthreads_or(bad)) break;
#pragma unroll
    for (int rb = 0; rb < SK_RB; ++rb)
#pragma unroll
      for (int i = 0; i < 16; ++i) { nm[rb][i] = -SK_NEG; ls[rb][i] = 0.f; }
  }

  // merge the per-lane states of each row across the 32 lanes of a half-wave and fold the
  // normaliser into the offset: p = exp2(logit * c + nm), nm = -(max * c) - log2(sum)
#pragma unroll
  for (int rb = 0; rb < SK_RB; ++rb)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      float mm = nm[rb][i], ll = ls[rb][i];
#pragma unroll
      for (int o = 1; o < 32; o <<= 1) {
        const float m2 = __shfl_xor(mm, o, 64), l2 = __shfl_xor(ll, o, 64);
        const float mn = fminf(mm, m2);
        ll = ll * sk_exp2(mn - mm) + l2 * sk_exp2(mn - m2);
        mm = mn;
      }
      const int qa = qi[rb] + (i >> 2) * 8 + lhalf * 4 + (i & 3);
      const bool ok = rb_valid[rb] && qa < W;
      nm[rb][i] = ok ? mm - __builtin_amdgcn_logf(ll) : SK_NEG;   // v_log_f32 is log2
    }

  // ================= sweep 2: probabilities, per-key sums, moving average ======================
  for (int t = 0; t < T; ++t) {
    const int cur = (pb + t) & 1;
    if (t >= 1 && tid < SK_KT) {
      // fold the wavefronts' partial sums of tile t-1 (fixed order) into the ring
      float v = 0.f;
#pragma unroll
      for (int w = 0; w < NW; ++w) v += vpart[cur ^ 1][w][tid];
      vraw[(t - 1) & 3][tid] = v;
      // moving average for tile t-3: its neighbours t-4 .. t-2 are complete
      if (t >= 3) {
        const int s = (t - 3) * SK_KT + tid;
        if (s < SW) {
          float acc = 0.f;
          const int hw = ksz >> 1;
          for (int j = -hw; j <= hw; ++j) {
            const int x = s + j;
            if (x >= 0 && x < SW) acc += vraw[(x / SK_KT) & 3][x % SK_KT];
          }
          out_row[s] = acc * out_mul;
        }
      }
    }
    const bool more = t + 1 < T;
    if (more) load_tile(t + 1);
#pragma unroll
    for (int cb = 0; cb < 2; ++cb) {
      f32x16 acc[SK_RB];
      logits(cur, cb, acc);
      float vs = 0.f;
#pragma unroll
      for (int rb = 0; rb < SK_RB; ++rb)
#pragma unroll
        for (int i = 0; i < 16; ++i) vs += sk_exp2(fmaf(acc[rb][i], c, nm[rb][i]));
      vs += __shfl_xor(vs, 32, 64);
      if (lane < 32) vpart[cur][wave][cb * 32 + lane] = vs;
    }
    if (more) store_tile(cur ^ 1);
    __syncthreads();
  }
  const int last_buf = (pb + T - 1) & 1;

  // ---- drain: last tile's sums, then the moving average of the last three tiles ------------
  if (tid < SK_KT) {
    float v = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) v += vpart[last_buf][w][tid];
    vraw[(T - 1) & 3][tid] = v;
  }
  __syncthreads();
  {
    const int first = T >= 3 ? (T - 3) * SK_KT : 0;
    const int hw = ksz >> 1;
    for (int s = first + tid; s < SW; s += THREADS) {
      float acc = 0.f;
      for (int j = -hw; j <= hw; ++j) {
        const int x = s + j;
        if (x >= 0 && x < SW) acc += vraw[(x / SK_KT) & 3][x % SK_KT];
      }
      out_row[s] = acc * out_mul;
    }
    for (int s = S + tid; s < score_stride; s += THREADS) out_row[s] = -INFINITY;
  }
  if (row_max) {   // maximum of this row's scores, for the window fill: re-read what this workgroup wrote
    __syncthreads();
    float rmax = -INFINITY;
    for (int s = tid; s < SW; s += THREADS) rmax = fmaxf(rmax, out_row[s]);
    rmax = fc_wave_max(rmax);
    if (lane == 0) vpart[0][wave][0] = rmax;
    __syncthreads();
    if (tid == 0) {
      float m = vpart[0][0][0];
#pragma unroll
      for (int w = 1; w < NW; ++w) m = fmaxf(m, vpart[0][w][0]);
      row_max[((long long)l * kv.batch + b) * Hkv + h] = m;
    }
  }
}

// Window fill.  With the per-row maxima from the scoring kernel: one small workgroup per row takes
// the maximum over its layer's rows and writes its own window.  Without them: one workgroup per
// layer scans the scored part of every row first.
__global__ __launch_bounds__(64) void snapkv_fill_rows_kernel(float* __restrict__ scores, int score_stride, int batch,
                                                              int Hkv, const int* __restrict__ seq_lens,
                                                              int max_seq_len, int W,
                                                              const float* __restrict__ row_max) {
  const int r = blockIdx.x, l = blockIdx.y, lane = threadIdx.x;
  const int rows = batch * Hkv;
  float mx = -INFINITY;
  for (int i = lane; i < rows; i += 64) mx = fmaxf(mx, row_max[(long long)l * rows + i]);
  mx = fc_wave_max(mx);
  int S = seq_lens ? seq_lens[r / Hkv] : max_seq_len;
  S = min(S, max_seq_len);
  float* row = scores + ((long long)l * rows + r) * score_stride;
  for (int j = lane; j < W; j += 64)
    if (S - W + j >= 0) row[S - W + j] = mx;
}

__global__ __launch_bounds__(1024) void snapkv_fill_kernel(float* __restrict__ scores, int score_stride, int batch,
                                                           int Hkv, const int* __restrict__ seq_lens, int max_seq_len,
                                                           int W) {
  __shared__ float red[16];
  const int l = blockIdx.x, tid = threadIdx.x;
  float* base = scores + (long long)l * batch * Hkv * score_stride;
  float mx = -INFINITY;
  const int rows = batch * Hkv;
  for (int r = 0; r < rows; ++r) {
    int S = seq_lens ? seq_lens[r / Hkv] : max_seq_len;
    S = min(S, max_seq_len);
    const float* row = base + (long long)r * score_stride;
    for (int s = tid; s < S - W; s += 1024) mx = fmaxf(mx, row[s]);
  }
  mx = fc_wave_max(mx);
  if ((tid & 63) == 0) red[tid >> 6] = mx;
  __syncthreads();
  mx = red[0];
#pragma unroll
  for (int w = 1; w < 16; ++w) mx = fmaxf(mx, red[w]);
  for (int i = tid; i < rows * W; i += 1024) {
    const int r = i / W, j = i - r * W;
    int S = seq_lens ? seq_lens[r / Hkv] : max_seq_len;
    S = min(S, max_seq_len);
    const int s = S - W + j;
    if (s >= 0) base[(long long)r * score_stride + s] = mx;
  }
}

extern "C" int fc_snapkv_score(const fc_kv_view* keys, const void* queries, int32_t num_q_heads, int32_t window,
                               int32_t kernel_size, int32_t causal_window, float scale, float out_scale,
                               float* scores, int32_t score_stride, float* row_max, void* stream) {
  const char* who = "fc_snapkv_score";
  int rc = fc_check_view(keys, who);
  if (rc) return rc;
  FC_REQUIRE(queries && scores, FC_EINVAL, "%s: null pointer", who);
  FC_REQUIRE(((uintptr_t)queries & 15) == 0, FC_EINVAL, "%s: queries not 16-byte aligned", who);
  FC_REQUIRE(keys->dtype == FC_F16 || keys->dtype == FC_BF16, FC_EUNSUPPORTED,
             "%s: fp16/bf16 caches only (got dtype %d)", who, keys->dtype);
  FC_REQUIRE(num_q_heads > 0 && num_q_heads % keys->num_kv_heads == 0, FC_EINVAL,
             "%s: num_q_heads %d not a multiple of num_kv_heads %d", who, num_q_heads, keys->num_kv_heads);
  FC_REQUIRE(window > 0, FC_EINVAL, "%s: window must be positive", who);
  FC_REQUIRE(kernel_size >= 1 && (kernel_size & 1) && kernel_size <= 63, FC_EINVAL,
             "%s: kernel_size %d must be odd and <= 63", who, kernel_size);
  FC_REQUIRE(score_stride >= keys->max_seq_len, FC_EINVAL, "%s: score_stride %d < max_seq_len %d", who,
             score_stride, keys->max_seq_len);
  const int G = num_q_heads / keys->num_kv_heads;
  const int rbt = G * ((window + 31) / 32);
  const int waves = (rbt + SK_RB - 1) / SK_RB;
  FC_REQUIRE(waves <= 16, FC_EUNSUPPORTED, "%s: group of %d heads x window %d needs %d wavefronts (max 16)", who, G,
             window, waves);
  if (keys->max_seq_len == 0) return FC_OK;
  KvView kv = fc_make_view(keys);
  dim3 grid(keys->num_kv_heads, keys->batch, keys->num_layers);
  hipStream_t st = (hipStream_t)stream;
  const float c = scale * 1.4426950408889634f;
  const float out_mul = out_scale / (float)kernel_size;
  const char* q = (const char*)queries;
#define SK_LAUNCH(DT, NWV)                                                                                   \
  hipLaunchKernelGGL((snapkv_kernel<DT, NWV>), grid, dim3(NWV * 64), 0, st, kv, q, num_q_heads, window,      \
                     kernel_size, causal_window, c, out_mul, scores, score_stride, row_max)
#define SK_DISPATCH(DT)                 \
  if (waves <= 1) SK_LAUNCH(DT, 1);     \
  else if (waves <= 2) SK_LAUNCH(DT, 2);\
  else if (waves <= 4) SK_LAUNCH(DT, 4);\
  else if (waves <= 8) SK_LAUNCH(DT, 8);\
  else SK_LAUNCH(DT, 16)
  if (keys->dtype == FC_BF16) { SK_DISPATCH(FC_BF16); } else { SK_DISPATCH(FC_F16); }
#undef SK_DISPATCH
#undef SK_LAUNCH
  FC_CHECK_LAUNCH(who);
  return FC_OK;
}

extern "C" int fc_snapkv_fill_window(float* scores, int32_t score_stride, int32_t num_layers, int32_t batch,
                                     int32_t num_kv_heads, const int32_t* seq_lens, int32_t max_seq_len,
                                     int32_t window, const float* row_max, void* stream) {
  const char* who = "fc_snapkv_fill_window";
  FC_REQUIRE(scores, FC_EINVAL, "%s: null scores", who);
  FC_REQUIRE(num_layers > 0 && batch > 0 && num_kv_heads > 0 && window > 0 && max_seq_len >= 0 &&
                 score_stride >= max_seq_len,
             FC_EINVAL, "%s: bad sizes", who);
  if (row_max) {
    FC_REQUIRE(num_layers <= 65535, FC_EUNSUPPORTED, "%s: too many layers", who);
    hipLaunchKernelGGL(snapkv_fill_rows_kernel, dim3(batch * num_kv_heads, num_layers), dim3(64), 0,
                       (hipStream_t)stream, scores, score_stride, batch, num_kv_heads, seq_lens, max_seq_len, window,
                       row_max);
  } else {
    hipLaunchKernelGGL(snapkv_fill_kernel, dim3(num_layers), dim3(1024), 0, (hipStream_t)stream, scores, score_stride,
                       batch, num_kv_heads, seq_lens, max_seq_len, window);
  }
  FC_CHECK_LAUNCH(who);
  return FC_OK;
}
