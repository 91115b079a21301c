// One Linear layer with optional bias and ReLU on dense row-major fp16/bf16 matrices:
//   Y[M][N] = act(X[M][K] * W^T + b),   W given as [N][K] (nn.Linear layout).
//
// A wavefront owns 32 rows of X and walks K in steps of 16: its A fragment (row = lane % 32,
// 8 consecutive k per lane) is loaded once per step straight from global memory and multiplied
// with the B fragments of up to four 32-column tiles of W (rows of W are contiguous in k, so a
// B fragment is one 16-byte load per lane as well; W is small and stays in the caches).  X is
// therefore read exactly once from HBM.  Accumulation is fp32 (v_mfma_f32_32x32x16), the result
// is rounded to the storage dtype once.  Wider outputs are covered 128 columns at a time.
#include "fc_common.h"


#define LN_WAVES 4

// NT = 32-column tiles handled per pass (1..4)
template <int DTYPE, int NT>
__global__ __launch_bounds__(LN_WAVES * 64) void linear_act_kernel(const char* __restrict__ x, long long ldx,
                                                                    const char* __restrict__ w,
                                                                    const char* __restrict__ bias,
                                                                    char* __restrict__ y, long long ldy, long long M,
                                                                    int N, int K, int relu) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int lrow = lane & 31, lhalf = lane >> 5;
  const long long row0 = ((long long)blockIdx.x * LN_WAVES + wave) * 32;
  if (row0 >= M) return;
  const long long arow = row0 + lrow < M ? row0 + lrow : M - 1;   // rows past the end re-read the last row
  const char* xp = x + (arow * ldx + lhalf * 8) * 2;
  const int n0 = blockIdx.y * (NT * 32);

  f32x16 acc[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[t][i] = 0.f;

  const char* wp = w + ((long long)(n0 + lrow) * K + lhalf * 8) * 2;
  for (int k0 = 0; k0 < K; k0 += 16) {
    const uint4 a = *reinterpret_cast<const uint4*>(xp + k0 * 2);
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const uint4 b = *reinterpret_cast<const uint4*>(wp + ((long long)t * 32 * K + k0) * 2);
      acc[t] = fc_mfma<DTYPE>(a, b, acc[t]);
    }
  }

  // C layout: the lane holds column n0 + t*32 + lrow and rows (i/4)*8 + lhalf*4 + i%4
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int col = n0 + t * 32 + lrow;
    float bv = 0.f;
    if (bias) {
      const unsigned short raw = *reinterpret_cast<const unsigned short*>(bias + col * 2);
      bv = DTYPE == FC_BF16 ? fc_bf16_to_float(raw) : fc_half_to_float(raw);
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const long long r = row0 + (i >> 2) * 8 + lhalf * 4 + (i & 3);
      if (r < M) {
        float v = acc[t][i] + bv;
        if (relu) v = fmaxf(v, 0.f);
        const unsigned short o = DTYPE == FC_BF16 ? fc_float_to_bf16(v) : fc_float_to_half(v);
        *reinterpret_cast<unsigned short*>(y + (r * ldy + col) * 2) = o;
      }
    }
  }
}

extern "C" int fc_linear_act(const void* x, int64_t ldx, const void* weight, const void* bias, void* y, int64_t ldy,
                             int64_t m, int32_t n, int32_t k, int32_t dtype, int32_t apply_relu, void* stream) {
  const char* who = "fc_linear_act";
  FC_REQUIRE(x && weight && y, FC_EINVAL, "%s: null pointer", who);
  FC_REQUIRE(dtype == FC_F16 || dtype == FC_BF16, FC_EUNSUPPORTED, "%s: fp16/bf16 only (got dtype %d)", who, dtype);
  FC_REQUIRE(m >= 0 && n > 0 && k > 0, FC_EINVAL, "%s: bad sizes m=%lld n=%d k=%d", who, (long long)m, n, k);
  FC_REQUIRE(k % 16 == 0 && n % 32 == 0, FC_EUNSUPPORTED, "%s: k must be a multiple of 16 and n of 32 (k=%d n=%d)",
             who, k, n);
  FC_REQUIRE(ldx >= k && ldx % 8 == 0 && ldy >= n, FC_EINVAL, "%s: bad leading dimensions ldx=%lld ldy=%lld", who,
             (long long)ldx, (long long)ldy);
  FC_REQUIRE(((uintptr_t)x & 15) == 0 && ((uintptr_t)weight & 15) == 0, FC_EINVAL, "%s: x and weight must be 16-byte aligned",
             who);
  if (m == 0) return FC_OK;
  const long long row_blocks = (m + LN_WAVES * 32 - 1) / (LN_WAVES * 32);
  FC_REQUIRE(row_blocks <= 2147483647LL, FC_EUNSUPPORTED, "%s: too many rows", who);
  hipStream_t st = (hipStream_t)stream;
  const char *xp = (const char*)x, *wp = (const char*)weight, *bp = (const char*)bias;
  char* yp = (char*)y;
  // full passes of 128 columns, then one pass for what is left
  const int full = n / 128, rest = (n % 128) / 32;
#define LN_LAUNCH(DT, NTV, GY, COL0)                                                                           \
  hipLaunchKernelGGL((linear_act_kernel<DT, NTV>), dim3((unsigned)row_blocks, GY), dim3(LN_WAVES * 64), 0, st, xp, \
                     (long long)ldx, wp + (long long)(COL0) * k * 2, bp ? bp + (COL0) * 2 : nullptr,            \
                     yp + (long long)(COL0) * 2, (long long)ldy, (long long)m, n, k, apply_relu)
#define LN_DISPATCH(DT)                                     \
  do {                                                      \
    if (full) LN_LAUNCH(DT, 4, full, 0);                    \
    if (rest == 1) LN_LAUNCH(DT, 1, 1, full * 128);         \
    else if (rest == 2) LN_LAUNCH(DT, 2, 1, full * 128);    \
    else if (rest == 3) LN_LAUNCH(DT, 3, 1, full * 128);    \
  } while (0)
  if (dtype == FC_BF16) LN_DISPATCH(FC_BF16); else LN_DISPATCH(FC_F16);
#undef LN_DISPATCH
#undef LN_LAUNCH
  FC_CHECK_LAUNCH(who);
  return FC_OK;
}
