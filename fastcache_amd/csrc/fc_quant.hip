// Quantisation of KV rows: symmetric per-row int8 storage (4- or 8-bit range) and back, asymmetric 8-bit rows,
// packed 4-bit groups (integer and NF4), 8-bit floating point codes with one scale for the tensor, and
// quantise -> dequantise in one pass with a per-row or whole-tensor scale.
//
// One wavefront per row of `d` elements.  The arithmetic follows what a tensor library does on a
// tensor of the row's dtype, step by step: every intermediate (row maximum, scale, quotient) is
// computed in fp32 and rounded to the storage dtype before the next step, so that the integers
// and scales are bit-identical to the eager expression
//   scale = clamp(max|x| / qmax, min=1e-8);  q = clamp(round(x / scale), -qmax-1, qmax).
#include "fc_common.h"

template <int DTYPE>
__device__ __forceinline__ float qz_load(const char* p, long long i) {
  if constexpr (DTYPE == FC_F32) return reinterpret_cast<const float*>(p)[i];
  const unsigned short r = reinterpret_cast<const unsigned short*>(p)[i];
  return DTYPE == FC_BF16 ? fc_bf16_to_float(r) : fc_half_to_float(r);
}
template <int DTYPE>
__device__ __forceinline__ float qz_round(float v) {   // round to the storage dtype, back to fp32
  if constexpr (DTYPE == FC_F32) return v;
  return DTYPE == FC_BF16 ? fc_bf16_to_float(fc_float_to_bf16(v)) : fc_half_to_float(fc_float_to_half(v));
}
template <int DTYPE>
__device__ __forceinline__ void qz_store(char* p, long long i, float v) {
  if constexpr (DTYPE == FC_F32) reinterpret_cast<float*>(p)[i] = v;
  else reinterpret_cast<unsigned short*>(p)[i] = DTYPE == FC_BF16 ? fc_float_to_bf16(v) : fc_float_to_half(v);
}

template <int DTYPE>
__global__ __launch_bounds__(256) void quantize_rows_kernel(const char* __restrict__ x, long long rows, int d,
                                                            float qmax, signed char* __restrict__ q,
                                                            char* __restrict__ scale) {
  const long long r = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (r >= rows) return;
  const long long base = r * d;
  float mx = 0.f;
  bool has_nan = false;
  for (int j = lane; j < d; j += 64) {
    const float v = qz_load<DTYPE>(x, base + j);
    has_nan |= v != v;
    mx = fmaxf(mx, fabsf(v));
  }
  mx = fc_wave_max(mx);
  if (__any(has_nan)) mx = __builtin_nanf("");   // a NaN in the row makes the maximum NaN
  // scale = max / qmax, rounded; clamp(min=1e-8) in fp32, rounded again (1e-8 underflows to 0 in fp16)
  float sc = qz_round<DTYPE>(mx / qmax);
  sc = qz_round<DTYPE>(sc != sc ? sc : fmaxf(sc, 1e-8f));
  if (lane == 0) qz_store<DTYPE>(scale, r, sc);
  for (int j = lane; j < d; j += 64) {
    const float v = qz_load<DTYPE>(x, base + j);
    float t = qz_round<DTYPE>(v / sc);
    t = rintf(t);                                   // round half to even
    const bool is_nan = t != t;                     // the integer cast of NaN gives 0 (fmaxf would turn it into the bound)
    t = fminf(fmaxf(t, -qmax - 1.f), qmax);
    q[base + j] = is_nan ? (signed char)0 : (signed char)(int)t;
  }
}

// out = float(q) * scale, rounded to the output dtype.  SDT = dtype of scale, ODT = dtype of out.
template <int SDT, int ODT>
__global__ __launch_bounds__(256) void dequantize_rows_kernel(const signed char* __restrict__ q,
                                                              const char* __restrict__ scale, long long rows, int d,
                                                              char* __restrict__ out) {
  const long long r = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (r >= rows) return;
  const float sc = qz_load<SDT>(scale, r);
  const long long base = r * d;
  for (int j = lane; j < d; j += 64) qz_store<ODT>(out, base + j, (float)q[base + j] * sc);
}

// 4-bit codes of groups of `g` elements, two per byte (element 2j in the low nibble).
// MODE 0: integer codes, scale = clamp(max|x| / 7, 1e-8), code = clamp(round(x / scale), -8, 7) + 8.
// MODE 1: NF4, scale = clamp(max|x|, 1e-8), code = index of the table entry nearest to x / scale
//         (table rounded to the tensor dtype, differences rounded to it as well, first minimum wins).
__constant__ float kNf4Table[16] = {-1.0f, -0.6961928009986877f, -0.5250730514526367f, -0.39491748809814453f,
                                    -0.28444138169288635f, -0.18477343022823334f, -0.09105003625154495f, 0.0f,
                                    0.07958029955625534f, 0.16093020141124725f, 0.24611230194568634f,
                                    0.33791524171829224f, 0.44070982933044434f, 0.5626170039176941f,
                                    0.7229568362236023f, 1.0f};

// the NF4 levels rounded to the tensor dtype, once per workgroup (the caller synchronises)
template <int DTYPE>
__device__ __forceinline__ void qz_fill_levels(float* levels) {
  if (threadIdx.x < 16) levels[threadIdx.x] = qz_round<DTYPE>(kNf4Table[threadIdx.x]);
}

template <int DTYPE, int MODE>
__device__ __forceinline__ int qz_code4(float v, float sc, const float* levels) {
  const float t = qz_round<DTYPE>(v / sc);
  if constexpr (MODE == 0) {
    float r = rintf(t);
    if (r != r) return 8;                           // the integer cast of NaN gives 0, stored with the offset of 8
    r = fminf(fmaxf(r, -8.f), 7.f);
    return (int)r + 8;
  } else {
    // argmin over |t - level|, every difference rounded to the dtype, first minimum wins.  The levels are at least
    // 0.079 apart and |t| <= 1, so two differences on the same side of t never round to the same number: the
    // minimum is the nearest level below-or-equal t or the nearest above, and a tie goes to the lower one.
    if (t != t || fabsf(t) == INFINITY) return 0;     // NaN: every difference is NaN; infinite: all are equal
    int lo = 0;
#pragma unroll
    for (int step = 8; step >= 1; step >>= 1)
      if (levels[lo + step] <= t) lo += step;
    const int hi = lo < 15 ? lo + 1 : 15;
    const float d_lo = fabsf(qz_round<DTYPE>(t - levels[lo]));
    const float d_hi = fabsf(qz_round<DTYPE>(t - levels[hi]));
    return d_hi < d_lo ? hi : lo;
  }
}

template <int DTYPE, int MODE>
__global__ __launch_bounds__(256) void quantize_group4_kernel(const char* __restrict__ x, long long groups, int g,
                                                              unsigned char* __restrict__ packed,
                                                              char* __restrict__ scale) {
  __shared__ float levels[16];
  if (MODE == 1) {
    qz_fill_levels<DTYPE>(levels);
    __syncthreads();
  }
  const long long r = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (r >= groups) return;
  const long long base = r * g;
  float mx = 0.f;
  bool has_nan = false;
  for (int j = lane; j < g; j += 64) {
    const float v = qz_load<DTYPE>(x, base + j);
    has_nan |= v != v;
    mx = fmaxf(mx, fabsf(v));
  }
  mx = fc_wave_max(mx);
  if (__any(has_nan)) mx = __builtin_nanf("");
  float sc = MODE == 0 ? qz_round<DTYPE>(mx / 7.f) : mx;
  sc = qz_round<DTYPE>(sc != sc ? sc : fmaxf(sc, 1e-8f));
  if (lane == 0) qz_store<DTYPE>(scale, r, sc);
  for (int j = lane; j < g / 2; j += 64) {
    const int lo = qz_code4<DTYPE, MODE>(qz_load<DTYPE>(x, base + 2 * j), sc, levels);
    const int hi = qz_code4<DTYPE, MODE>(qz_load<DTYPE>(x, base + 2 * j + 1), sc, levels);
    packed[base / 2 + j] = (unsigned char)(lo | (hi << 4));
  }
}

// TDT: dtype the level table is rounded to (the dtype asked for); SDT: dtype of scale; ODT: output dtype
template <int TDT, int SDT, int ODT, int MODE>
__global__ __launch_bounds__(256) void dequantize_group4_kernel(const unsigned char* __restrict__ packed,
                                                                const char* __restrict__ scale, long long groups,
                                                                int g, char* __restrict__ out) {
  const long long r = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (r >= groups) return;
  const float sc = qz_load<SDT>(scale, r);
  const long long base = r * g;
  for (int j = lane; j < g / 2; j += 64) {
    const unsigned b = packed[base / 2 + j];
    float lo, hi;
    if constexpr (MODE == 0) {
      lo = (float)(int)(b & 15u) - 8.f;
      hi = (float)(int)(b >> 4) - 8.f;
    } else {
      lo = qz_round<TDT>(kNf4Table[b & 15u]);
      hi = qz_round<TDT>(kNf4Table[b >> 4]);
    }
    qz_store<ODT>(out, base + 2 * j, lo * sc);
    qz_store<ODT>(out, base + 2 * j + 1, hi * sc);
  }
}

// ---- quantise -> dequantise in one pass ("fake quantisation") ---------------------------------------
// y = clamp(round(x / scale), -qmax-1, qmax) * scale, scale = max|x| / qmax taken per row of d elements
// or over the whole tensor; no floor on the scale (an all-zero row gives 0/0 = NaN, as the eager
// expression does), NaN and infinities propagate the IEEE way.  Same rounding discipline as above.
template <int DTYPE>
__device__ __forceinline__ float qz_fake(float v, float sc, float qmax) {
  float t = rintf(qz_round<DTYPE>(v / sc));
  t = (t != t) ? t : fminf(fmaxf(t, -qmax - 1.f), qmax);   // clamp keeps NaN
  return t * sc;
}

template <int DTYPE>
__global__ __launch_bounds__(256) void fake_quant_rows_kernel(const char* __restrict__ x, long long rows, int d,
                                                              float qmax, char* __restrict__ y,
                                                              char* __restrict__ scale, char* __restrict__ absmax) {
  const long long r = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (r >= rows) return;
  const long long base = r * d;
  float mx = 0.f;
  bool has_nan = false;
  for (int j = lane; j < d; j += 64) {
    const float v = qz_load<DTYPE>(x, base + j);
    has_nan |= v != v;
    mx = fmaxf(mx, fabsf(v));
  }
  mx = fc_wave_max(mx);
  if (__any(has_nan)) mx = __builtin_nanf("");
  const float sc = qz_round<DTYPE>(mx / qmax);
  if (lane == 0) {
    if (scale) qz_store<DTYPE>(scale, r, sc);
    if (absmax) qz_store<DTYPE>(absmax, r, mx);
  }
  for (int j = lane; j < d; j += 64) qz_store<DTYPE>(y, base + j, qz_fake<DTYPE>(qz_load<DTYPE>(x, base + j), sc, qmax));
}

#define QZ_PARTS 1024   // partial maxima of the whole-tensor variant

// largest |x| of this block's grid-stride share; NaN if it saw one
template <int DTYPE>
__global__ __launch_bounds__(256) void absmax_partial_kernel(const char* __restrict__ x, long long n,
                                                             float* __restrict__ partial) {
  __shared__ float wm[4];
  float mx = 0.f;
  bool has_nan = false;
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long long)gridDim.x * 256) {
    const float v = qz_load<DTYPE>(x, i);
    has_nan |= v != v;
    mx = fmaxf(mx, fabsf(v));
  }
  mx = fc_wave_max(mx);
  if (__any(has_nan)) mx = __builtin_nanf("");
  if ((threadIdx.x & 63) == 0) wm[threadIdx.x >> 6] = mx;
  __syncthreads();
  if (threadIdx.x == 0) {
    float m = wm[0];
    for (int w = 1; w < 4; ++w) m = (m != m || wm[w] != wm[w]) ? __builtin_nanf("") : fmaxf(m, wm[w]);
    partial[blockIdx.x] = m;
  }
}

template <int DTYPE>
__global__ __launch_bounds__(256) void fake_quant_tensor_kernel(const char* __restrict__ x, long long n,
                                                                const float* __restrict__ partial, int nparts,
                                                                float qmax, char* __restrict__ y,
                                                                char* __restrict__ scale, char* __restrict__ absmax) {
  __shared__ float wm[4];
  float mx = 0.f;
  bool has_nan = false;
  for (int i = threadIdx.x; i < nparts; i += 256) {
    const float v = partial[i];
    has_nan |= v != v;
    mx = fmaxf(mx, v);
  }
  mx = fc_wave_max(mx);
  if (__any(has_nan)) mx = __builtin_nanf("");
  if ((threadIdx.x & 63) == 0) wm[threadIdx.x >> 6] = mx;
  __syncthreads();
  mx = wm[0];
  for (int w = 1; w < 4; ++w) mx = (mx != mx || wm[w] != wm[w]) ? __builtin_nanf("") : fmaxf(mx, wm[w]);
  const float sc = qz_round<DTYPE>(mx / qmax);
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    if (scale) qz_store<DTYPE>(scale, 0, sc);
    if (absmax) qz_store<DTYPE>(absmax, 0, mx);
  }
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long long)gridDim.x * 256)
    qz_store<DTYPE>(y, i, qz_fake<DTYPE>(qz_load<DTYPE>(x, i), sc, qmax));
}

// ---- 8-bit floating point codes ------------------------------------------------------------------
// Round to nearest even from an fp32 value.  E4M3 (finite-only variant: bias 7, largest value 448, codes 0x7f / 0xff
// are NaN, no infinity): whatever rounds past 448, infinities and NaN included, becomes NaN.  E5M2 (bias 15, IEEE
// style): whatever rounds past 57344 becomes infinity, NaN stays NaN.  Values under the smallest normal number are
// rounded by adding the power of two whose unit in the last place is the target's subnormal spacing.
template <int E5M2>
__device__ __forceinline__ unsigned char qz_to_fp8(float f) {
  unsigned u = __float_as_uint(f);
  const unsigned sign = (u >> 24) & 0x80u;
  u &= 0x7fffffffu;
  unsigned r;
  if constexpr (!E5M2) {
    if (u >= (1087u << 20)) {                      // 480 and above
      r = 0x7f;
    } else if (u < (121u << 23)) {                 // below 2^-6: multiples of 2^-9
      r = __float_as_uint(__uint_as_float(u) + __uint_as_float(141u << 23)) - (141u << 23);
    } else {
      const unsigned odd = (u >> 20) & 1u;
      r = (u - (120u << 23) + 0x7ffffu + odd) >> 20;
    }
  } else {
    if (u >= (143u << 23)) {                       // 65536 and above
      r = u > 0x7f800000u ? 0x7f : 0x7c;
    } else if (u < (113u << 23)) {                 // below 2^-14: multiples of 2^-16
      r = __float_as_uint(__uint_as_float(u) + __uint_as_float(134u << 23)) - (134u << 23);
    } else {
      const unsigned odd = (u >> 21) & 1u;
      r = (u - (112u << 23) + 0xfffffu + odd) >> 21;
    }
  }
  return (unsigned char)(r | sign);
}

template <int E5M2>
__device__ __forceinline__ float qz_from_fp8(unsigned char c) {
  const unsigned sign = ((unsigned)c & 0x80u) << 24;
  const unsigned mag = c & 0x7fu;
  constexpr int MB = E5M2 ? 2 : 3, BIAS = E5M2 ? 15 : 7;
  const unsigned e = mag >> MB, m = mag & ((1u << MB) - 1u);
  float v;
  if (E5M2 ? (e == 31u) : (mag == 0x7fu)) v = (E5M2 && m == 0u) ? INFINITY : __builtin_nanf("");
  else if (e == 0u) v = (float)m * (E5M2 ? 1.52587890625e-05f : 0.001953125f);          // m * 2^(1 - BIAS - MB)
  else v = __uint_as_float(((e + 127u - BIAS) << 23) | (m << (23 - MB)));
  return __uint_as_float(__float_as_uint(v) | sign);
}

// scale = clamp(max|x| / 448, min=1e-8) over the whole tensor (both formats divide by 448), code = fp8(x / scale)
template <int DTYPE, int E5M2>
__global__ __launch_bounds__(256) void quantize_fp8_kernel(const char* __restrict__ x, long long n,
                                                           const float* __restrict__ partial, int nparts,
                                                           unsigned char* __restrict__ q, char* __restrict__ scale) {
  __shared__ float wm[4];
  float mx = 0.f;
  bool has_nan = false;
  for (int i = threadIdx.x; i < nparts; i += 256) {
    const float v = partial[i];
    has_nan |= v != v;
    mx = fmaxf(mx, v);
  }
  mx = fc_wave_max(mx);
  if (__any(has_nan)) mx = __builtin_nanf("");
  if ((threadIdx.x & 63) == 0) wm[threadIdx.x >> 6] = mx;
  __syncthreads();
  mx = wm[0];
  for (int w = 1; w < 4; ++w) mx = (mx != mx || wm[w] != wm[w]) ? __builtin_nanf("") : fmaxf(mx, wm[w]);
  float sc = qz_round<DTYPE>(mx / 448.f);
  sc = qz_round<DTYPE>(sc != sc ? sc : fmaxf(sc, 1e-8f));
  if (blockIdx.x == 0 && threadIdx.x == 0) qz_store<DTYPE>(scale, 0, sc);
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long long)gridDim.x * 256)
    q[i] = qz_to_fp8<E5M2>(qz_round<DTYPE>(qz_load<DTYPE>(x, i) / sc));
}

// out = float(code) * scale, rounded to the output dtype (every fp8 value is exact in fp16 and bf16)
template <int SDT, int ODT, int E5M2>
__global__ __launch_bounds__(256) void dequantize_fp8_kernel(const unsigned char* __restrict__ q,
                                                             const char* __restrict__ scale, long long n,
                                                             char* __restrict__ out) {
  const float sc = qz_load<SDT>(scale, 0);
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long long)gridDim.x * 256)
    qz_store<ODT>(out, i, qz_from_fp8<E5M2>(q[i]) * sc);
}

// ---- asymmetric 8-bit rows -----------------------------------------------------------------------
// scale = clamp((max - min) / 255, 1e-8), zero = clamp(round(-min / scale), 0, 255),
// code = clamp(round((x - min) / scale), 0, 255); params[row] = (scale, zero) in the dtype of x
template <int DTYPE>
__global__ __launch_bounds__(256) void quantize_rows_asym_kernel(const char* __restrict__ x, long long rows, int d,
                                                                 unsigned char* __restrict__ q,
                                                                 char* __restrict__ params) {
  const long long r = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (r >= rows) return;
  const long long base = r * d;
  float mn = INFINITY, mx = -INFINITY;
  bool has_nan = false;
  for (int j = lane; j < d; j += 64) {
    const float v = qz_load<DTYPE>(x, base + j);
    has_nan |= v != v;
    mn = fminf(mn, v);
    mx = fmaxf(mx, v);
  }
  mn = -fc_wave_max(-mn);
  mx = fc_wave_max(mx);
  if (__any(has_nan)) mn = mx = __builtin_nanf("");
  float sc = qz_round<DTYPE>(qz_round<DTYPE>(mx - mn) / 255.f);
  sc = qz_round<DTYPE>(sc != sc ? sc : fmaxf(sc, 1e-8f));
  float zp = rintf(qz_round<DTYPE>(-mn / sc));
  zp = (zp != zp) ? zp : fminf(fmaxf(zp, 0.f), 255.f);   // clamp keeps NaN
  if (lane == 0) {
    qz_store<DTYPE>(params, 2 * r, sc);
    qz_store<DTYPE>(params, 2 * r + 1, zp);
  }
  for (int j = lane; j < d; j += 64) {
    float t = qz_round<DTYPE>(qz_round<DTYPE>(qz_load<DTYPE>(x, base + j) - mn) / sc);
    t = fminf(fmaxf(rintf(t), 0.f), 255.f);
    q[base + j] = (t != t) ? (unsigned char)0 : (unsigned char)(int)t;
  }
}

// ---- 16 bytes per lane: rows (or groups) of 128, 256 or 512 bytes, and flat element-wise passes ------------------
// A row is covered by LPR = row bytes / 16 lanes with one 16-byte load each and stays in registers between the
// reduction and the second step; a thread handles QZ_U rows so that several loads are in flight.  The arithmetic is
// the same, step for step, as in the kernels above, which remain the path for every other row length.
// largest grids of the flat passes (their workgroups loop beyond that)
#ifndef QZ_GRID_CAP
#define QZ_GRID_CAP 8192
#endif
#ifndef QZ_GRID_CAP8
#define QZ_GRID_CAP8 16384
#endif
#ifndef QZ_U
#define QZ_U 4
#endif

template <int DTYPE>
struct QzV {
  static constexpr int EB = DTYPE == FC_F32 ? 4 : 2;
  static constexpr int EPL = 16 / EB;   // elements per lane
};

template <int DTYPE>
__device__ __forceinline__ void qz_unpack(const uint4& x, float (&v)[QzV<DTYPE>::EPL]) {
  const unsigned w[4] = {x.x, x.y, x.z, x.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if constexpr (DTYPE == FC_F32) {
      v[i] = __uint_as_float(w[i]);
    } else {
      v[2 * i] = DTYPE == FC_BF16 ? fc_bf16_to_float((unsigned short)(w[i] & 0xffff)) : fc_half_to_float((unsigned short)(w[i] & 0xffff));
      v[2 * i + 1] = DTYPE == FC_BF16 ? fc_bf16_to_float((unsigned short)(w[i] >> 16)) : fc_half_to_float((unsigned short)(w[i] >> 16));
    }
  }
}
template <int DTYPE>
__device__ __forceinline__ uint4 qz_pack(const float (&v)[QzV<DTYPE>::EPL]) {
  unsigned w[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if constexpr (DTYPE == FC_F32) {
      w[i] = __float_as_uint(v[i]);
    } else {
      const unsigned lo = DTYPE == FC_BF16 ? fc_float_to_bf16(v[2 * i]) : fc_float_to_half(v[2 * i]);
      const unsigned hi = DTYPE == FC_BF16 ? fc_float_to_bf16(v[2 * i + 1]) : fc_float_to_half(v[2 * i + 1]);
      w[i] = lo | (hi << 16);
    }
  }
  return make_uint4(w[0], w[1], w[2], w[3]);
}
// reductions over the LPR consecutive lanes that share a row (LPR = 8, 16 or 32)
template <int LPR>
__device__ __forceinline__ float qz_row_max(float v) {
  v = fc_group_max<(LPR < 16 ? LPR : 16)>(v);
  if constexpr (LPR == 32) v = fmaxf(v, __shfl_xor(v, 16, 64));
  return v;
}

// KIND 0: symmetric codes (int8 store), 1: asymmetric codes + (scale, zero), 2: quantise -> dequantise,
// 3 / 4: packed 4-bit integer / NF4 codes of a group
template <int DTYPE, int LPR, int KIND>
__global__ __launch_bounds__(256) void quant_rows_fast_kernel(const char* __restrict__ x, long long rows, float qmax,
                                                              char* __restrict__ out, char* __restrict__ scale,
                                                              char* __restrict__ absmax) {
  constexpr int EPL = QzV<DTYPE>::EPL;
  constexpr int RPB = 256 / LPR;   // rows per block and step
  __shared__ float levels[16];
  if (KIND == 4) {
    qz_fill_levels<DTYPE>(levels);
    __syncthreads();
  }
  const int sub = threadIdx.x % LPR, rg = threadIdx.x / LPR;
  uint4 xin[QZ_U];
  long long row[QZ_U];
#pragma unroll
  for (int u = 0; u < QZ_U; ++u) {   // every lane loads (a row past the end re-reads the last one)
    row[u] = ((long long)blockIdx.x * QZ_U + u) * RPB + rg;
    const long long rc = row[u] < rows ? row[u] : rows - 1;
    xin[u] = *reinterpret_cast<const uint4*>(x + (rc * LPR + sub) * 16);
  }
#pragma unroll
  for (int u = 0; u < QZ_U; ++u) {
    const bool live = row[u] < rows;
    const long long r = row[u];
    float v[EPL];
    qz_unpack<DTYPE>(xin[u], v);
    float mx = KIND == 1 ? -INFINITY : 0.f, mn = INFINITY, nanf = 0.f;
#pragma unroll
    for (int j = 0; j < EPL; ++j) {
      if (v[j] != v[j]) nanf = 1.f;
      mx = fmaxf(mx, KIND == 1 ? v[j] : fabsf(v[j]));
      if (KIND == 1) mn = fminf(mn, v[j]);
    }
    mx = qz_row_max<LPR>(mx);
    if (KIND == 1) mn = -qz_row_max<LPR>(-mn);
    if (qz_row_max<LPR>(nanf) > 0.f) mx = mn = __builtin_nanf("");
    if constexpr (KIND == 0 || KIND == 3 || KIND == 4) {
      float sc = KIND == 4 ? mx : qz_round<DTYPE>(mx / qmax);
      sc = qz_round<DTYPE>(sc != sc ? sc : fmaxf(sc, 1e-8f));
      if (live && sub == 0) qz_store<DTYPE>(scale, r, sc);
      if constexpr (KIND == 0) {
        unsigned w[EPL / 4] = {};
#pragma unroll
        for (int j = 0; j < EPL; ++j) {
          float t = rintf(qz_round<DTYPE>(v[j] / sc));
          const bool is_nan = t != t;
          t = fminf(fmaxf(t, -qmax - 1.f), qmax);
          const int c = is_nan ? 0 : (int)t;
          w[j / 4] |= ((unsigned)c & 0xffu) << (8 * (j & 3));
        }
        if (live) {
          if constexpr (EPL == 8) *reinterpret_cast<uint2*>(out + (r * LPR + sub) * 8) = make_uint2(w[0], w[1]);
          else *reinterpret_cast<unsigned*>(out + (r * LPR + sub) * 4) = w[0];
        }
      } else {
        unsigned w = 0;
#pragma unroll
        for (int j = 0; j < EPL; ++j) w |= (unsigned)qz_code4<DTYPE, KIND == 4 ? 1 : 0>(v[j], sc, levels) << (4 * j);
        if (live) {
          if constexpr (EPL == 8) *reinterpret_cast<unsigned*>(out + (r * LPR + sub) * 4) = w;
          else *reinterpret_cast<unsigned short*>(out + (r * LPR + sub) * 2) = (unsigned short)w;
        }
      }
    } else if constexpr (KIND == 1) {
      float sc = qz_round<DTYPE>(qz_round<DTYPE>(mx - mn) / 255.f);
      sc = qz_round<DTYPE>(sc != sc ? sc : fmaxf(sc, 1e-8f));
      float zp = rintf(qz_round<DTYPE>(-mn / sc));
      zp = (zp != zp) ? zp : fminf(fmaxf(zp, 0.f), 255.f);   // clamp keeps NaN
      if (live && sub == 0) {
        qz_store<DTYPE>(scale, 2 * r, sc);
        qz_store<DTYPE>(scale, 2 * r + 1, zp);
      }
      unsigned w[EPL / 4] = {};
#pragma unroll
      for (int j = 0; j < EPL; ++j) {
        float t = qz_round<DTYPE>(qz_round<DTYPE>(v[j] - mn) / sc);
        t = fminf(fmaxf(rintf(t), 0.f), 255.f);
        const unsigned c = (t != t) ? 0u : (unsigned)(int)t;
        w[j / 4] |= c << (8 * (j & 3));
      }
      if (live) {
        if constexpr (EPL == 8) *reinterpret_cast<uint2*>(out + (r * LPR + sub) * 8) = make_uint2(w[0], w[1]);
        else *reinterpret_cast<unsigned*>(out + (r * LPR + sub) * 4) = w[0];
      }
    } else {
      const float sc = qz_round<DTYPE>(mx / qmax);
      if (live && sub == 0) {
        if (scale) qz_store<DTYPE>(scale, r, sc);
        if (absmax) qz_store<DTYPE>(absmax, r, mx);
      }
      float y[EPL];
#pragma unroll
      for (int j = 0; j < EPL; ++j) y[j] = qz_fake<DTYPE>(v[j], sc, qmax);
      if (live) *reinterpret_cast<uint4*>(out + (r * LPR + sub) * 16) = qz_pack<DTYPE>(y);
    }
  }
}

// ---- flat passes, 8 output elements (one 16- or 8-byte access on each side) per thread ---------------------------
// store 8 values in the output dtype
template <int ODT>
__device__ __forceinline__ void qz_store8(char* out, long long i8, const float (&y)[8]) {
  if constexpr (ODT == FC_F32) {
    uint4* o = reinterpret_cast<uint4*>(out) + 2 * i8;
    o[0] = make_uint4(__float_as_uint(y[0]), __float_as_uint(y[1]), __float_as_uint(y[2]), __float_as_uint(y[3]));
    o[1] = make_uint4(__float_as_uint(y[4]), __float_as_uint(y[5]), __float_as_uint(y[6]), __float_as_uint(y[7]));
  } else {
    reinterpret_cast<uint4*>(out)[i8] = qz_pack<ODT>(y);
  }
}

// out = float(code) * scale: int8 rows (KIND 0, one scale per d codes), fp8 (KIND 1 / 2 = E4M3 / E5M2, one scale)
template <int SDT, int ODT, int KIND>
__global__ __launch_bounds__(256) void dequantize_vec_kernel(const unsigned char* __restrict__ q,
                                                             const char* __restrict__ scale, long long n8, int d,
                                                             char* __restrict__ out) {
  const float sc1 = KIND == 0 ? 0.f : qz_load<SDT>(scale, 0);
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n8; i += (long long)gridDim.x * 256) {
    const uint2 c = reinterpret_cast<const uint2*>(q)[i];
    const float sc = KIND == 0 ? qz_load<SDT>(scale, (i * 8) / d) : sc1;
    float y[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const unsigned b = ((j < 4 ? c.x : c.y) >> (8 * (j & 3))) & 0xffu;
      const float v = KIND == 0 ? (float)(signed char)b : KIND == 1 ? qz_from_fp8<0>((unsigned char)b) : qz_from_fp8<1>((unsigned char)b);
      y[j] = v * sc;
    }
    qz_store8<ODT>(out, i, y);
  }
}

// 4-bit codes, 8 elements = 4 bytes per thread; one scale per g elements
template <int TDT, int SDT, int ODT, int MODE>
__global__ __launch_bounds__(256) void dequantize_group4_vec_kernel(const unsigned char* __restrict__ packed,
                                                                    const char* __restrict__ scale, long long n8, int g,
                                                                    char* __restrict__ out) {
  __shared__ float levels[16];
  if (MODE == 1) {
    qz_fill_levels<TDT>(levels);
    __syncthreads();
  }
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n8; i += (long long)gridDim.x * 256) {
    const unsigned c = reinterpret_cast<const unsigned*>(packed)[i];
    const float sc = qz_load<SDT>(scale, (i * 8) / g);
    float y[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const unsigned code = (c >> (4 * j)) & 15u;
      y[j] = (MODE == 0 ? (float)(int)code - 8.f : levels[code]) * sc;
    }
    qz_store8<ODT>(out, i, y);
  }
}

// whole-tensor passes over 16-byte pieces: the largest |x| of a block's share, fp8 codes, quantise -> dequantise
template <int DTYPE>
__global__ __launch_bounds__(256) void absmax_partial_vec_kernel(const char* __restrict__ x, long long nv, long long n,
                                                                 float* __restrict__ partial) {
  constexpr int EPL = QzV<DTYPE>::EPL;
  __shared__ float wm[4];
  float mx = 0.f;
  bool has_nan = false;
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < nv; i += (long long)gridDim.x * 256) {
    float v[EPL];
    qz_unpack<DTYPE>(reinterpret_cast<const uint4*>(x)[i], v);
#pragma unroll
    for (int j = 0; j < EPL; ++j) {
      has_nan |= v[j] != v[j];
      mx = fmaxf(mx, fabsf(v[j]));
    }
  }
  for (long long i = nv * EPL + (long long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long long)gridDim.x * 256) {
    const float v = qz_load<DTYPE>(x, i);
    has_nan |= v != v;
    mx = fmaxf(mx, fabsf(v));
  }
  mx = fc_wave_max(mx);
  if (__any(has_nan)) mx = __builtin_nanf("");
  if ((threadIdx.x & 63) == 0) wm[threadIdx.x >> 6] = mx;
  __syncthreads();
  if (threadIdx.x == 0) {
    float m = wm[0];
    for (int w = 1; w < 4; ++w) m = (m != m || wm[w] != wm[w]) ? __builtin_nanf("") : fmaxf(m, wm[w]);
    partial[blockIdx.x] = m;
  }
}

// the tensor's largest |x| from the partial maxima (every block repeats this small reduction)
__device__ __forceinline__ float qz_reduce_partials(const float* __restrict__ partial, int nparts, float* wm) {
  float mx = 0.f;
  bool has_nan = false;
  for (int i = threadIdx.x; i < nparts; i += 256) {
    const float v = partial[i];
    has_nan |= v != v;
    mx = fmaxf(mx, v);
  }
  mx = fc_wave_max(mx);
  if (__any(has_nan)) mx = __builtin_nanf("");
  if ((threadIdx.x & 63) == 0) wm[threadIdx.x >> 6] = mx;
  __syncthreads();
  mx = wm[0];
  for (int w = 1; w < 4; ++w) mx = (mx != mx || wm[w] != wm[w]) ? __builtin_nanf("") : fmaxf(mx, wm[w]);
  return mx;
}

// MODE 0: y = quantise -> dequantise with the whole-tensor scale; MODE 1 / 2: fp8 codes (E4M3 / E5M2)
template <int DTYPE, int MODE>
__global__ __launch_bounds__(256) void tensor_apply_vec_kernel(const char* __restrict__ x, long long nv, long long n,
                                                               const float* __restrict__ partial, int nparts,
                                                               float qmax, char* __restrict__ y,
                                                               char* __restrict__ scale, char* __restrict__ absmax) {
  constexpr int EPL = QzV<DTYPE>::EPL;
  __shared__ float wm[4];
  const float mx = qz_reduce_partials(partial, nparts, wm);
  float sc;
  if (MODE == 0) {
    sc = qz_round<DTYPE>(mx / qmax);
  } else {
    sc = qz_round<DTYPE>(mx / 448.f);
    sc = qz_round<DTYPE>(sc != sc ? sc : fmaxf(sc, 1e-8f));
  }
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    if (scale) qz_store<DTYPE>(scale, 0, sc);
    if (absmax) qz_store<DTYPE>(absmax, 0, mx);
  }
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < nv; i += (long long)gridDim.x * 256) {
    float v[EPL];
    qz_unpack<DTYPE>(reinterpret_cast<const uint4*>(x)[i], v);
    if constexpr (MODE == 0) {
      float o[EPL];
#pragma unroll
      for (int j = 0; j < EPL; ++j) o[j] = qz_fake<DTYPE>(v[j], sc, qmax);
      reinterpret_cast<uint4*>(y)[i] = qz_pack<DTYPE>(o);
    } else {
      unsigned w[EPL / 4] = {};
#pragma unroll
      for (int j = 0; j < EPL; ++j)
        w[j / 4] |= (unsigned)qz_to_fp8<MODE == 2>(qz_round<DTYPE>(v[j] / sc)) << (8 * (j & 3));
      if constexpr (EPL == 8) reinterpret_cast<uint2*>(y)[i] = make_uint2(w[0], w[1]);
      else reinterpret_cast<unsigned*>(y)[i] = w[0];
    }
  }
  for (long long i = nv * EPL + (long long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long long)gridDim.x * 256) {
    const float v = qz_load<DTYPE>(x, i);
    if constexpr (MODE == 0) qz_store<DTYPE>(y, i, qz_fake<DTYPE>(v, sc, qmax));
    else reinterpret_cast<unsigned char*>(y)[i] = qz_to_fp8<MODE == 2>(qz_round<DTYPE>(v / sc));
  }
}

// row bytes 128 / 256 / 512 and 16-byte aligned input -> lanes per row, else 0
static inline int qz_fast_lpr(const void* x, long long row_elems, int dtype) {
  const long long bytes = row_elems * (dtype == FC_F32 ? 4 : 2);
  if (((uintptr_t)x & 15) != 0) return 0;
  return bytes == 128 ? 8 : bytes == 256 ? 16 : bytes == 512 ? 32 : 0;
}

#define QZ_FAST_LAUNCH(DT, LPRV, KIND, ...)                                                                        \
  do {                                                                                                             \
    const long long per_block = (256 / (LPRV)) * QZ_U;                                                             \
    const long long nb = (rows_ + per_block - 1) / per_block;                                                      \
    if (nb > 2147483647LL) { fc_set_error("%s: too many rows", who); return FC_EUNSUPPORTED; }                     \
    hipLaunchKernelGGL((quant_rows_fast_kernel<DT, LPRV, KIND>), dim3((unsigned)nb), dim3(256), 0, st, __VA_ARGS__); \
  } while (0)
#define QZ_FAST_LPR(DT, KIND, ...)                                   \
  do {                                                               \
    if (lpr == 8) QZ_FAST_LAUNCH(DT, 8, KIND, __VA_ARGS__);          \
    else if (lpr == 16) QZ_FAST_LAUNCH(DT, 16, KIND, __VA_ARGS__);   \
    else QZ_FAST_LAUNCH(DT, 32, KIND, __VA_ARGS__);                  \
  } while (0)
#define QZ_FAST(KIND, ...)                                           \
  do {                                                               \
    if (dtype == FC_F32) QZ_FAST_LPR(FC_F32, KIND, __VA_ARGS__);     \
    else if (dtype == FC_F16) QZ_FAST_LPR(FC_F16, KIND, __VA_ARGS__); \
    else QZ_FAST_LPR(FC_BF16, KIND, __VA_ARGS__);                    \
  } while (0)

extern "C" int64_t fc_fake_quantize_workspace_bytes(void) { return QZ_PARTS * (int64_t)sizeof(float); }

extern "C" int fc_fake_quantize(const void* x, void* y, int64_t rows, int32_t d, int32_t dtype, int32_t bits,
                                int32_t per_tensor, void* scale, void* absmax, void* workspace,
                                int64_t workspace_bytes, void* stream) {
  const char* who = "fc_fake_quantize";
  FC_REQUIRE(x && y, FC_EINVAL, "%s: null pointer", who);
  FC_REQUIRE(rows >= 0 && d > 0, FC_EINVAL, "%s: bad sizes rows=%lld d=%d", who, (long long)rows, d);
  FC_REQUIRE(bits >= 2 && bits <= 16, FC_EINVAL, "%s: bits must be in [2, 16] (got %d)", who, bits);
  FC_REQUIRE(dtype == FC_F32 || dtype == FC_F16 || dtype == FC_BF16, FC_EUNSUPPORTED, "%s: dtype %d", who, dtype);
  if (rows == 0) return FC_OK;
  const float qmax = (float)((1 << (bits - 1)) - 1);
  hipStream_t st = (hipStream_t)stream;
  if (!per_tensor && qz_fast_lpr(x, d, dtype) && ((uintptr_t)y & 15) == 0) {
    const int lpr = qz_fast_lpr(x, d, dtype);
    const long long rows_ = rows;
    QZ_FAST(2, (const char*)x, (long long)rows, qmax, (char*)y, (char*)scale, (char*)absmax);
  } else if (!per_tensor) {
    const long long blocks = (rows + 3) / 4;
    FC_REQUIRE(blocks <= 2147483647LL, FC_EUNSUPPORTED, "%s: too many rows", who);
#define FQ(DT) hipLaunchKernelGGL((fake_quant_rows_kernel<DT>), dim3((unsigned)blocks), dim3(256), 0, st, (const char*)x, \
                                  (long long)rows, d, qmax, (char*)y, (char*)scale, (char*)absmax)
    if (dtype == FC_F32) FQ(FC_F32); else if (dtype == FC_F16) FQ(FC_F16); else FQ(FC_BF16);
#undef FQ
  } else {
    FC_REQUIRE(workspace && workspace_bytes >= fc_fake_quantize_workspace_bytes(), FC_EINVAL,
               "%s: the whole-tensor scale needs a workspace of %lld bytes", who,
               (long long)fc_fake_quantize_workspace_bytes());
    const long long n = rows * (long long)d;
    const int nparts = (int)((n + 255) / 256 < QZ_PARTS ? (n + 255) / 256 : QZ_PARTS);
    const long long want = (n + 1023) / 1024;
    const unsigned blocks = (unsigned)(want < QZ_GRID_CAP ? (want > 0 ? want : 1) : QZ_GRID_CAP);
    const bool vec = (((uintptr_t)x | (uintptr_t)y) & 15) == 0;
#define FT(DT)                                                                                                       \
  do {                                                                                                               \
    if (vec) {                                                                                                       \
      const long long nv = n / QzV<DT>::EPL;                                                                         \
      hipLaunchKernelGGL((absmax_partial_vec_kernel<DT>), dim3(nparts), dim3(256), 0, st, (const char*)x, nv, n,     \
                         (float*)workspace);                                                                         \
      hipLaunchKernelGGL((tensor_apply_vec_kernel<DT, 0>), dim3(blocks), dim3(256), 0, st, (const char*)x, nv, n,    \
                         (const float*)workspace, nparts, qmax, (char*)y, (char*)scale, (char*)absmax);              \
    } else {                                                                                                         \
      hipLaunchKernelGGL((absmax_partial_kernel<DT>), dim3(nparts), dim3(256), 0, st, (const char*)x, n,             \
                         (float*)workspace);                                                                         \
      hipLaunchKernelGGL((fake_quant_tensor_kernel<DT>), dim3(blocks), dim3(256), 0, st, (const char*)x, n,          \
                         (const float*)workspace, nparts, qmax, (char*)y, (char*)scale, (char*)absmax);              \
    }                                                                                                                \
  } while (0)
    if (dtype == FC_F32) FT(FC_F32); else if (dtype == FC_F16) FT(FC_F16); else FT(FC_BF16);
#undef FT
  }
  FC_CHECK_LAUNCH(who);
  return FC_OK;
}

extern "C" int fc_quantize_rows(const void* x, int64_t rows, int32_t d, int32_t dtype, int32_t bits, int8_t* q,
                                void* scale, void* stream) {
  const char* who = "fc_quantize_rows";
  FC_REQUIRE(x && q && scale, FC_EINVAL, "%s: null pointer", who);
  FC_REQUIRE(rows >= 0 && d > 0, FC_EINVAL, "%s: bad sizes rows=%lld d=%d", who, (long long)rows, d);
  FC_REQUIRE(bits >= 2 && bits <= 8, FC_EINVAL, "%s: bits must be in [2, 8] (got %d)", who, bits);
  FC_REQUIRE(dtype == FC_F32 || dtype == FC_F16 || dtype == FC_BF16, FC_EUNSUPPORTED, "%s: dtype %d", who, dtype);
  if (rows == 0) return FC_OK;
  const long long blocks = (rows + 3) / 4;
  FC_REQUIRE(blocks <= 2147483647LL, FC_EUNSUPPORTED, "%s: too many rows", who);
  const float qmax = (float)((1 << (bits - 1)) - 1);
  hipStream_t st = (hipStream_t)stream;
  if (const int lpr = qz_fast_lpr(x, d, dtype); lpr && ((uintptr_t)q & 7) == 0) {
    const long long rows_ = rows;
    QZ_FAST(0, (const char*)x, (long long)rows, qmax, (char*)q, (char*)scale, (char*)nullptr);
    FC_CHECK_LAUNCH(who);
    return FC_OK;
  }
#define QZ(DT) hipLaunchKernelGGL((quantize_rows_kernel<DT>), dim3((unsigned)blocks), dim3(256), 0, st, (const char*)x, \
                                  (long long)rows, d, qmax, (signed char*)q, (char*)scale)
  if (dtype == FC_F32) QZ(FC_F32); else if (dtype == FC_F16) QZ(FC_F16); else QZ(FC_BF16);
#undef QZ
  FC_CHECK_LAUNCH(who);
  return FC_OK;
}

extern "C" int fc_dequantize_rows(const int8_t* q, const void* scale, int64_t rows, int32_t d, int32_t scale_dtype,
                                  int32_t out_dtype, void* out, void* stream) {
  const char* who = "fc_dequantize_rows";
  FC_REQUIRE(q && scale && out, FC_EINVAL, "%s: null pointer", who);
  FC_REQUIRE(rows >= 0 && d > 0, FC_EINVAL, "%s: bad sizes rows=%lld d=%d", who, (long long)rows, d);
  if (rows == 0) return FC_OK;
  const long long blocks = (rows + 3) / 4;
  FC_REQUIRE(blocks <= 2147483647LL, FC_EUNSUPPORTED, "%s: too many rows", who);
  hipStream_t st = (hipStream_t)stream;
  const bool vec = d % 8 == 0 && ((uintptr_t)q & 7) == 0 && ((uintptr_t)out & 15) == 0;
  const long long n8 = rows * (long long)d / 8, want8 = (n8 + 255) / 256;
  // one pass per workgroup (no loop) as far as a grid reaches: the int8 form has nothing to set up per workgroup, and
  // short-lived workgroups stream fastest (2.4 GB of bf16 out: 0.644 ms against 0.712 ms with 16384 looping workgroups)
  const unsigned blocks8 = (unsigned)(want8 < 0x7fffffffLL ? (want8 > 0 ? want8 : 1) : 0x7fffffffLL);
#define DQ(S, O)                                                                                                     \
  do {                                                                                                               \
    if (vec)                                                                                                         \
      hipLaunchKernelGGL((dequantize_vec_kernel<S, O, 0>), dim3(blocks8), dim3(256), 0, st, (const unsigned char*)q, \
                         (const char*)scale, n8, d, (char*)out);                                                     \
    else                                                                                                             \
      hipLaunchKernelGGL((dequantize_rows_kernel<S, O>), dim3((unsigned)blocks), dim3(256), 0, st,                   \
                         (const signed char*)q, (const char*)scale, (long long)rows, d, (char*)out);                 \
  } while (0)
  // the output dtype is the promotion of the two: equal dtypes, or fp32 when either side is fp32
  if (scale_dtype == out_dtype) {
    if (out_dtype == FC_F32) DQ(FC_F32, FC_F32);
    else if (out_dtype == FC_F16) DQ(FC_F16, FC_F16);
    else if (out_dtype == FC_BF16) DQ(FC_BF16, FC_BF16);
    else { fc_set_error("%s: dtype %d", who, out_dtype); return FC_EUNSUPPORTED; }
  } else if (out_dtype == FC_F32 && scale_dtype == FC_F16) DQ(FC_F16, FC_F32);
  else if (out_dtype == FC_F32 && scale_dtype == FC_BF16) DQ(FC_BF16, FC_F32);
  else { fc_set_error("%s: scale dtype %d with output dtype %d", who, scale_dtype, out_dtype); return FC_EUNSUPPORTED; }
#undef DQ
  FC_CHECK_LAUNCH(who);
  return FC_OK;
}

extern "C" int fc_quantize_fp8(const void* x, int64_t n, int32_t dtype, int32_t e5m2, uint8_t* q, void* scale,
                               void* workspace, int64_t workspace_bytes, void* stream) {
  const char* who = "fc_quantize_fp8";
  FC_REQUIRE(x && q && scale, FC_EINVAL, "%s: null pointer", who);
  FC_REQUIRE(n >= 0, FC_EINVAL, "%s: bad size %lld", who, (long long)n);
  FC_REQUIRE(dtype == FC_F32 || dtype == FC_F16 || dtype == FC_BF16, FC_EUNSUPPORTED, "%s: dtype %d", who, dtype);
  FC_REQUIRE(workspace && workspace_bytes >= fc_fake_quantize_workspace_bytes(), FC_EINVAL,
             "%s: needs a workspace of %lld bytes", who, (long long)fc_fake_quantize_workspace_bytes());
  if (n == 0) return FC_OK;
  hipStream_t st = (hipStream_t)stream;
  const int nparts = (int)((n + 255) / 256 < QZ_PARTS ? (n + 255) / 256 : QZ_PARTS);
  const long long want = (n + 1023) / 1024;
  const unsigned blocks = (unsigned)(want < QZ_GRID_CAP ? want : QZ_GRID_CAP);
  const bool vec = ((uintptr_t)x & 15) == 0 && ((uintptr_t)q & 7) == 0;
#define F8(DT)                                                                                                       \
  do {                                                                                                               \
    if (vec) {                                                                                                       \
      const long long nv = n / QzV<DT>::EPL;                                                                         \
      hipLaunchKernelGGL((absmax_partial_vec_kernel<DT>), dim3(nparts), dim3(256), 0, st, (const char*)x, nv,        \
                         (long long)n, (float*)workspace);                                                           \
      if (e5m2)                                                                                                      \
        hipLaunchKernelGGL((tensor_apply_vec_kernel<DT, 2>), dim3(blocks), dim3(256), 0, st, (const char*)x, nv,     \
                           (long long)n, (const float*)workspace, nparts, 0.f, (char*)q, (char*)scale,               \
                           (char*)nullptr);                                                                          \
      else                                                                                                           \
        hipLaunchKernelGGL((tensor_apply_vec_kernel<DT, 1>), dim3(blocks), dim3(256), 0, st, (const char*)x, nv,     \
                           (long long)n, (const float*)workspace, nparts, 0.f, (char*)q, (char*)scale,               \
                           (char*)nullptr);                                                                          \
      break;                                                                                                         \
    }                                                                                                                \
    hipLaunchKernelGGL((absmax_partial_kernel<DT>), dim3(nparts), dim3(256), 0, st, (const char*)x, (long long)n,   \
                       (float*)workspace);                                                                           \
    if (e5m2)                                                                                                        \
      hipLaunchKernelGGL((quantize_fp8_kernel<DT, 1>), dim3(blocks), dim3(256), 0, st, (const char*)x, (long long)n, \
                         (const float*)workspace, nparts, (unsigned char*)q, (char*)scale);                          \
    else                                                                                                             \
      hipLaunchKernelGGL((quantize_fp8_kernel<DT, 0>), dim3(blocks), dim3(256), 0, st, (const char*)x, (long long)n, \
                         (const float*)workspace, nparts, (unsigned char*)q, (char*)scale);                          \
  } while (0)
  if (dtype == FC_F32) F8(FC_F32); else if (dtype == FC_F16) F8(FC_F16); else F8(FC_BF16);
#undef F8
  FC_CHECK_LAUNCH(who);
  return FC_OK;
}

extern "C" int fc_dequantize_fp8(const uint8_t* q, const void* scale, int64_t n, int32_t e5m2, int32_t scale_dtype,
                                 int32_t out_dtype, void* out, void* stream) {
  const char* who = "fc_dequantize_fp8";
  FC_REQUIRE(q && scale && out, FC_EINVAL, "%s: null pointer", who);
  FC_REQUIRE(n >= 0, FC_EINVAL, "%s: bad size %lld", who, (long long)n);
  if (n == 0) return FC_OK;
  hipStream_t st = (hipStream_t)stream;
  const long long want = (n + 1023) / 1024;
  const unsigned blocks = (unsigned)(want < QZ_GRID_CAP ? want : QZ_GRID_CAP);
  const bool vec = n % 8 == 0 && ((uintptr_t)q & 7) == 0 && ((uintptr_t)out & 15) == 0;
  const long long want8 = (n / 8 + 255) / 256;
  const unsigned blocks8 = (unsigned)(want8 < QZ_GRID_CAP8 ? (want8 > 0 ? want8 : 1) : QZ_GRID_CAP8);
#define D8(S, O)                                                                                                     \
  do {                                                                                                               \
    if (vec) {                                                                                                       \
      if (e5m2)                                                                                                      \
        hipLaunchKernelGGL((dequantize_vec_kernel<S, O, 2>), dim3(blocks8), dim3(256), 0, st,                        \
                           (const unsigned char*)q, (const char*)scale, (long long)(n / 8), 1, (char*)out);          \
      else                                                                                                           \
        hipLaunchKernelGGL((dequantize_vec_kernel<S, O, 1>), dim3(blocks8), dim3(256), 0, st,                        \
                           (const unsigned char*)q, (const char*)scale, (long long)(n / 8), 1, (char*)out);          \
      break;                                                                                                         \
    }                                                                                                                \
    if (e5m2)                                                                                                        \
      hipLaunchKernelGGL((dequantize_fp8_kernel<S, O, 1>), dim3(blocks), dim3(256), 0, st, (const unsigned char*)q,  \
                         (const char*)scale, (long long)n, (char*)out);                                              \
    else                                                                                                             \
      hipLaunchKernelGGL((dequantize_fp8_kernel<S, O, 0>), dim3(blocks), dim3(256), 0, st, (const unsigned char*)q,  \
                         (const char*)scale, (long long)n, (char*)out);                                              \
  } while (0)
  // the output dtype is the promotion of the two: equal dtypes, or fp32 when either side is fp32
  if (scale_dtype == out_dtype) {
    if (out_dtype == FC_F32) D8(FC_F32, FC_F32);
    else if (out_dtype == FC_F16) D8(FC_F16, FC_F16);
    else if (out_dtype == FC_BF16) D8(FC_BF16, FC_BF16);
    else { fc_set_error("%s: dtype %d", who, out_dtype); return FC_EUNSUPPORTED; }
  } else if (out_dtype == FC_F32 && scale_dtype == FC_F16) D8(FC_F16, FC_F32);
  else if (out_dtype == FC_F32 && scale_dtype == FC_BF16) D8(FC_BF16, FC_F32);
  else { fc_set_error("%s: scale dtype %d with output dtype %d", who, scale_dtype, out_dtype); return FC_EUNSUPPORTED; }
#undef D8
  FC_CHECK_LAUNCH(who);
  return FC_OK;
}

extern "C" int fc_quantize_rows_asym(const void* x, int64_t rows, int32_t d, int32_t dtype, uint8_t* q, void* params,
                                     void* stream) {
  const char* who = "fc_quantize_rows_asym";
  FC_REQUIRE(x && q && params, FC_EINVAL, "%s: null pointer", who);
  FC_REQUIRE(rows >= 0 && d > 0, FC_EINVAL, "%s: bad sizes rows=%lld d=%d", who, (long long)rows, d);
  FC_REQUIRE(dtype == FC_F32 || dtype == FC_F16 || dtype == FC_BF16, FC_EUNSUPPORTED, "%s: dtype %d", who, dtype);
  if (rows == 0) return FC_OK;
  const long long blocks = (rows + 3) / 4;
  FC_REQUIRE(blocks <= 2147483647LL, FC_EUNSUPPORTED, "%s: too many rows", who);
  hipStream_t st = (hipStream_t)stream;
  if (const int lpr = qz_fast_lpr(x, d, dtype); lpr && ((uintptr_t)q & 7) == 0) {
    const long long rows_ = rows;
    QZ_FAST(1, (const char*)x, (long long)rows, 0.f, (char*)q, (char*)params, (char*)nullptr);
    FC_CHECK_LAUNCH(who);
    return FC_OK;
  }
#define QA(DT) hipLaunchKernelGGL((quantize_rows_asym_kernel<DT>), dim3((unsigned)blocks), dim3(256), 0, st,          \
                                  (const char*)x, (long long)rows, d, (unsigned char*)q, (char*)params)
  if (dtype == FC_F32) QA(FC_F32); else if (dtype == FC_F16) QA(FC_F16); else QA(FC_BF16);
#undef QA
  FC_CHECK_LAUNCH(who);
  return FC_OK;
}

extern "C" int fc_quantize_group4(const void* x, int64_t groups, int32_t group_size, int32_t dtype, int32_t nf4,
                                  uint8_t* packed, void* scale, void* stream) {
  const char* who = "fc_quantize_group4";
  FC_REQUIRE(x && packed && scale, FC_EINVAL, "%s: null pointer", who);
  FC_REQUIRE(groups >= 0 && group_size > 0 && group_size % 2 == 0, FC_EINVAL, "%s: bad sizes groups=%lld group_size=%d",
             who, (long long)groups, group_size);
  FC_REQUIRE(dtype == FC_F32 || dtype == FC_F16 || dtype == FC_BF16, FC_EUNSUPPORTED, "%s: dtype %d", who, dtype);
  if (groups == 0) return FC_OK;
  const long long blocks = (groups + 3) / 4;
  FC_REQUIRE(blocks <= 2147483647LL, FC_EUNSUPPORTED, "%s: too many groups", who);
  hipStream_t st = (hipStream_t)stream;
  if (const int lpr = qz_fast_lpr(x, group_size, dtype); lpr && ((uintptr_t)packed & 3) == 0) {
    const long long rows_ = groups;
    if (nf4) QZ_FAST(4, (const char*)x, (long long)groups, 1.f, (char*)packed, (char*)scale, (char*)nullptr);
    else QZ_FAST(3, (const char*)x, (long long)groups, 7.f, (char*)packed, (char*)scale, (char*)nullptr);
    FC_CHECK_LAUNCH(who);
    return FC_OK;
  }
#define QG(DT, MD) hipLaunchKernelGGL((quantize_group4_kernel<DT, MD>), dim3((unsigned)blocks), dim3(256), 0, st,     \
                                      (const char*)x, (long long)groups, group_size, (unsigned char*)packed, (char*)scale)
#define QGD(DT) do { if (nf4) QG(DT, 1); else QG(DT, 0); } while (0)
  if (dtype == FC_F32) QGD(FC_F32); else if (dtype == FC_F16) QGD(FC_F16); else QGD(FC_BF16);
#undef QGD
#undef QG
  FC_CHECK_LAUNCH(who);
  return FC_OK;
}

extern "C" int fc_dequantize_group4(const uint8_t* packed, const void* scale, int64_t groups, int32_t group_size,
                                    int32_t scale_dtype, int32_t table_dtype, int32_t nf4, void* out, void* stream) {
  const char* who = "fc_dequantize_group4";
  FC_REQUIRE(packed && scale && out, FC_EINVAL, "%s: null pointer", who);
  FC_REQUIRE(groups >= 0 && group_size > 0 && group_size % 2 == 0, FC_EINVAL, "%s: bad sizes groups=%lld group_size=%d",
             who, (long long)groups, group_size);
  if (groups == 0) return FC_OK;
  const long long blocks = (groups + 3) / 4;
  FC_REQUIRE(blocks <= 2147483647LL, FC_EUNSUPPORTED, "%s: too many groups", who);
  hipStream_t st = (hipStream_t)stream;
  const bool vec = group_size % 8 == 0 && ((uintptr_t)packed & 3) == 0 && ((uintptr_t)out & 15) == 0;
  const long long n8 = groups * (long long)group_size / 8, want8 = (n8 + 255) / 256;
  const unsigned blocks8 = (unsigned)(want8 < QZ_GRID_CAP8 ? (want8 > 0 ? want8 : 1) : QZ_GRID_CAP8);
#define DG(T, S, O, MD)                                                                                              \
  do {                                                                                                               \
    if (vec)                                                                                                         \
      hipLaunchKernelGGL((dequantize_group4_vec_kernel<T, S, O, MD>), dim3(blocks8), dim3(256), 0, st,               \
                         (const unsigned char*)packed, (const char*)scale, n8, group_size, (char*)out);              \
    else                                                                                                             \
      hipLaunchKernelGGL((dequantize_group4_kernel<T, S, O, MD>), dim3((unsigned)blocks), dim3(256), 0, st,          \
                         (const unsigned char*)packed, (const char*)scale, (long long)groups, group_size,            \
                         (char*)out);                                                                                \
  } while (0)
#define DGD(T, S, O) do { if (nf4) DG(T, S, O, 1); else DG(T, S, O, 0); } while (0)
  // output dtype = promotion of (table dtype, scale dtype): equal dtypes, or fp32 when either is fp32
  const int t = table_dtype, sd = scale_dtype;
  if (t == FC_F32 && sd == FC_F32) DGD(FC_F32, FC_F32, FC_F32);
  else if (t == FC_F16 && sd == FC_F16) DGD(FC_F16, FC_F16, FC_F16);
  else if (t == FC_BF16 && sd == FC_BF16) DGD(FC_BF16, FC_BF16, FC_BF16);
  else if (t == FC_F32 && sd == FC_F16) DGD(FC_F32, FC_F16, FC_F32);
  else if (t == FC_F32 && sd == FC_BF16) DGD(FC_F32, FC_BF16, FC_F32);
  else if (t == FC_F16 && sd == FC_F32) DGD(FC_F16, FC_F32, FC_F32);
  else if (t == FC_BF16 && sd == FC_F32) DGD(FC_BF16, FC_F32, FC_F32);
  else { fc_set_error("%s: table dtype %d with scale dtype %d", who, t, sd); return FC_EUNSUPPORTED; }
#undef DGD
#undef DG
  FC_CHECK_LAUNCH(who);
  return FC_OK;
}
