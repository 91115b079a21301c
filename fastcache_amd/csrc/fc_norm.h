// Squared-norm pieces shared by the kernels that score keys by their L2 norm.
#pragma once
#include "fc_common.h"

// sum of squares of the 16 bytes a lane holds of its row
template <int DTYPE>
__device__ __forceinline__ float row_sumsq_part(const uint4& x) {
  if (DTYPE == FC_F32) {
    const float a = __uint_as_float(x.x), b = __uint_as_float(x.y), c = __uint_as_float(x.z), d = __uint_as_float(x.w);
    return a * a + b * b + c * c + d * d;
  } else {
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
