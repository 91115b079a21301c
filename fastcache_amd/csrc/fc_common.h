// Shared host/device helpers for libfastcache_hip (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdarg.h>
#include <stdio.h>
#include "../../include/fastcache_hip.h"

#define FC_HEAD_DIM 128
#define FC_WAVE 64

// ---- error reporting -------------------------------------------------------------------------
void fc_set_error(const char* fmt, ...);

#define FC_REQUIRE(cond, code, ...)            \
  do {                                         \
    if (!(cond)) {                             \
      fc_set_error(__VA_ARGS__);               \
      return (code);                           \
    }                                          \
  } while (0)

#define FC_CHECK_LAUNCH(name)                                                  \
  do {                                                                         \
    hipError_t e__ = hipGetLastError();                                        \
    if (e__ != hipSuccess) {                                                   \
      fc_set_error("%s: launch failed: %s", name, hipGetErrorString(e__));     \
      return FC_ELAUNCH;                                                       \
    }                                                                          \
  } while (0)

// Kernels that use more than 64 KB of dynamic LDS need their limit raised once per device; `fn` names one
// instantiation (a separate flag word per expansion of the macro, one bit per device).  Setting it twice is harmless.
#define FC_ALLOW_LDS(fn, bytes)                                                                            \
  do {                                                                                                     \
    static unsigned long long allowed__ = 0ull;                                                            \
    int dev__ = 0;                                                                                         \
    (void)hipGetDevice(&dev__);                                                                            \
    if (!((allowed__ >> (dev__ & 63)) & 1ull)) {                                                           \
      (void)hipFuncSetAttribute((const void*)(fn), hipFuncAttributeMaxDynamicSharedMemorySize, (int)(bytes)); \
      allowed__ |= 1ull << (dev__ & 63);                                                                   \
    }                                                                                                      \
  } while (0)

int fc_check_view(const fc_kv_view* v, const char* who);

static inline int fc_elem_bytes(int dtype) { return dtype == FC_F32 ? 4 : 2; }

// ---- device-side copy of a view ---------------------------------------------------------------
// Passed by value as a kernel argument; strides are in elements.
struct KvView {
  char* base;
  long long stride_layer, stride_block, stride_batch, stride_token, stride_head;
  const int* block_tables;
  const int* seq_lens;
  int table_stride, block_size, block_shift;  // block_shift >= 0 when block_size is a power of two
  int batch, num_kv_heads, max_seq_len, num_layers;
};

static inline KvView fc_make_view(const fc_kv_view* v) {
  KvView d;
  d.base = (char*)v->base;
  d.stride_layer = v->stride_layer;
  d.stride_block = v->stride_block;
  d.stride_batch = v->stride_batch;
  d.stride_token = v->stride_token;
  d.stride_head = v->stride_head;
  d.block_tables = v->block_tables;
  d.seq_lens = v->seq_lens;
  d.table_stride = v->table_stride;
  d.block_size = v->block_size > 0 ? v->block_size : 1;
  d.block_shift = -1;
  for (int s = 0; s < 31; ++s)
    if ((1 << s) == d.block_size) d.block_shift = s;
  d.batch = v->batch;
  d.num_kv_heads = v->num_kv_heads;
  d.max_seq_len = v->max_seq_len;
  d.num_layers = v->num_layers;
  return d;
}

#ifdef __HIPCC__
// Element offset of token s of sequence b (layer and head offsets are added by the caller).
// Returns -1 for a paged view whose table entry is negative (unallocated).
__device__ __forceinline__ long long fc_token_offset(const KvView& v, int b, int s) {
  if (v.block_tables) {
    int blk_i, slot;
    if (v.block_shift >= 0) {
      blk_i = s >> v.block_shift;
      slot = s & (v.block_size - 1);
    } else {
      blk_i = s / v.block_size;
      slot = s - blk_i * v.block_size;
    }
    int blk = v.block_tables[(long long)b * v.table_stride + blk_i];
    if (blk < 0) return -1;
    return (long long)blk * v.stride_block + (long long)slot * v.stride_token;
  }
  return (long long)b * v.stride_batch + (long long)s * v.stride_token;
}

__device__ __forceinline__ int fc_seq_len(const KvView& v, int b) {
  // never trust a length beyond what the host validated the block table against
  int n = v.seq_lens ? v.seq_lens[b] : v.max_seq_len;
  return n < v.max_seq_len ? (n < 0 ? 0 : n) : v.max_seq_len;
}

__device__ __forceinline__ float fc_bf16_to_float(unsigned short h) {
  return __uint_as_float(((unsigned)h) << 16);
}
// round-to-nearest-even fp32 -> bf16, NaN preserved (the rounding torch applies on .to(bfloat16))
__device__ __forceinline__ unsigned short fc_float_to_bf16(float f) {
  unsigned u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (unsigned short)((u >> 16) | 0x40);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (unsigned short)(u >> 16);
}
__device__ __forceinline__ float fc_half_to_float(unsigned short h) {
  _Float16 x;
  __builtin_memcpy(&x, &h, 2);
  return (float)x;
}
__device__ __forceinline__ unsigned short fc_float_to_half(float f) {
  _Float16 x = (_Float16)f;  // round-to-nearest-even
  unsigned short h;
  __builtin_memcpy(&h, &x, 2);
  return h;
}

__device__ __forceinline__ float fc_wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ float fc_wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}

// ---- matrix pipe ---------------------------------------------------------------------------------
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

// C[32][32] += A[32][16] * B[16][32] in fp32 (v_mfma_f32_32x32x16).  Operands: lane (row or column l % 32,
// half l / 32) holds the 8 consecutive k = half * 8 .. half * 8 + 7 as 16 bytes.  Result: the lane holds column
// l % 32 and, in register i, row (i / 4) * 8 + half * 4 + i % 4.
#ifdef FC_ABLATE_MFMA16
// Timing-only ablation (results are wrong): the multiply-accumulates of one v_mfma_f32_32x32x16 as two
// v_mfma_f32_16x16x32 on the same operand registers; which two quarters of the accumulator they write alternates with
// the k-step, so that every accumulator register stays the result of matrix instructions.
typedef float fc_f32x4 __attribute__((ext_vector_type(4)));
template <int DTYPE>
__device__ __forceinline__ f32x16 fc_mfma(const uint4& a, const uint4& b, f32x16 c, int ks) {
  const int o = (ks & 1) * 8;
  fc_f32x4 q0 = {c[o], c[o + 1], c[o + 2], c[o + 3]}, q1 = {c[o + 4], c[o + 5], c[o + 6], c[o + 7]};
  q0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), q0, 0, 0, 0);
  q1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, b), __builtin_bit_cast(bf16x8, a), q1, 0, 0, 0);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    c[o + i] = q0[i];
    c[o + 4 + i] = q1[i];
  }
  return c;
}
#endif

template <int DTYPE>
__device__ __forceinline__ f32x16 fc_mfma(const uint4& a, const uint4& b, f32x16 c) {
  if constexpr (DTYPE == FC_BF16)
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c,
                                                   0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0,
                                                  0, 0);
}

// ---- cross-lane sums and maxima without LDS traffic ----------------------------------------------
// One DPP step: every lane reads the lane that CTRL names inside its row of 16 lanes.
template <int CTRL>
__device__ __forceinline__ float fc_dpp(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
// Sum over aligned groups of N consecutive lanes (N a power of two up to 16), in a fixed order; every
// lane of a group ends up with the group's sum.
template <int N>
__device__ __forceinline__ float fc_group_sum(float v) {
  if constexpr (N >= 2) v += fc_dpp<0xB1>(v);    // quad_perm [1,0,3,2]
  if constexpr (N >= 4) v += fc_dpp<0x4E>(v);    // quad_perm [2,3,0,1]
  if constexpr (N >= 8) v += fc_dpp<0x141>(v);   // row_half_mirror
  if constexpr (N >= 16) v += fc_dpp<0x140>(v);  // row_mirror
  return v;
}
template <int N>
__device__ __forceinline__ float fc_group_max(float v) {
  if constexpr (N >= 2) v = fmaxf(v, fc_dpp<0xB1>(v));
  if constexpr (N >= 4) v = fmaxf(v, fc_dpp<0x4E>(v));
  if constexpr (N >= 8) v = fmaxf(v, fc_dpp<0x141>(v));
  if constexpr (N >= 16) v = fmaxf(v, fc_dpp<0x140>(v));
  return v;
}
__device__ __forceinline__ float fc_read_lane(float v, int l) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), l));
}
// Wave-wide, wave-uniform results: DPP inside the four rows, then four lane reads.
__device__ __forceinline__ float fc_wave_sum_uniform(float v) {
  v = fc_group_sum<16>(v);
  return (fc_read_lane(v, 0) + fc_read_lane(v, 16)) + (fc_read_lane(v, 32) + fc_read_lane(v, 48));
}
__device__ __forceinline__ float fc_wave_max_uniform(float v) {
  v = fc_group_max<16>(v);
  return fmaxf(fmaxf(fc_read_lane(v, 0), fc_read_lane(v, 16)), fmaxf(fc_read_lane(v, 32), fc_read_lane(v, 48)));
}

// ---- global memory -> LDS without register staging --------------------------------------------
__device__ __forceinline__ unsigned fc_lds_addr(const void* p) {
  return (unsigned)(size_t)(__attribute__((address_space(3))) const char*)p;
}

// 16 bytes from an absolute LDS address (what fc_lds_addr returns, plus offsets): one ds_read_b128 with the
// address taken as it is, no base added
__device__ __forceinline__ uint4 fc_lds_read128(unsigned addr) {
  typedef unsigned fc_u32x4 __attribute__((ext_vector_type(4)));
  const fc_u32x4 v = *reinterpret_cast<const __attribute__((address_space(3))) fc_u32x4*>((size_t)addr);
  return make_uint4(v.x, v.y, v.z, v.w);
}

// 16 bytes per lane from global memory straight into LDS at lds_base + lane * 16 (lds_base is
// wave-uniform).  The load is counted in vmcnt; the compiler does not know it writes LDS, so
// every consumer sits behind an explicit wait (fc_wait_barrier, fc_wait_vm).
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
__device__ __forceinline__ void fc_load_lds(const char* g, unsigned lds_base) {
  lds_base = __builtin_amdgcn_readfirstlane(lds_base);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_base), "v"(g)
               : "memory", "m0");
}
// same with a wave-uniform 64-bit base and a 32-bit per-lane byte offset
__device__ __forceinline__ void fc_load_lds(const char* g_uniform, unsigned lane_off, unsigned lds_base) {
  lds_base = __builtin_amdgcn_readfirstlane(lds_base);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_base), "v"(lane_off),
               "s"(g_uniform)
               : "memory", "m0");
}
#pragma clang diagnostic pop

// Wait until at most N vector-memory operations of this wave are outstanding and all its LDS
// operations are done, then synchronise the workgroup.
template <int N>
__device__ __forceinline__ void fc_wait_barrier() {
  asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(N) : "memory");
}

// Wait until at most N vector-memory operations of this wave are outstanding (no barrier).
template <int N>
__device__ __forceinline__ void fc_wait_vm() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
// All LDS operations of this wave done, then synchronise the workgroup; outstanding vector-memory
// operations stay in flight.
__device__ __forceinline__ void fc_lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}
#endif  // __HIPCC__
