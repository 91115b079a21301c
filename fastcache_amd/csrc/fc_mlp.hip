// CCM compressor: Linear(cf*128 -> 128) -> ReLU -> Linear(128 -> 128) -> ReLU -> Linear(128 -> 128)
// over rows made of `cf` consecutive tokens of one head, fp16/bf16 storage, fp32 accumulation,
// each Linear's output rounded to the storage dtype.  Reads and writes the caches in place.
//
// Shape of the work: one workgroup of 8 wavefronts (two per SIMD, so that one multiplies while
// the other converts, loads or stores) per group of (sequence, head) columns of one
// layer; a wavefront owns 32 rows of one column per iteration.  The three GEMMs are transposed
// (features along the accumulator registers, one token per lane) and chained through registers:
//   layer 1  H1^T = W1 * X^T   A = W1 rows from LDS, B = X token rows;
//   layer 2  H2^T = W2 * H1^T  B = layer 1's accumulators, converted in place;
//   layer 3  Y^T  = W3 * H2^T  B = layer 2's accumulators.
// A 32x32 accumulator block holds, per lane, 16 values of one token column; taking registers
// 0..7 and 8..15 as two k-steps gives a complete, if permuted, set of 16 k indices across the two
// half-waves, so the next layer's weights are stored in LDS with the same permutation
// ([0-3, 8-11 | 4-7, 12-15] inside every group of 16) and no data moves between lanes.
//
// Token rows enter and leave in the layout memory likes, not the one the MFMA wants: four adjacent
// lanes read (write) 64 contiguous bytes of a row, 16 rows per instruction, and the 32 rows x 64
// bytes of two k-steps (of one 32-feature block of the output) are re-laid through 2 KB of LDS
// private to the wavefront.  With one row per lane instead, every 16-byte access of an instruction
// falls into a cache line of its own and the vector memory pipeline, not HBM, sets the pace.
//
// W2 and W3 (permuted) stay in LDS for the life of the workgroup; W1 streams through a double
// buffer one 128-column chunk (one source token) at a time, shared by the wavefronts; each
// wavefront prefetches the X rows of the next chunk into registers while it multiplies the current one.
// In-place safety: output row j lands on token dst_start + j <= seg_start + cf*j; all rows of an
// iteration are read before the workgroup barrier that precedes its stores, and later iterations
// read tokens no earlier iteration writes.
#include "fc_common.h"

typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

#define ML_WAVES 8                  // wavefronts per workgroup (two per SIMD)
#define ML_ROWS 32                  // rows per wavefront and iteration
#define ML_THREADS (ML_WAVES * 64)
#define ML_ROWB 272                 // LDS bytes per weight row: 128 elements + 16 bytes of padding
#define ML_WBYTES (128 * ML_ROWB)   // one 128 x 128 weight block in LDS
#define ML_TBLTOT 768               // block-table entries cached per workgroup and view, divided among its columns
#define ML_XS 2048                  // per-wavefront LDS bytes for re-laying token rows: 32 rows x 64 bytes
#define ML_LDS (4 * ML_WBYTES + 3 * 128 * 4 + 2 * ML_TBLTOT * 4 + ML_WAVES * ML_XS + ML_WAVES * 4)
// Nothing is scheduled across this point.  Without it the compiler, short of registers, sinks every
// prefetch (weight fragments from LDS, token rows from memory) to just before its use and the
// multiplications wait out the full latency each time.
#define ML_PIN() __builtin_amdgcn_sched_barrier(0)

// two fp32 -> packed storage dtype, round to nearest even
template <int DTYPE>
__device__ __forceinline__ unsigned ml_pack2(float a, float b) {
  f32x2 v = {a, b};
  if constexpr (DTYPE == FC_BF16)
    return __builtin_bit_cast(unsigned, __builtin_convertvector(v, bf16x2));
  else
    return __builtin_bit_cast(unsigned, __builtin_convertvector(v, f16x2));
}

template <int DTYPE>
__device__ __forceinline__ float ml_to_float(unsigned short h) {
  return DTYPE == FC_BF16 ? fc_bf16_to_float(h) : fc_half_to_float(h);
}

// relu + round for 8 consecutive accumulator registers (the bias is already in the accumulator)
// -> one MFMA operand.  ReLU before rounding equals rounding before ReLU.
template <int DTYPE>
__device__ __forceinline__ uint4 ml_act_operand(const f32x16& acc, int i0) {
  unsigned p[4];
#pragma unroll
  for (int e = 0; e < 4; ++e)
    p[e] = ml_pack2<DTYPE>(fmaxf(acc[i0 + 2 * e], 0.f), fmaxf(acc[i0 + 2 * e + 1], 0.f));
  return make_uint4(p[0], p[1], p[2], p[3]);
}

// accumulator block initialised with the bias of its 16 features: register i holds feature
// fb + (i/4)*8 + lhalf*4 + i%4
__device__ __forceinline__ void ml_bias_init(f32x16& acc, const float* __restrict__ bias, int fb, int lhalf) {
#pragma unroll
  for (int i4 = 0; i4 < 4; ++i4) {
    const float4 bv = *reinterpret_cast<const float4*>(bias + fb + i4 * 8 + lhalf * 4);
    acc[i4 * 4 + 0] = bv.x;
    acc[i4 * 4 + 1] = bv.y;
    acc[i4 * 4 + 2] = bv.z;
    acc[i4 * 4 + 3] = bv.w;
  }
}

// orders a wavefront's LDS writes before its following LDS reads of other lanes' data (the hardware executes
// one wavefront's LDS instructions in order; this only keeps the compiler from moving them)
__device__ __forceinline__ void ml_wave_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// SRC_T / DST_T: 0 = dense view (no table), 1 = paged view whose table row fits the LDS cache,
// 2 = paged view read through global memory.
// W1R: all of W1 fits the two LDS chunk buffers (cf <= 2) and is loaded once; otherwise W1 streams
// through them one chunk per stage, which costs a workgroup barrier per chunk.
// RAG: every sequence has its own segment: seg_start_v / seg_len_v / dst_start_v [batch] in device memory; c_rows is
// then the largest row count any sequence can have (it bounds the loops), and a sequence whose segment gives fewer
// than min_rows rows is left to the copy kernel below.
template <int DTYPE, int SRC_T, int DST_T, bool W1R, bool RAG>
__global__ __launch_bounds__(ML_THREADS, ML_WAVES / 4) void mlp_kernel(KvView src, KvView dst, const char* __restrict__ w1,
                                                            const char* __restrict__ b1, const char* __restrict__ w2,
                                                            const char* __restrict__ b2, const char* __restrict__ w3,
                                                            const char* __restrict__ b3, int cf, int seg_start,
                                                            int c_rows, int dst_start, int wpc, int ncols, int ncg,
                                                            const int* __restrict__ seg_start_v,
                                                            const int* __restrict__ seg_len_v,
                                                            const int* __restrict__ dst_start_v, int min_rows) {
  extern __shared__ __align__(16) char lds[];
  char* w1buf = lds;                       // 2 x ML_WBYTES
  char* w2buf = lds + 2 * ML_WBYTES;       // permuted
  char* w3buf = lds + 3 * ML_WBYTES;       // permuted
  float* bias = reinterpret_cast<float*>(lds + 4 * ML_WBYTES);  // [3][128] fp32
  int* tbls = reinterpret_cast<int*>(lds + 4 * ML_WBYTES + 3 * 128 * 4);  // [2 views][columns of the workgroup][tcap]
  char* xsw = lds + 4 * ML_WBYTES + 3 * 128 * 4 + 2 * ML_TBLTOT * 4 + (threadIdx.x >> 6) * ML_XS;
  int* wave_rows = reinterpret_cast<int*>(lds + 4 * ML_WBYTES + 3 * 128 * 4 + 2 * ML_TBLTOT * 4 + ML_WAVES * ML_XS);

  const int l = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lrow = lane & 31, lhalf = lane >> 5;
  const int lq = lane >> 2, lp = lane & 3;   // memory-side layout: row lq (and 16 + lq), 16-byte piece lp of 64 bytes
  const int cols_per_wg = ML_WAVES / wpc;
  const int sub = wave % wpc;
  const int H = src.num_kv_heads;
  const int K1 = cf * 128;
  // the column this wavefront works on; a workgroup takes column groups blockIdx.x, blockIdx.x + gridDim.x, ...
  int col = 0, b = 0, h = 0;
  bool col_ok = false;

  // this column's block-table rows (source and destination), so that no row address waits on a table read;
  // filled by the wavefronts that share the column
  const int tcap = ML_TBLTOT / cols_per_wg;
  int* stbl = tbls + (wave / wpc) * tcap;
  int* dtbl = stbl + ML_TBLTOT;
  // this wavefront's column: first source token, rows, first destination token (the launch's, or the sequence's own)
  int ss = seg_start, cr = c_rows, ds = dst_start;
  auto fill_tables = [&]() {
    // a column without rows still loads (clamped) rows of its first cf tokens: its table covers them
    const int s_last = min(ss + max(cr, 1) * cf, src.max_seq_len) - 1, d_last = ds + cr - 1;
    // also for a wavefront whose column is past the last one (b = 0): its loads are unconditional and need valid addresses
    if (SRC_T == 1)
      for (int i = sub * 64 + lane; i <= (s_last >> src.block_shift); i += 64 * wpc)
        stbl[i] = src.block_tables[(long long)b * src.table_stride + i];
    if (col_ok && DST_T == 1)
      for (int i = sub * 64 + lane; i <= (d_last >> dst.block_shift); i += 64 * wpc)
        dtbl[i] = dst.block_tables[(long long)b * dst.table_stride + i];
  };
  auto src_off = [&](int s) -> long long {
    if (SRC_T == 0) return (long long)b * src.stride_batch + (long long)s * src.stride_token;
    if (SRC_T == 1) {
      const int blk = stbl[s >> src.block_shift];
      return blk < 0 ? -1 : (long long)blk * src.stride_block + (long long)(s & (src.block_size - 1)) * src.stride_token;
    }
    return fc_token_offset(src, b, s);
  };
  auto dst_off = [&](int s) -> long long {
    if (DST_T == 0) return (long long)b * dst.stride_batch + (long long)s * dst.stride_token;
    if (DST_T == 1) {
      const int blk = dtbl[s >> dst.block_shift];
      return blk < 0 ? -1 : (long long)blk * dst.stride_block + (long long)(s & (dst.block_size - 1)) * dst.stride_token;
    }
    return fc_token_offset(dst, b, s);
  };

  // ---- resident weights: W2, W3 with the k permutation, biases as fp32 ------------------------------
  {
    const char* w2l = w2 + (long long)l * 128 * 128 * 2;
    const char* w3l = w3 + (long long)l * 128 * 128 * 2;
    // 8-byte pieces: piece p of a row holds k = 4p .. 4p+3; inside each group of 4 pieces the order
    // becomes [0, 2, 1, 3]
    for (int i = tid; i < 128 * 32; i += ML_THREADS) {
      const int n = i >> 5, p = i & 31;
      const int q = p & 3;
      const int pp = (p & ~3) | ((q == 1) ? 2 : (q == 2) ? 1 : q);
      *reinterpret_cast<uint2*>(w2buf + n * ML_ROWB + pp * 8) = *reinterpret_cast<const uint2*>(w2l + (n * 128 + p * 4) * 2);
      *reinterpret_cast<uint2*>(w3buf + n * ML_ROWB + pp * 8) = *reinterpret_cast<const uint2*>(w3l + (n * 128 + p * 4) * 2);
    }
    for (int i = tid; i < 384; i += ML_THREADS) {
      const int which = i >> 7, n = i & 127;
      const char* bp = which == 0 ? b1 : which == 1 ? b2 : b3;
      bias[i] = ml_to_float<DTYPE>(*reinterpret_cast<const unsigned short*>(bp + ((long long)l * 128 + n) * 2));
    }
  }

  // W1 chunk kc covers columns [kc*128, kc*128+128) of W1[l]: 2048 pieces of 16 bytes
  constexpr int WCH = 2048 / ML_THREADS;
  const char* w1l = w1 + (long long)l * 128 * K1 * 2;
  u32x4 wpre[WCH];
  auto w1_load = [&](int kc) {
#pragma unroll
    for (int u = 0; u < WCH; ++u) {
      const int ch = tid + u * ML_THREADS;  // row n = ch / 16, part = ch % 16
      wpre[u] = *reinterpret_cast<const u32x4*>(w1l + ((long long)(ch >> 4) * K1 + kc * 128) * 2 + (ch & 15) * 16);
    }
  };
  auto w1_store = [&](int buf) {
#pragma unroll
    for (int u = 0; u < WCH; ++u) {
      const int ch = tid + u * ML_THREADS;
      *reinterpret_cast<u32x4*>(w1buf + buf * ML_WBYTES + (ch >> 4) * ML_ROWB + (ch & 15) * 16) = wpre[u];
    }
  };

  const int rows_per_iter = ML_ROWS * wpc;
  int n_iter = (c_rows + rows_per_iter - 1) / rows_per_iter;
  int q_total = n_iter * cf;      // W1 chunk q = (iteration q / cf, token kc = q % cf) sits in buffer q & 1
  const char* sbase = nullptr;   // this lane's piece of token 0 of the column's head, per column group
  char* dbase = nullptr;

  // X rows of chunk q: xf[2*c4 + rh] holds bytes [64*c4 + 16*lp, +16) of the token row of output row 16*rh + lq
  auto x_load = [&](uint4 (&xf)[8], int q) {
    const int it = q / cf, kc = q - it * cf;
    const int row0 = it * rows_per_iter + sub * ML_ROWS;
    // Every lane always loads (no branch around the loads, so that the compiler keeps exact counts of
    // the loads in flight and the prefetch really overlaps the multiplications): rows past the end, a
    // column past the last one (b = h = 0) and unallocated pages read some valid row instead; what is
    // computed from them is never stored.
#pragma unroll
    for (int rh = 0; rh < 2; ++rh) {
      int r = min(row0 + rh * 16 + lq, cr - 1);
      int tok = ss + cf * r + kc;
      if constexpr (RAG) {   // a column with no rows, or fewer than the launch's bound, reads some valid token
        r = max(r, 0);
        tok = min(ss + cf * r + kc, src.max_seq_len - 1);
      }
      long long off = src_off(tok);
      off = off < 0 ? 0 : off;
#pragma unroll
      for (int c4 = 0; c4 < 4; ++c4) xf[c4 * 2 + rh] = *reinterpret_cast<const uint4*>(sbase + off * 2 + c4 * 64);
    }
  };
  // Re-laying through this wavefront's 2 KB of LDS: rows of 64 bytes, the four 16-byte pieces of a row XOR-ed
  // with a 2-bit function of the row number chosen so that the operand-side accesses (consecutive rows, same
  // piece) touch every bank once whether 8 rows share a 128-byte bank window or 16 rows a 256-byte one:
  // rows r, r+2, r+4, r+6 and rows r, r+4, r+8, r+12 all get different pieces.
  auto piece_swz = [](int r) { return (unsigned)((((r >> 1) ^ (r >> 3)) & 1) | (((r >> 2) & 1) << 1)); };
  const unsigned mem_at = (unsigned)lq * 64 + ((lp ^ piece_swz(lq)) << 4);   // row lq; row 16 + lq is 1024 further
  const unsigned swz = piece_swz(lrow);
  const unsigned op_at0 = (unsigned)lrow * 64 + (((0 + lhalf) ^ swz) << 4);    // k-step 0 of the pair: pieces 0, 1
  const unsigned op_at1 = (unsigned)lrow * 64 + (((2 + lhalf) ^ swz) << 4);    // k-step 1: pieces 2, 3
  auto relay_put = [&](uint4 lo_rows, uint4 hi_rows) {
    *reinterpret_cast<uint4*>(xsw + mem_at) = lo_rows;
    *reinterpret_cast<uint4*>(xsw + mem_at + 1024) = hi_rows;
    ml_wave_sync();
  };
  auto relay_get = [&](int e) { return *reinterpret_cast<const uint4*>(xsw + (e ? op_at1 : op_at0)); };

  f32x16 acc[4];

  // One pipeline stage: chunk q of layer 1 from `xcur` while chunk q+1's rows load into `xnext`;
  // after the last chunk of an iteration, layers 2 and 3 and the stores.
  auto stage = [&](uint4 (&xcur)[8], uint4 (&xnext)[8], int q) {
    const int it = q / cf, kc = q - it * cf;
    // The prefetches are unconditional (straight-line code keeps the staging registers out of
    // scratch memory): past the last chunk the X rows are clamped to valid ones, and the
    // extra W1 chunk lands in the buffer nobody reads again.
    x_load(xnext, q + 1);
    ML_PIN();   // the prefetch stays ahead of this stage's multiplications
    if (!W1R) {
      __syncthreads();  // chunk q is in w1buf[q & 1]; every wavefront is done with chunk q - 1
      w1_load((kc + 1 < cf) ? kc + 1 : 0);
    }
    {
      const char* wa = w1buf + (W1R ? kc : (q & 1)) * ML_WBYTES + lrow * ML_ROWB + lhalf * 16;
      uint4 af[2][4];      // weight fragments of k-step ks+1 are read while k-step ks multiplies
      uint4 bop[2][2];     // token operands of two k-steps (64 bytes of every row), re-laid one pair ahead
      relay_put(xcur[0], xcur[1]);
      bop[0][0] = relay_get(0);
      bop[0][1] = relay_get(1);
#pragma unroll
      for (int mb = 0; mb < 4; ++mb) af[0][mb] = *reinterpret_cast<const uint4*>(wa + mb * 32 * ML_ROWB);
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) {
        if ((ks & 1) == 0 && ks + 2 < 8) {
          relay_put(xcur[ks + 2], xcur[ks + 3]);
          bop[((ks >> 1) + 1) & 1][0] = relay_get(0);
          bop[((ks >> 1) + 1) & 1][1] = relay_get(1);
        }
        if (ks + 1 < 8) {
#pragma unroll
          for (int mb = 0; mb < 4; ++mb)
            af[(ks + 1) & 1][mb] = *reinterpret_cast<const uint4*>(wa + mb * 32 * ML_ROWB + (ks + 1) * 32);
        }
        ML_PIN();   // the reads of the next k-step are issued before this k-step's multiplications
#pragma unroll
        for (int mb = 0; mb < 4; ++mb) acc[mb] = fc_mfma<DTYPE>(af[ks & 1][mb], bop[(ks >> 1) & 1][ks & 1], acc[mb]);
        ML_PIN();
      }
    }
    if (!W1R) w1_store((q + 1) & 1);
    if (kc != cf - 1) return;

    // ---- layers 2 and 3: H^T = W * (previous H)^T, B operand taken from the previous layer's accumulators ----
    uint4 hf[8];
#pragma unroll
    for (int layer = 1; layer < 3; ++layer) {
#pragma unroll
      for (int mb = 0; mb < 4; ++mb) {
        hf[2 * mb] = ml_act_operand<DTYPE>(acc[mb], 0);
        hf[2 * mb + 1] = ml_act_operand<DTYPE>(acc[mb], 8);
        ml_bias_init(acc[mb], bias + layer * 128, mb * 32, lhalf);
      }
      const char* wa = (layer == 1 ? w2buf : w3buf) + lrow * ML_ROWB + lhalf * 16;
      uint4 af[2][4];
#pragma unroll
      for (int mb = 0; mb < 4; ++mb) af[0][mb] = *reinterpret_cast<const uint4*>(wa + mb * 32 * ML_ROWB);
#pragma unroll
      for (int g = 0; g < 8; ++g) {
        if (g + 1 < 8) {
#pragma unroll
          for (int mb = 0; mb < 4; ++mb)
            af[(g + 1) & 1][mb] = *reinterpret_cast<const uint4*>(wa + mb * 32 * ML_ROWB + (g + 1) * 32);
        }
        ML_PIN();
#pragma unroll
        for (int mb = 0; mb < 4; ++mb) acc[mb] = fc_mfma<DTYPE>(af[g & 1][mb], hf[g], acc[mb]);
        ML_PIN();
      }
    }
    // every wavefront of the column has consumed this iteration's source rows: stores may alias them
    // (a wavefront that owns its column alone is ordered by its own data dependences)
    if (wpc > 1) __syncthreads();
    {
      // The lane owns output row lrow and, per 32-feature block, features (i/4)*8 + lhalf*4 + i%4: four 8-byte
      // pieces go to the wavefront's LDS rows (64 bytes = one feature block of a row); read back in the
      // memory-side layout, 16 rows x 64 bytes leave per store instruction.
      const int row0 = it * rows_per_iter + sub * ML_ROWS;
      char* rowp[2];
#pragma unroll
      for (int rh = 0; rh < 2; ++rh) {
        const int r = row0 + rh * 16 + lq;
        long long off = -1;
        if (col_ok && r < cr) off = dst_off(ds + r);
        rowp[rh] = off >= 0 ? dbase + off * 2 : nullptr;
      }
      // (a half-wave writes one 8-byte half per row, so rows that share a piece position in a bank window keep
      // their halves swapped: bit 3 xor bit 4 of the row number)
      const unsigned y_at = (unsigned)lrow * 64 + (((lhalf ^ (lrow >> 3) ^ (lrow >> 4)) & 1) << 3);
      const bool swap0 = (lq >> 3) & 1;     // row lq has its halves swapped; row 16 + lq the opposite
#pragma unroll
      for (int mb = 0; mb < 4; ++mb) {
#pragma unroll
        for (int i4 = 0; i4 < 4; ++i4) {
          uint2 w;
          w.x = ml_pack2<DTYPE>(acc[mb][i4 * 4 + 0], acc[mb][i4 * 4 + 1]);
          w.y = ml_pack2<DTYPE>(acc[mb][i4 * 4 + 2], acc[mb][i4 * 4 + 3]);
          *reinterpret_cast<uint2*>(xsw + y_at + ((i4 ^ swz) << 4)) = w;
        }
        ml_wave_sync();
        const uint4 y0 = *reinterpret_cast<const uint4*>(xsw + mem_at);
        const uint4 y1 = *reinterpret_cast<const uint4*>(xsw + mem_at + 1024);
        if (rowp[0])
          *reinterpret_cast<uint4*>(rowp[0] + mb * 64) = swap0 ? make_uint4(y0.z, y0.w, y0.x, y0.y) : y0;
        if (rowp[1])
          *reinterpret_cast<uint4*>(rowp[1] + mb * 64) = swap0 ? y1 : make_uint4(y1.z, y1.w, y1.x, y1.y);
      }
    }
#pragma unroll
    for (int mb = 0; mb < 4; ++mb) ml_bias_init(acc[mb], bias, mb * 32, lhalf);
  };

  uint4 xa[8], xb[8];
  if (W1R) {
    w1_load(0);
    w1_store(0);
    if (cf > 1) {
      w1_load(1);
      w1_store(1);
    }
  }
  for (int cg = blockIdx.x; cg < ncg; cg += gridDim.x) {
    if (cg != (int)blockIdx.x) __syncthreads();   // every wavefront is done with the previous group's tables and W1 buffers
    col = cg * cols_per_wg + wave / wpc;
    col_ok = col < ncols;
    b = col_ok ? col / H : 0;
    h = col_ok ? col - (col / H) * H : 0;
    sbase = src.base + ((long long)l * src.stride_layer + (long long)h * src.stride_head) * 2 + lp * 16;
    dbase = dst.base + ((long long)l * dst.stride_layer + (long long)h * dst.stride_head) * 2 + lp * 16;
    if constexpr (RAG) {
      // The sequence's own segment.  Numbers from device memory are cut to what the host validated: the views'
      // max_seq_len (which their block tables cover) and the launch's row bound.
      ss = min(max(__builtin_amdgcn_readfirstlane(seg_start_v[b]), 0), src.max_seq_len);
      const int sl = min(max(__builtin_amdgcn_readfirstlane(seg_len_v[b]), 0), src.max_seq_len - ss);
      ds = min(max(__builtin_amdgcn_readfirstlane(dst_start_v[b]), 0), dst.max_seq_len);
      cr = sl / cf;
      if (cr < min_rows || !col_ok) cr = 0;
      cr = min(min(cr, c_rows), dst.max_seq_len - ds);
      if (lane == 0) wave_rows[wave] = cr;
    }
    fill_tables();
    if (!W1R) {
      w1_load(0);
      w1_store(0);
    }
    __syncthreads();   // block tables, biases and the first weights are in LDS
    if constexpr (RAG) {   // the workgroup walks as many iterations as its longest column needs
      int most = 0;
#pragma unroll
      for (int w = 0; w < ML_WAVES; ++w) most = max(most, wave_rows[w]);
      n_iter = (most + rows_per_iter - 1) / rows_per_iter;
      q_total = n_iter * cf;
    }
#pragma unroll
    for (int mb = 0; mb < 4; ++mb) ml_bias_init(acc[mb], bias, mb * 32, lhalf);
    x_load(xa, 0);
    for (int q = 0; q < q_total; q += 2) {
      stage(xa, xb, q);
      if (q + 1 < q_total) stage(xb, xa, q + 1);
    }
    // the streaming variant is launched with one column group per workgroup (its groups are long, and the
    // loop would cost it registers it does not have)
    if (!W1R) break;
  }
}

// compute units of the current device (0 if the query fails)
static int ml_compute_units() {
  static int cus[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
  if (cus[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0) cus[dev] = n;
  }
  return cus[dev];
}

// What the MLP leaves of a ragged segment: the seg_len % cf remainder tokens, or the whole segment of a sequence
// too short to compress, copied to their place behind the compressed rows.  One workgroup per (head, sequence,
// layer); 16 tokens per pass, all loaded before any is stored (destination token <= source token, ascending).
__global__ __launch_bounds__(256) void mlp_tail_copy_kernel(KvView src, KvView dst, int cf, int min_rows, int c_max,
                                                            const int* __restrict__ seg_start_v,
                                                            const int* __restrict__ seg_len_v,
                                                            const int* __restrict__ dst_start_v, int same_place) {
  const int h = blockIdx.x, b = blockIdx.y, l = blockIdx.z;
  const int ss = min(max(seg_start_v[b], 0), src.max_seq_len);
  const int sl = min(max(seg_len_v[b], 0), src.max_seq_len - ss);
  const int ds = min(max(dst_start_v[b], 0), dst.max_seq_len);
  int c = sl / cf;
  if (c < min_rows) c = 0;
  c = min(min(c, c_max), dst.max_seq_len - ds);
  const int s0 = ss + c * cf, d0 = ds + c;
  const int cnt = min(sl - c * cf, dst.max_seq_len - d0);
  if (cnt <= 0 || (same_place && s0 == d0)) return;
  const int sub = threadIdx.x & 15, tr = threadIdx.x >> 4;
  const char* sb = src.base + ((long long)l * src.stride_layer + (long long)h * src.stride_head) * 2 + sub * 16;
  char* db = dst.base + ((long long)l * dst.stride_layer + (long long)h * dst.stride_head) * 2 + sub * 16;
  for (int i0 = 0; i0 < cnt; i0 += 16) {
    const int i = i0 + tr;
    uint4 row = make_uint4(0, 0, 0, 0);
    long long so = -1, dof = -1;
    if (i < cnt) {
      so = fc_token_offset(src, b, s0 + i);
      dof = fc_token_offset(dst, b, d0 + i);
    }
    if (so >= 0) row = *reinterpret_cast<const uint4*>(sb + so * 2);
    __syncthreads();
    if (so >= 0 && dof >= 0) *reinterpret_cast<uint4*>(db + dof * 2) = row;
  }
}

extern "C" int fc_copy_tokens(const fc_kv_view* src, const fc_kv_view* dst, int32_t seg_start, int32_t count,
                              int32_t dst_start, void* stream);

static int ml_check(const char* who, const fc_kv_view* src, const fc_kv_view* dst, const fc_mlp_weights* w, int cf) {
  int rc;
  if ((rc = fc_check_view(src, who)) || (rc = fc_check_view(dst, who))) return rc;
  FC_REQUIRE(src->dtype == dst->dtype && src->num_layers == dst->num_layers && src->batch == dst->batch &&
                 src->num_kv_heads == dst->num_kv_heads,
             FC_EINVAL, "%s: source and destination views disagree", who);
  FC_REQUIRE(src->dtype == FC_F16 || src->dtype == FC_BF16, FC_EUNSUPPORTED, "%s: fp16/bf16 caches only", who);
  FC_REQUIRE(w && w->w1 && w->b1 && w->w2 && w->b2 && w->w3 && w->b3, FC_EINVAL, "%s: null weights", who);
  FC_REQUIRE(cf >= 1 && cf <= 64, FC_EINVAL, "%s: compression factor %d out of range", who, cf);
  return FC_OK;
}

// The MLP launch for c > 0 rows per column: c rows for every sequence from (seg_start, dst_start), or, with the
// three arrays, every sequence's own segment with at most c rows.
static int ml_launch(const char* who, const fc_kv_view* src, const fc_kv_view* dst, const fc_mlp_weights* w, int cf,
                     int seg_start, int c, int dst_start, const int32_t* seg_start_v, const int32_t* seg_len_v,
                     const int32_t* dst_start_v, int min_rows, hipStream_t st) {
  const bool rag = seg_len_v != nullptr;
  const int ncols = src->batch * src->num_kv_heads;
  int wpc = 1;
  while (wpc < ML_WAVES && (int64_t)ncols * wpc / ML_WAVES * src->num_layers < 1024 && ML_ROWS * wpc * 2 <= c) wpc *= 2;
  const int cols_per_wg = ML_WAVES / wpc;
  // One workgroup occupies a compute unit (its LDS), and loading the weights costs it a few microseconds.
  // When a column group is short work, let each workgroup walk several groups of its layer; pick the number
  // per workgroup that minimises rounds * (groups * time per group + start-up) in a coarse model.
  const int ncg = (ncols + cols_per_wg - 1) / cols_per_wg;
  int gx = ncg;
  {
    const int ncu = ml_compute_units();
    const int n_iter = (c + ML_ROWS * wpc - 1) / (ML_ROWS * wpc);
    const double t_group = 1.5 * n_iter * (cf + 2), t_start = 4.0;   // microseconds, roughly
    double best = -1.0;
    for (int per = 1; cf <= 2 && ncu > 0 && per <= ncg && per <= 64; ++per) {
      const int g = (ncg + per - 1) / per;
      const long long rounds = ((long long)g * src->num_layers + ncu - 1) / ncu;
      const double cost = (double)rounds * (((ncg + g - 1) / g) * t_group + t_start);
      if (best < 0 || cost < best) {
        best = cost;
        gx = g;
      }
    }
  }
  dim3 grid(gx, src->num_layers);
  const size_t lds = ML_LDS;
  KvView s = fc_make_view(src), d = fc_make_view(dst);
  auto table_mode = [&](const KvView& v, int last_token) {
    if (!v.block_tables) return 0;
    return (v.block_shift >= 0 && (last_token >> v.block_shift) < ML_TBLTOT / cols_per_wg) ? 1 : 2;
  };
  // ragged segments may end anywhere inside the views
  const int sm = table_mode(s, rag ? src->max_seq_len - 1 : seg_start + c * cf - 1);
  const int dm = table_mode(d, rag ? dst->max_seq_len - 1 : dst_start + c - 1);
  // dense/dense, LDS-cached tables, or the general path through global tables (which also serves dense views)
  int mode = (sm == 0 && dm == 0) ? 0 : (sm == 1 && dm == 1) ? 1 : (sm == 0 && dm == 1) ? 2 : (sm == 1 && dm == 0) ? 3 : 4;
  if (rag && mode != 1) mode = 4;
#define ML_LAUNCH(DT, ST, DTT, WR, RG)                                                                                 \
  do {                                                                                                             \
    FC_ALLOW_LDS((mlp_kernel<DT, ST, DTT, WR, RG>), (int)lds);                                                    \
    hipLaunchKernelGGL((mlp_kernel<DT, ST, DTT, WR, RG>), grid, dim3(ML_THREADS), lds, st, s, d, (const char*)w->w1, \
                       (const char*)w->b1, (const char*)w->w2, (const char*)w->b2, (const char*)w->w3,             \
                       (const char*)w->b3, cf, seg_start, c, dst_start, wpc, ncols, ncg, seg_start_v, seg_len_v,   \
                       dst_start_v, min_rows);                                                                     \
  } while (0)
#define ML_DISPATCH(DT, WR)                                                         \
  if (rag) {                                                                        \
    if (mode == 1) ML_LAUNCH(DT, 1, 1, WR, true); else ML_LAUNCH(DT, 2, 2, WR, true); \
  } else switch (mode) {                                                            \
    case 0: ML_LAUNCH(DT, 0, 0, WR, false); break;                                  \
    case 1: ML_LAUNCH(DT, 1, 1, WR, false); break;                                  \
    case 2: ML_LAUNCH(DT, 0, 1, WR, false); break;                                  \
    case 3: ML_LAUNCH(DT, 1, 0, WR, false); break;                                  \
    default: ML_LAUNCH(DT, 2, 2, WR, false); break;                                 \
  }
  if (src->dtype == FC_BF16) {
    if (cf <= 2) { ML_DISPATCH(FC_BF16, true) } else { ML_DISPATCH(FC_BF16, false) }
  } else {
    if (cf <= 2) { ML_DISPATCH(FC_F16, true) } else { ML_DISPATCH(FC_F16, false) }
  }
#undef ML_DISPATCH
#undef ML_LAUNCH
  FC_CHECK_LAUNCH(who);
  return FC_OK;
}

extern "C" int fc_ccm_mlp(const fc_kv_view* src, const fc_kv_view* dst, const fc_mlp_weights* w, int32_t cf,
                          int32_t seg_start, int32_t seg_len, int32_t dst_start, void* stream) {
  const char* who = "fc_ccm_mlp";
  int rc = ml_check(who, src, dst, w, cf);
  if (rc) return rc;
  FC_REQUIRE(seg_start >= 0 && seg_len >= 0 && dst_start >= 0, FC_EINVAL, "%s: negative range", who);
  FC_REQUIRE((int64_t)seg_start + seg_len <= src->max_seq_len, FC_EINVAL,
             "%s: segment [%d, %d) exceeds the source view's max_seq_len %d", who, seg_start, seg_start + seg_len,
             src->max_seq_len);
  const int c = seg_len / cf;
  const int rem = seg_len - c * cf;
  FC_REQUIRE((int64_t)dst_start + c + rem <= dst->max_seq_len, FC_EINVAL,
             "%s: output [%d, %d) exceeds the destination view's max_seq_len %d", who, dst_start,
             dst_start + c + rem, dst->max_seq_len);
  if (c > 0 && (rc = ml_launch(who, src, dst, w, cf, seg_start, c, dst_start, nullptr, nullptr, nullptr, 0,
                               (hipStream_t)stream)))
    return rc;
  if (rem > 0) return fc_copy_tokens(src, dst, seg_start + c * cf, rem, dst_start + c, stream);
  return FC_OK;
}

extern "C" int fc_ccm_mlp_ragged(const fc_kv_view* src, const fc_kv_view* dst, const fc_mlp_weights* w, int32_t cf,
                                 const int32_t* seg_start, const int32_t* seg_len, const int32_t* dst_start,
                                 int32_t max_seg_len, int32_t min_rows, void* stream) {
  const char* who = "fc_ccm_mlp_ragged";
  int rc = ml_check(who, src, dst, w, cf);
  if (rc) return rc;
  FC_REQUIRE(seg_start && seg_len && dst_start, FC_EINVAL, "%s: null segment arrays", who);
  FC_REQUIRE(max_seg_len >= 0 && max_seg_len <= src->max_seq_len, FC_EINVAL,
             "%s: max_seg_len %d outside [0, max_seq_len %d]", who, max_seg_len, src->max_seq_len);
  FC_REQUIRE(min_rows >= 0, FC_EINVAL, "%s: negative min_rows", who);
  FC_REQUIRE(src->num_kv_heads <= 65535, FC_EUNSUPPORTED, "%s: too many heads", who);
  if (max_seg_len == 0) return FC_OK;
  hipStream_t st = (hipStream_t)stream;
  const int c = max_seg_len / cf;
  if (c > 0 && c >= min_rows &&
      (rc = ml_launch(who, src, dst, w, cf, 0, c, 0, seg_start, seg_len, dst_start, min_rows, st)))
    return rc;
  // remainders and pass-through segments; nothing to move when a pass-through segment already lies at its place
  const int same = src->base == dst->base && src->block_tables == dst->block_tables &&
                   src->stride_layer == dst->stride_layer && src->stride_batch == dst->stride_batch;
  hipLaunchKernelGGL(mlp_tail_copy_kernel, dim3(src->num_kv_heads, src->batch, src->num_layers), dim3(256), 0, st,
                     fc_make_view(src), fc_make_view(dst), cf, min_rows, c, seg_start, seg_len, dst_start, same);
  FC_CHECK_LAUNCH(who);
  return FC_OK;
}
