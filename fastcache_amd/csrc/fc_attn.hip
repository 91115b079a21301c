// Decode-side kernels over the paged cache: append one K/V row per sequence, advance the lengths,
// and single-query paged attention (split over chunks of 256 to 1024 tokens, then merged).
//
// Attention is HBM-bound (one pass over K and V, ~1 FLOP per byte per query head), so the kernel is
// organised around keeping loads in flight.  A workgroup owns one (sequence, kv head, chunk of
// 256..1024 tokens, a multiple of 32 the host picks per launch) and serves all query heads of the group from the same K/V bytes; each of its four
// wavefronts streams two 32-token K tiles and then the matching V tiles from global memory straight
// into a private two-stage LDS ring (global_load_lds, rows XOR-swizzled), 16 KB per wavefront in
// flight, no workgroup barrier between a load and its use.
//   phase 1  logits: one v_mfma_f32_32x32x16 block per tile, query heads as (zero-padded) rows;
//   phase 2  chunk softmax statistics (max, sum of exp2), one wavefront per query head;
//   phase 3  sum of p * V rows from LDS: on the VALU, 8 output dims per lane, 16 partial sums folded through
//            LDS; for 8 heads per workgroup on the matrix pipe with V read transposed from LDS;
// Each chunk writes (max, sum, unnormalised output) to the workspace; a second kernel merges the
// chunks of a sequence.  Grid sizes depend only on the view's max_seq_len, never on the lengths on
// the device, so both launches can be replayed from a graph while the lengths grow.
#include "fc_common.h"
#include <atomic>
#include <stdlib.h>

#define DA_THREADS 256
#define DA_CHUNK 256               // smallest chunk (tokens per workgroup); it sizes the workspace
#define DA_CHUNK_MAX 1024          // largest: the host picks a multiple of 32 in between from the launch's shape
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


#define DA_PV_MFMA_MIN 8               // heads per workgroup from which p * V runs on the matrix pipe (measured: no gain below)
#define DA_TILE 32                     // keys per tile: one MFMA block, 8 KB of K or V rows
// The chunk's block-table entries are prefetched one per lane of a wavefront: the largest chunk in the smallest
// page the fast path takes (32 tokens, block_shift >= 5), starting anywhere in a page, must span at most 64 entries.
static_assert(DA_CHUNK_MAX / DA_TILE + 1 <= 64, "a chunk's block-table entries must fit one per lane");
static_assert(DA_CHUNK % DA_TILE == 0 && DA_CHUNK_MAX % 64 == 0, "chunk bounds: whole tiles, whole statistics registers");
#define DA_TILEB (DA_TILE * 256)
#define DA_RING (4 * 2 * DA_TILEB)     // four wavefronts, two stages each

template <int GT>
struct DaCfg {
  // ring | logits, then probabilities [GT][chunk]: fp32, or with eight heads (p * V on the matrix pipe) each
  // probability as two 16-bit halves hi + lo in the cache dtype
  static constexpr bool PV_MFMA = GT >= DA_PV_MFMA_MIN;
  static constexpr int lds(int chunk) { return DA_RING + GT * chunk * 4; }
};

// GT = query heads served per workgroup (a tile of the group, at most 8).
// FAST = a 32-token tile never straddles two pages (dense view, or pages of 32*2^n tokens), so a tile
// load is a wave-uniform base plus a per-lane offset.
//
// Wavefront w owns the key tiles w and w+4 of the chunk (32 tokens each) and streams them through
// its private two-stage ring in LDS with global_load_lds: K tile a, K tile b, then V tile a and
// V tile b into the same stages as soon as the logits of the K tile in them are done, so 16 KB per
// wavefront are in flight for most of the kernel and no load waits behind a workgroup barrier.
// Logits are one v_mfma_f32_32x32x16 block per tile with the query heads as rows (padded with zero
// rows to 32): whatever the group size, K is read from LDS once.
template <int DTYPE, int GT, bool FAST>
__global__ __launch_bounds__(DA_THREADS, 2) void decode_attn_kernel(KvView kc, KvView vc, int layer,
                                                                    const char* __restrict__ q, int Hq,
                                                                    const int* __restrict__ lens, float c,
                                                                    float* __restrict__ part_o,
                                                                    float* __restrict__ part_ml, int max_splits,
                                                                    int chunk) {
  extern __shared__ __align__(16) char smem[];
  float* sc = reinterpret_cast<float*>(smem + DA_RING);          // [GT][chunk]
  unsigned* p2 = reinterpret_cast<unsigned*>(smem + DA_RING);    // the same seen as (hi, lo) pairs
  constexpr bool PV_MFMA = DaCfg<GT>::PV_MFMA;
  float(*red)[GT][FC_HEAD_DIM] = reinterpret_cast<float(*)[GT][FC_HEAD_DIM]>(smem);  // [16] partial outputs, reuses the ring
  static_assert(16 * GT * FC_HEAD_DIM * 4 <= DA_RING, "partial outputs must fit in the ring");

  // Workgroups go to the eight XCDs round-robin in launch order (blockIdx.x fastest).  With the chunk
  // index taken straight from blockIdx.x and a multiple of eight chunks per sequence, each XCD would
  // serve one chunk position of every sequence, and the late positions are mostly empty; rotating the
  // chunk index by the head and sequence spreads the live chunks over all XCDs.
  const int b = blockIdx.z;
  const int split = (int)((blockIdx.x + blockIdx.y + blockIdx.z) % gridDim.x);
  const int Hkv = kc.num_kv_heads;
  const int G = Hq / Hkv;
  const int gtiles = (G + GT - 1) / GT;
  const int h = blockIdx.y / gtiles, g0 = (blockIdx.y - h * gtiles) * GT;
  const int tid = threadIdx.x, lane = tid & 63;
  const int t0 = split * chunk;
  // The chunk's block-table entries, one per lane (a chunk of at most 1024 tokens in pages of at least 32 spans at
  // most 33), fetched before anything waits for the sequence length: a tile's address then costs a lane read instead
  // of a table load that the tile's own loads would have to wait for.
  int ktbl = 0, vtbl = 0;
  if constexpr (FAST) {
    if (kc.block_tables) {
      const int e = min((t0 >> kc.block_shift) + lane, kc.table_stride - 1);
      ktbl = kc.block_tables[(long long)b * kc.table_stride + e];
    }
    if (vc.block_tables) {
      const int e = min((t0 >> vc.block_shift) + lane, vc.table_stride - 1);
      vtbl = vc.block_tables[(long long)b * vc.table_stride + e];
    }
  }
  int len = __builtin_amdgcn_readfirstlane(lens[b]);
  len = min(len, kc.max_seq_len);
  if (t0 >= len) return;
  const int ntok = min(chunk, len - t0);

  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lrow = lane & 31, lhalf = lane >> 5;
  const int sub = lane & 15, rg = lane >> 4;   // V rows: 16 lanes per row, 4 rows per pass

  // query heads as MFMA A-operand rows; rows past the group tile are zero
  uint4 qf[8];
  {
    const bool ok = lrow < GT && g0 + lrow < G;
    const char* qp = q + (((long long)b * Hq + (h * G + g0 + (ok ? lrow : 0))) * FC_HEAD_DIM + lhalf * 8) * 2;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) qf[ks] = ok ? *reinterpret_cast<const uint4*>(qp + ks * 32) : make_uint4(0, 0, 0, 0);
  }

  const char* kbase = kc.base + ((long long)layer * kc.stride_layer + (long long)h * kc.stride_head) * 2;
  const char* vbase = vc.base + ((long long)layer * vc.stride_layer + (long long)h * vc.stride_head) * 2;
  const unsigned ring_lds = __builtin_amdgcn_readfirstlane(fc_lds_addr(smem)) + wave * (2 * DA_TILEB);
  char* ring = smem + wave * (2 * DA_TILEB);

  // Tile `tile` of the chunk into this wavefront's stage: eight wave-loads of four rows.  Lane i
  // writes LDS chunk i of the 64 chunks of those rows and fetches the global chunk (i & 15) ^ (row & 15)
  // of row i / 16 (XOR swizzle, so that the operand reads of 32 rows at the same chunk fall on
  // distinct banks).  Rows past the sequence end re-read its last row; their logits are masked.
  auto issue = [&](const KvView& v, const char* base, int tile, int stage, int tbl_reg) {
    const int s0 = t0 + tile * DA_TILE;
    const unsigned dst = ring_lds + stage * DA_TILEB;
    const int rmax = len - 1 - s0;
    if constexpr (FAST) {
      long long tb;
      if (v.block_tables) {
        const int blk = max(__builtin_amdgcn_readlane(tbl_reg, (s0 >> v.block_shift) - (t0 >> v.block_shift)), 0);
        tb = (long long)blk * v.stride_block + (long long)(s0 & (v.block_size - 1)) * v.stride_token;
      } else {
        tb = (long long)b * v.stride_batch + (long long)s0 * v.stride_token;
      }
      const char* g = base + tb * 2;
      const unsigned tok_bytes = (unsigned)v.stride_token * 2;
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int r = 4 * u + rg;
        const unsigned lo = (unsigned)min(r, rmax) * tok_bytes + ((sub ^ (r & 15)) << 4);
        fc_load_lds(g, lo, dst + u * 1024);
      }
    } else {
      long long off[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int r = 4 * u + rg;
        off[u] = fc_token_offset(v, b, s0 + min(r, rmax));
        if (off[u] < 0) off[u] = 0;
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int r = 4 * u + rg;
        fc_load_lds(base + off[u] * 2 + ((sub ^ (r & 15)) << 4), dst + u * 1024);
      }
    }
  };

  // This wavefront's tiles are wave, wave + 4, wave + 8, ...: nj of them hold tokens.  Their K tiles and then
  // their V tiles form one stream of 2 * nj items; item i goes to stage i & 1 and is issued as soon as item
  // i - 2 has been consumed, so two items (16 KB) are in flight for most of the kernel.
  const int live_tiles = (ntok + DA_TILE - 1) / DA_TILE;
  const int nj = wave < live_tiles ? (live_tiles - wave + 3) / 4 : 0;   // wave-uniform
  auto issue_item = [&](int i) {
    if (i < nj) issue(kc, kbase, wave + 4 * i, i & 1, ktbl);
    else if (i < 2 * nj) issue(vc, vbase, wave + 4 * (i - nj), i & 1, vtbl);
  };
  // item i has landed when at most the loads of item i + 1 (eight per lane) are outstanding
  auto wait_item = [&](int i) {
    if (i + 1 < 2 * nj) fc_wait_vm<8>(); else fc_wait_vm<0>();
  };
  issue_item(0);
  issue_item(1);

  // ---- phase 1: logits of this wavefront's tiles --------------------------------------------------
  // C[head][key]: the lane owns key lrow of the tile and the heads (i/4)*8 + lhalf*4 + i%4, of which
  // only heads < 8 exist, that is registers 0..3.  Tokens past the sequence end get -inf; tiles past
  // it are never read (the statistics below stop at ntok).
  const unsigned xs = (unsigned)((lhalf ^ (lrow & 15)) << 4) + lrow * 256;
  auto logits = [&](int tile, int stage) {
    f32x16 acc;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.f;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      const uint4 kf = *reinterpret_cast<const uint4*>(ring + stage * DA_TILEB + (xs ^ (unsigned)(ks * 32)));
      acc = fc_mfma<DTYPE>(qf[ks], kf, acc);
    }
    const int t = tile * DA_TILE + lrow;
    const bool live = t < ntok;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int g = lhalf * 4 + i;
      if (g < GT) sc[g * chunk + t] = live ? acc[i] * c : -INFINITY;
    }
  };
  for (int i = 0; i < nj; ++i) {
    wait_item(i);
    logits(wave + 4 * i, i & 1);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the stage's reads are done before the next item lands in it
    issue_item(i + 2);
  }
  fc_lds_barrier();

  // ---- phase 2: chunk statistics, one wavefront per query head -------------------------------------
  for (int g = wave; g < GT; g += 4) {
    float x[DA_CHUNK_MAX / 64];
#pragma unroll
    for (int j = 0; j < DA_CHUNK_MAX / 64; ++j) x[j] = lane + 64 * j < ntok ? sc[g * chunk + lane + 64 * j] : -INFINITY;
    float mx = x[0];
#pragma unroll
    for (int j = 1; j < DA_CHUNK_MAX / 64; ++j) mx = fmaxf(mx, x[j]);
    const float m = fc_wave_max_uniform(mx);
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < DA_CHUNK_MAX / 64; ++j) {
      const float p = __builtin_amdgcn_exp2f(x[j] - m);   // exp2(-inf) = 0 for the padded slots
      if (lane + 64 * j < live_tiles * DA_TILE) {         // every slot of a live tile is read by phase 3
        if constexpr (PV_MFMA) {
          const unsigned short hi = da_pack<DTYPE>(p);
          const float hf = DTYPE == FC_BF16 ? fc_bf16_to_float(hi) : fc_half_to_float(hi);
          p2[g * chunk + lane + 64 * j] = (unsigned)hi | ((unsigned)da_pack<DTYPE>(p - hf) << 16);
        } else {
          sc[g * chunk + lane + 64 * j] = p;
        }
      }
      sum += p;
    }
    sum = fc_wave_sum_uniform(sum);
    if (lane == 0 && g0 + g < G) {
      float* ml = part_ml + (((long long)b * Hq + (h * G + g0 + g)) * max_splits + split) * 2;
      ml[0] = m;
      ml[1] = sum;
    }
  }
  fc_lds_barrier();

  // ---- phase 3: sum of p * V over this wavefront's tiles -------------------------------------------
  if constexpr (PV_MFMA) {
    // O[head][d] = P[head][key] * V[key][d] on the matrix pipe.  A = P rows from LDS (8 consecutive keys per
    // lane), as two operands hi and lo so that the probabilities keep ~16-22 mantissa bits; the B operand
    // wants 8 consecutive KEYS of one output dimension per lane, i.e. V transposed, which is read as
    // 2-byte pieces from the swizzled rows (lanes of a half-wave read neighbouring dimensions of one row,
    // the two half-waves rows 8 apart whose chunks are swizzled onto other banks).
    f32x16 oacc[4];
#pragma unroll
    for (int nb = 0; nb < 4; ++nb)
#pragma unroll
      for (int i = 0; i < 16; ++i) oacc[nb][i] = 0.f;
    auto pv = [&](int tile, int stage) {
      const char* vt = ring + stage * DA_TILEB + (lrow & 7) * 2;
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        const int k0 = s * 16 + lhalf * 8;   // first of this lane's 8 keys of the k-step
        uint4 a = make_uint4(0, 0, 0, 0), a2 = make_uint4(0, 0, 0, 0);
        if (lrow < GT) {
          const uint4 d0 = *reinterpret_cast<const uint4*>(&p2[lrow * chunk + tile * DA_TILE + k0]);
          const uint4 d1 = *reinterpret_cast<const uint4*>(&p2[lrow * chunk + tile * DA_TILE + k0 + 4]);
          // v_perm_b32 bytes: 0-3 second operand, 4-7 first operand
          a = make_uint4(__builtin_amdgcn_perm(d0.y, d0.x, 0x05040100u), __builtin_amdgcn_perm(d0.w, d0.z, 0x05040100u),
                         __builtin_amdgcn_perm(d1.y, d1.x, 0x05040100u), __builtin_amdgcn_perm(d1.w, d1.z, 0x05040100u));
          a2 = make_uint4(__builtin_amdgcn_perm(d0.y, d0.x, 0x07060302u), __builtin_amdgcn_perm(d0.w, d0.z, 0x07060302u),
                          __builtin_amdgcn_perm(d1.y, d1.x, 0x07060302u), __builtin_amdgcn_perm(d1.w, d1.z, 0x07060302u));
        }
#pragma unroll
        for (int nb = 0; nb < 4; ++nb) {
          const int chunk = nb * 4 + (lrow >> 3);
          unsigned w[4];
#pragma unroll
          for (int e2 = 0; e2 < 4; ++e2) {
            const int ka = k0 + 2 * e2, kb = ka + 1;
            const unsigned lo = *reinterpret_cast<const unsigned short*>(vt + ka * 256 + ((chunk ^ (ka & 15)) << 4));
            const unsigned hi = *reinterpret_cast<const unsigned short*>(vt + kb * 256 + ((chunk ^ (kb & 15)) << 4));
            w[e2] = lo | (hi << 16);
          }
          const uint4 bfrag = make_uint4(w[0], w[1], w[2], w[3]);
          oacc[nb] = fc_mfma<DTYPE>(a, bfrag, oacc[nb]);
          oacc[nb] = fc_mfma<DTYPE>(a2, bfrag, oacc[nb]);
        }
      }
    };
    for (int i = nj; i < 2 * nj; ++i) {
      wait_item(i);
      pv(wave + 4 * (i - nj), i & 1);
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      issue_item(i + 2);
    }
    fc_lds_barrier();   // every wavefront is done with its ring before the ring becomes `red`
    // C layout: the lane holds output dimension nb*32 + lrow of the heads lhalf*4 + i (registers 0..3)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int g = lhalf * 4 + i;
      if (g < GT) {
#pragma unroll
        for (int nb = 0; nb < 4; ++nb) red[wave][g][nb * 32 + lrow] = oacc[nb][i];
      }
    }
    fc_lds_barrier();
    for (int i = tid; i < GT * FC_HEAD_DIM; i += DA_THREADS) {
      const int g = i / FC_HEAD_DIM, d = i - g * FC_HEAD_DIM;
      if (g0 + g < G) {
        const float o = (red[0][g][d] + red[1][g][d]) + (red[2][g][d] + red[3][g][d]);
        part_o[(((long long)b * Hq + (h * G + g0 + g)) * max_splits + split) * FC_HEAD_DIM + d] = o;
      }
    }
  } else {
    float acc[GT][8];
#pragma unroll
    for (int g = 0; g < GT; ++g)
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[g][e] = 0.f;
    auto pv = [&](int tile, int stage) {
#pragma unroll
      for (int p = 0; p < 8; ++p) {
        const int r = 4 * p + rg;
        const uint4 vx = *reinterpret_cast<const uint4*>(ring + stage * DA_TILEB + r * 256 + ((sub ^ (r & 15)) << 4));
        float vf[8];
        da_unpack8<DTYPE>(vx, vf);
#pragma unroll
        for (int g = 0; g < GT; ++g) {
          const float pr = sc[g * chunk + tile * DA_TILE + r];
#pragma unroll
          for (int e = 0; e < 8; ++e) acc[g][e] = fmaf(pr, vf[e], acc[g][e]);
        }
      }
    };
    for (int i = nj; i < 2 * nj; ++i) {
      wait_item(i);
      pv(wave + 4 * (i - nj), i & 1);
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      issue_item(i + 2);
    }
    fc_lds_barrier();   // every wavefront is done with its ring before the ring becomes `red`
    // 16 partial outputs (4 wavefronts x 4 row slots) through LDS, summed in a fixed order
    {
      const int slot = wave * 4 + rg;
#pragma unroll
      for (int g = 0; g < GT; ++g) {
        float4* dst = reinterpret_cast<float4*>(&red[slot][g][sub * 8]);
        dst[0] = make_float4(acc[g][0], acc[g][1], acc[g][2], acc[g][3]);
        dst[1] = make_float4(acc[g][4], acc[g][5], acc[g][6], acc[g][7]);
      }
    }
    fc_lds_barrier();
    for (int i = tid; i < GT * FC_HEAD_DIM; i += DA_THREADS) {
      const int g = i / FC_HEAD_DIM, d = i - g * FC_HEAD_DIM;
      if (g0 + g < G) {
        float o = 0.f;
#pragma unroll
        for (int sl = 0; sl < 16; ++sl) o += red[sl][g][d];
        part_o[(((long long)b * Hq + (h * G + g0 + g)) * max_splits + split) * FC_HEAD_DIM + d] = o;
      }
    }
  }
}

template <int DTYPE>
__global__ __launch_bounds__(FC_HEAD_DIM) void decode_merge_kernel(const float* __restrict__ part_o,
                                                                   const float* __restrict__ part_ml,
                                                                   const int* __restrict__ lens, int max_seq_len,
                                                                   int Hq, int max_splits, int chunk,
                                                                   char* __restrict__ out) {
  const int hq = blockIdx.x, b = blockIdx.y, d = threadIdx.x;
  int len = min(lens[b], max_seq_len);
  unsigned short* o = reinterpret_cast<unsigned short*>(out) + ((long long)b * Hq + hq) * FC_HEAD_DIM + d;
  if (len <= 0) {
    *o = 0;
    return;
  }
  const int ns = (len + chunk - 1) / chunk;
  const float* ml = part_ml + ((long long)b * Hq + hq) * max_splits * 2;
  const float* po = part_o + ((long long)b * Hq + hq) * max_splits * FC_HEAD_DIM + d;
  // eight splits per step so that their loads are in flight together
  float M = -INFINITY;
  for (int s0 = 0; s0 < ns; s0 += 8) {
    float m[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) m[j] = s0 + j < ns ? ml[2 * (s0 + j)] : -INFINITY;
#pragma unroll
    for (int j = 0; j < 8; ++j) M = fmaxf(M, m[j]);
  }
  float L = 0.f, acc = 0.f;
  for (int s0 = 0; s0 < ns; s0 += 8) {
    float m[8], l[8], x[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const bool ok = s0 + j < ns;
      m[j] = ok ? ml[2 * (s0 + j)] : -INFINITY;
      l[j] = ok ? ml[2 * (s0 + j) + 1] : 0.f;
      x[j] = ok ? po[(long long)(s0 + j) * FC_HEAD_DIM] : 0.f;
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float w = __builtin_amdgcn_exp2f(m[j] - M);
      L = fmaf(w, l[j], L);
      acc = fmaf(w, x[j], acc);
    }
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

// compute units of the current device (0 if the query fails), cached per device
static int da_compute_units() {
  static std::atomic<int> cus[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
  int n = cus[dev].load(std::memory_order_relaxed);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n < 0) n = 0;
    cus[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}

// Checks and launches shared by the entry points; `workspace` is a device address.
static int da_enqueue(const char* who, const fc_kv_view* k_cache, const fc_kv_view* v_cache, int32_t layer,
                      const void* q, void* out, int32_t num_q_heads, const int32_t* context_lens, float scale,
                      void* workspace, int64_t workspace_bytes, void* stream) {
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
  const int B = k_cache->batch, Hkv = k_cache->num_kv_heads, G = num_q_heads / Hkv;
  // the smallest tile that holds the whole group (padded head rows cost nothing; splitting a group would
  // read its K and V once per tile); groups of more than 8 heads are served 8 at a time
  const int gt = G > 4 ? 8 : G > 2 ? 4 : G > 1 ? 2 : 1;
  const int gtiles = (G + gt - 1) / gt;
  // Tokens per workgroup: the multiple of 32 between 256 and 1024 that minimises rounds * (chunk + fixed part),
  // rounds = workgroups / (two per compute unit), rounded up.  Longer chunks spend less of a workgroup's life on
  // its ramp (first tiles in flight, nothing to compute yet) and its tail (statistics, partial results, no loads
  // in flight); a launch of few workgroups wants the chunk that fills whole rounds.  Measured: cfg4 (2880
  // columns, up to 2304 tokens) 0.327 ms per layer with 256, 0.297 with 512, 0.294 with 768; cfg5's decode (64
  // columns, 3584 tokens) 33.3 us with 256, 30.4 with 448.  Two workgroups must still fit a compute unit's LDS, which
  // caps the chunk for groups of 8 query heads.  Only the view's max_seq_len enters, never the lengths on the
  // device, so the choice is the same at capture and at every replay.
  int chunk = DA_CHUNK;
  {
    const int slots = 2 * da_compute_units();
    const long long cols = (long long)Hkv * gtiles * B;
    double best = -1.0;
    for (int cand = DA_CHUNK; slots > 0 && cand <= DA_CHUNK_MAX; cand += DA_TILE) {
      if ((DA_RING + gt * cand * 4) * 2 > 158 * 1024) break;
      const long long wgs = cols * ((k_cache->max_seq_len + cand - 1) / cand);
      const double cost = (double)((wgs + slots - 1) / slots) * (cand + 96.0);
      if (best < 0 || cost < best - 1e-9) {
        best = cost;
        chunk = cand;
      }
    }
  }
  const int splits = (k_cache->max_seq_len + chunk - 1) / chunk;
  float* part_o = (float*)workspace;
  float* part_ml = part_o + (int64_t)B * num_q_heads * (splits > 0 ? splits : 1) * FC_HEAD_DIM;
  KvView k = fc_make_view(k_cache), v = fc_make_view(v_cache);
  hipStream_t st = (hipStream_t)stream;
  const float c = scale * DA_LOG2E;
  const bool bf = k_cache->dtype == FC_BF16;
  if (splits > 0) {
    FC_REQUIRE(Hkv * gtiles <= 65535 && B <= 65535, FC_EUNSUPPORTED, "%s: grid too large", who);
    dim3 grid(splits, Hkv * gtiles, B);
    const auto tile_in_page = [](const fc_kv_view* v, const KvView& d) {
      return v->stride_token >= 0 && v->stride_token < (1 << 24) &&   // a tile's byte offsets fit 32 bits
             (v->block_tables == nullptr || (d.block_shift >= 5));
    };
    const bool fast = tile_in_page(k_cache, k) && tile_in_page(v_cache, v);
#define DA_LAUNCH(DT, GTV, FA)                                                                                   \
  do {                                                                                                          \
    FC_ALLOW_LDS((decode_attn_kernel<DT, GTV, FA>), DaCfg<GTV>::lds(DA_CHUNK_MAX));                             \
    hipLaunchKernelGGL((decode_attn_kernel<DT, GTV, FA>), grid, dim3(DA_THREADS), DaCfg<GTV>::lds(chunk), st, k, \
                       v, layer, (const char*)q, num_q_heads, context_lens, c, part_o, part_ml, splits, chunk); \
  } while (0)
#define DA_DISPATCH2(DT, FA)                        \
  switch (gt) {                                     \
    case 8: DA_LAUNCH(DT, 8, FA); break;            \
    case 4: DA_LAUNCH(DT, 4, FA); break;            \
    case 2: DA_LAUNCH(DT, 2, FA); break;            \
    default: DA_LAUNCH(DT, 1, FA); break;           \
  }
#define DA_DISPATCH(DT) \
  if (fast) { DA_DISPATCH2(DT, true) } else { DA_DISPATCH2(DT, false) }
    if (bf) { DA_DISPATCH(FC_BF16) } else { DA_DISPATCH(FC_F16) }
#undef DA_DISPATCH
#undef DA_DISPATCH2
#undef DA_LAUNCH
    FC_CHECK_LAUNCH(who);
  }
  dim3 mgrid(num_q_heads, B);
  if (bf)
    hipLaunchKernelGGL((decode_merge_kernel<FC_BF16>), mgrid, dim3(FC_HEAD_DIM), 0, st, part_o, part_ml, context_lens,
                       k_cache->max_seq_len, num_q_heads, splits, chunk, (char*)out);
  else
    hipLaunchKernelGGL((decode_merge_kernel<FC_F16>), mgrid, dim3(FC_HEAD_DIM), 0, st, part_o, part_ml, context_lens,
                       k_cache->max_seq_len, num_q_heads, splits, chunk, (char*)out);
  FC_CHECK_LAUNCH(who);
  return FC_OK;
}

extern "C" int fc_decode_attn(const fc_kv_view* k_cache, const fc_kv_view* v_cache, int32_t layer, const void* q,
                              void* out, int32_t num_q_heads, const int32_t* context_lens, float scale,
                              void* workspace, int64_t workspace_bytes, void* stream) {
  return da_enqueue("fc_decode_attn", k_cache, v_cache, layer, q, out, num_q_heads, context_lens, scale, workspace,
                    workspace_bytes, stream);
}

// ---- the same attention for callers that cannot allocate -------------------------------------------------
// The chunk partials live in a file-scope device array instead of a caller workspace.  `scratch` below is the
// host-side handle of that array, not a device address: its address on the current device is looked up once
// per device (every GPU holds its own copy) and only that address is ever handed to a kernel.
#define DA_STATIC_BYTES (16ll << 20)
static __device__ __align__(256) unsigned char scratch[DA_STATIC_BYTES];

#define DA_MAX_DEVICES 64
// filled per device on first use; two threads racing here store the same value
static std::atomic<void*> da_scratch_ptr[DA_MAX_DEVICES];
// Every call on a device shares that device's array, so two calls whose kernels overlap (different streams, or a
// graph replay beside an eager call) corrupt each other's chunk partials.  The library cannot see that in general
// without synchronising; with FC_STATIC_GUARD=1 in the environment it checks the one case it can name cheaply: a
// call on another stream than the previous call's while that stream still has work pending is refused.  The check
// queries the previous stream, so leave it off when streams are being captured.
static std::atomic<void*> da_last_stream[DA_MAX_DEVICES];
static std::atomic<int> da_last_stream_set[DA_MAX_DEVICES];
static bool da_guard_enabled() {
  static const bool on = [] {
    const char* e = getenv("FC_STATIC_GUARD");
    return e && e[0] && e[0] != '0';
  }();
  return on;
}

extern "C" int64_t fc_decode_attn_static_capacity(void) { return DA_STATIC_BYTES; }

extern "C" int fc_decode_attn_static(const fc_kv_view* k_cache, const fc_kv_view* v_cache, int32_t layer,
                                     const void* q, void* out, int32_t num_q_heads, const int32_t* context_lens,
                                     float scale, void* stream) {
  const char* who = "fc_decode_attn_static";
  FC_REQUIRE(k_cache && num_q_heads > 0, FC_EINVAL, "%s: null view or bad head count", who);
  const int64_t need = fc_decode_attn_workspace_bytes(k_cache->batch, num_q_heads, k_cache->max_seq_len);
  FC_REQUIRE(need > 0, FC_EINVAL, "%s: bad sizes", who);
  FC_REQUIRE(need <= DA_STATIC_BYTES, FC_EUNSUPPORTED,
             "%s: batch %d x %d query heads x max_seq_len %d needs %lld bytes of chunk partials, the built-in "
             "buffer holds %lld; use fc_decode_attn with a workspace",
             who, k_cache->batch, num_q_heads, k_cache->max_seq_len, (long long)need, (long long)DA_STATIC_BYTES);
  int dev = -1;
  FC_REQUIRE(hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < DA_MAX_DEVICES, FC_EUNSUPPORTED,
             "%s: no current device below %d", who, DA_MAX_DEVICES);
  void* ws = da_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!ws) {
    const hipError_t e = hipGetSymbolAddress(&ws, HIP_SYMBOL(scratch));
    FC_REQUIRE(e == hipSuccess && ws, FC_ELAUNCH, "%s: hipGetSymbolAddress: %s", who, hipGetErrorString(e));
    da_scratch_ptr[dev].store(ws, std::memory_order_release);
  }
  if (da_guard_enabled()) {
    if (da_last_stream_set[dev].load(std::memory_order_acquire)) {
      void* last = da_last_stream[dev].load(std::memory_order_acquire);
      if (last != stream) {
        const hipError_t q = hipStreamQuery((hipStream_t)last);
        if (q != hipSuccess) (void)hipGetLastError();
        FC_REQUIRE(q != hipErrorNotReady, FC_EINVAL,
                   "%s: the previous call on this device used another stream that still has work pending; calls "
                   "that share the built-in buffer must not overlap", who);
      }
    }
    da_last_stream[dev].store(stream, std::memory_order_release);
    da_last_stream_set[dev].store(1, std::memory_order_release);
  }
  return da_enqueue(who, k_cache, v_cache, layer, q, out, num_q_heads, context_lens, scale, ws, DA_STATIC_BYTES,
                    stream);
}
