// SnapKV observation-window scoring for fp16/bf16 caches.
//
// One workgroup per (layer, sequence, kv head) with one wavefront per 32-row block of window
// queries (group of G query heads x ceil(W/32) blocks, up to 16 wavefronts).  A wavefront keeps
// its 32 query rows as MFMA operands in registers for the whole kernel.  Keys stream through LDS
// in tiles of 64 rows: global memory -> LDS directly (global_load_lds_dwordx4, no register
// staging), three or four tiles resident or in flight per workgroup, one barrier per tile.  Rows
// are unpadded; their 16-byte chunks are XOR-swizzled with the row number so that the operand
// reads of a half-wave (32 rows, same chunk) fall on distinct banks.  Logits come from
// v_mfma_f32_32x32x16, 16 per lane and 32x32 block.
//
// The softmax needs every key of a row before any probability is final, and the [G*W, S] logit
// matrix does not fit on chip, so the keys are swept twice:
//   sweep 1  C[key][query] orientation: a lane owns ONE query and 16 keys per block, so its
//            softmax state is two scalars (largest logit, sum of exp2).  The first tile fixes the
//            offset with the online-softmax update; later tiles only add exp2(logit - offset).
//            Should a sum overflow, the sweep is redone with the online update on every tile;
//   sweep 2  C[query][key] orientation, tiles in descending order (the tiles read last are the
//            likeliest to still be cached): logits recomputed, p = exp2(x - m) / l summed over the
//            lane's 16 queries, the two half-waves and the group's wavefronts (fixed order, no
//            atomics) into a 4-tile ring of per-key sums, from which the zero-padded moving
//            average of width `kernel_size` is written one tile later.
// In both sweeps the MFMAs of a block are issued together with the exponentials of the block
// before it (two accumulator sets, sched_group_barrier hints).  All arithmetic after the MFMA is
// fp32.  The second sweep reads K again (a workgroup's column does not stay in L2 between the
// sweeps), so the kernel's memory traffic is about twice the algorithmic figure.
// Optionally the kernel also emits the maximum of each score row for the window fill.
// When the caller supplies the log-sum-exp of every window query (a fused attention kernel returns it),
// sweep 1 is skipped: its result is exactly that number.
//
// Table entries of a live sequence must be allocated blocks: a negative entry inside the sequence
// reads block 0 instead of faulting.
#include "fc_press.h"

#define SK_KT 64           // keys per tile
#define SK_TILEB (SK_KT * 256)  // LDS bytes per key tile (rows unpadded, 16-byte chunks XOR-swizzled)
#define SK_NEG (-1.0e30f)  // "minus infinity" that stays finite under subtraction
#define SK_TBL 1024        // block-table entries of one sequence cached in LDS

__device__ __forceinline__ float sk_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

template <int NW>
struct SkCfg {
  static constexpr int ST = NW >= 8 ? 4 : 3;   // key tiles resident or in flight per workgroup
  // + 256: the key tiles start on a 256-byte LDS address (see the operand reads)
#ifndef SK_LDS_PAD
#define SK_LDS_PAD 0   // experiments: extra LDS per workgroup, to hold the number of workgroups per compute unit down
#endif
  static constexpr int LDS = ST * SK_TILEB + (4 * NW + 4) * SK_KT * 4 + SK_TBL * 4 + 256 + SK_LDS_PAD;
};

// MODE 0: the whole kernel for one (layer, sequence, kv head) column.
// The key range of a column can also be cut into `nsplit` pieces, one workgroup each, for launches with too few
// columns to fill the GPU:
// MODE 1: sweep 1 over the piece's tiles only; (largest scaled logit, sum of exp2) per query go to `part`;
// MODE 2: sweep 2 over the piece's tiles with the log-sum-exp given; the per-key sums go to `raw` unpooled
//         (a small kernel takes the moving average afterwards, across the pieces' borders).
// PRESS (MODE 0, at least four wavefronts): the workgroup goes on to select the column's kept positions (the
// window always among them) and to move the kept K and V rows to the front of the column, see the end of the kernel.
struct SkPress {
  KvView vv;            // the value plane, same geometry as the keys
  int k;                // kept positions per row when n_kept is null
  const int* n_kept;    // [batch] in device memory, or null
  int* indices;         // [layers][batch][kv heads][index_stride]
  int index_stride;
};

// LDS the press tail carves out of the key tiles and the per-key sum area behind them: the score row, the kept
// positions, the value view's block-table row and the selection's counters
template <int NW>
constexpr int sk_press_room() { return SkCfg<NW>::ST * SK_TILEB + (4 * NW + 4) * SK_KT * 4; }
__host__ __device__ constexpr int sk_press_need(int max_seq_len, int index_stride) {
  return 4 * max_seq_len + 4 * index_stride + 4 * SK_TBL + 4096 + 16 * CP_PT;   // + the selection's counters, page addresses
}

template <int DTYPE, int NW, bool FAST, int MODE, bool PRESS = false>
__global__ __launch_bounds__(NW * 64, (NW <= 8 ? 4 : 2)) void snapkv_kernel(
    KvView kv, const char* __restrict__ q, int Hq, int W, int ksz, int causal, float c, float out_mul,
    float* __restrict__ scores, int score_stride, float* __restrict__ row_max, const float* __restrict__ lse,
    int nsplit, float* __restrict__ part, float* __restrict__ raw, SkPress press) {
  constexpr int THREADS = NW * 64;
  constexpr int ST = SkCfg<NW>::ST;
  constexpr int LPW = 16 / NW;   // 1 KB wave-loads (4 key rows) per wavefront and tile
  static_assert(LPW * NW == 16, "NW must divide 16");
  extern __shared__ __align__(16) char smem_raw[];
  // The key tiles start on a multiple of 256 in LDS address terms, so that the LDS base can be folded into a lane's
  // operand address before the XOR that picks the 16-byte chunk (which touches address bits 4..7 only).
  char* smem = smem_raw + ((256u - (fc_lds_addr(smem_raw) & 255u)) & 255u);
  char* kbuf = smem;
  float(*vpart)[NW][SK_KT] = reinterpret_cast<float(*)[NW][SK_KT]>(smem + ST * SK_TILEB);
  float(*vraw)[SK_KT] = reinterpret_cast<float(*)[SK_KT]>(smem + ST * SK_TILEB + 4 * NW * SK_KT * 4);
  int* tbl = reinterpret_cast<int*>(smem + ST * SK_TILEB + (4 * NW + 4) * SK_KT * 4);

  const int Hkv = kv.num_kv_heads;
  const int b = blockIdx.y, l = blockIdx.z;
  const int h = MODE == 0 ? (int)blockIdx.x : (int)blockIdx.x % Hkv;
  const int split = MODE == 0 ? 0 : (int)blockIdx.x / Hkv;
  const int G = Hq / Hkv;
  const int WB = (W + 31) / 32;        // 32-row blocks per query head
  const int RBT = G * WB;              // row blocks of the group
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lrow = lane & 31, lhalf = lane >> 5;
  const int S = __builtin_amdgcn_readfirstlane(fc_seq_len(kv, b));
  float* out_row = scores + (((long long)l * kv.batch + b) * Hkv + h) * (long long)score_stride;

  if (S <= W) {  // nothing outside the window to score
    if (MODE != 0) return;   // the pooling kernel writes such rows
    for (int s = tid; s < score_stride; s += THREADS) out_row[s] = s < S ? 0.f : -INFINITY;
    if (row_max && tid == 0) row_max[((long long)l * kv.batch + b) * Hkv + h] = -INFINITY;
    if constexpr (PRESS) {   // every position is a window position: the first kept-count of them stay where they are
      int kk = press.n_kept ? press.n_kept[b] : press.k;
      kk = min(min(kk, S), press.index_stride);
      int* idx_row = press.indices + (((long long)l * kv.batch + b) * Hkv + h) * (long long)press.index_stride;
      for (int i = tid; i < kk; i += THREADS) idx_row[i] = i;
    }
    return;
  }
  const int SW = S - W;                       // scored keys
  const int T = (S + SK_KT - 1) / SK_KT;      // key tiles
  // this workgroup's tiles [tb, te) and the number of tile positions it walks
  int tb = 0, te = T;
  if (MODE != 0) {
    const int tps = (T + nsplit - 1) / nsplit;
    tb = split * tps;
    te = min(T, tb + tps);
    if (tb >= te) return;
  }
  const int P = MODE == 0 ? 2 * T : te - tb;

  // ---- query fragment: this wavefront's 32 query rows as MFMA A-operands ------------------
  uint4 qf[8];
  const bool rb_valid = wave < RBT;
  const int qg = rb_valid ? wave / WB : 0;
  const int qi = (rb_valid ? wave - qg * WB : 0) * 32;   // first query index of the block
  {
    const int qa = qi + lrow;
    const bool ok = rb_valid && qa < W;
    const char* qp = q + (((((long long)l * kv.batch + b) * Hq + (h * G + qg)) * W + qa) * FC_HEAD_DIM + lhalf * 8) * 2;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks)
      qf[ks] = ok ? *reinterpret_cast<const uint4*>(qp + ks * 32) : make_uint4(0, 0, 0, 0);
  }

  // this sequence's block-table row, so that the tile loads do not wait on a table read each
  const bool paged = kv.block_tables != nullptr;
  const bool tbl_lds = paged && kv.block_shift >= 0 && ((S - 1) >> kv.block_shift) < SK_TBL;
  if (tbl_lds) {
    const int nblk = ((S - 1) >> kv.block_shift) + 1;
    for (int i = tid; i < nblk; i += THREADS) tbl[i] = kv.block_tables[(long long)b * kv.table_stride + i];
  }
  __syncthreads();

  // ---- key tiles: global -> LDS, ST stages ---------------------------------------------------
  // A wave-load moves 4 key rows (1 KB).  Lane i writes LDS chunk i of those 64 chunks and fetches
  // the global chunk (i & 15) ^ (row & 15) of row i / 16, which is the XOR swizzle that keeps the
  // B-operand reads (32 rows, same chunk) free of bank conflicts.  Rows past the sequence end are
  // clamped to its last row (every lane always loads, so the outstanding-load count is exact);
  // those keys are masked in sweep 1 and never emitted in sweep 2.
  const char* kbase = kv.base + ((long long)l * kv.stride_layer + (long long)h * kv.stride_head) * 2;
  const unsigned kbuf_lds = __builtin_amdgcn_readfirstlane(fc_lds_addr(kbuf));
  // FAST: a tile lies inside one page (or the view is dense), so a load is a wave-uniform tile base
  // plus a per-lane byte offset; the offset is recomputed per load rather than kept in registers.
  const unsigned tok_bytes = (unsigned)kv.stride_token * 2;
  unsigned lofs[LPW];   // byte offset of this lane's 16 bytes inside a tile, per wave-load
#pragma unroll
  for (int u = 0; u < LPW; ++u) {
    const int r = 4 * (wave * LPW + u) + (lane >> 4);
    lofs[u] = (unsigned)r * tok_bytes + (((lane & 15) ^ (r & 15)) << 4);
  }
  auto issue = [&](int tile, int stage) {
    if constexpr (FAST) {
      const int s0 = tile * SK_KT;
      long long tb;
      if (paged) {
        const int blk = max(__builtin_amdgcn_readfirstlane(tbl[s0 >> kv.block_shift]), 0);
        tb = (long long)blk * kv.stride_block + (long long)(s0 & (kv.block_size - 1)) * kv.stride_token;
      } else {
        tb = (long long)b * kv.stride_batch + (long long)s0 * kv.stride_token;
      }
      // (wave-uniform by construction; said again so that it stays in scalar registers across the branch below)
      const unsigned long long gu = (unsigned long long)(kbase + tb * 2);
      const char* g = reinterpret_cast<const char*>(
          ((unsigned long long)(unsigned)__builtin_amdgcn_readfirstlane((int)(gu >> 32)) << 32) |
          (unsigned)__builtin_amdgcn_readfirstlane((int)(gu & 0xffffffffu)));
      const int rmax = S - 1 - s0;   // rows past the end re-read the last row
      if (rmax >= SK_KT - 1) {       // a whole tile: the lane offsets are the ones prepared before the loops
#pragma unroll
        for (int u = 0; u < LPW; ++u) fc_load_lds(g, lofs[u], kbuf_lds + stage * SK_TILEB + (wave * LPW + u) * 1024);
      } else {
#pragma unroll
        for (int u = 0; u < LPW; ++u) {
          const int r = 4 * (wave * LPW + u) + (lane >> 4);
          const unsigned lo = (unsigned)min(r, rmax) * tok_bytes + (((lane & 15) ^ (r & 15)) << 4);
          fc_load_lds(g, lo, kbuf_lds + stage * SK_TILEB + (wave * LPW + u) * 1024);
        }
      }
    } else {
#pragma unroll 1
    for (int u = 0; u < LPW; ++u) {
      const int j = wave * LPW + u;
      const int r = 4 * j + (lane >> 4);
      const int ch = (lane & 15) ^ (r & 15);
      const int s = min(tile * SK_KT + r, S - 1);
      long long off = fc_token_offset(kv, b, s);
      if (off < 0) off = 0;
      fc_load_lds(kbase + off * 2 + ch * 16, kbuf_lds + stage * SK_TILEB + j * 1024);
    }
    }
  };
  // One plan = sweep 1 over the tiles in ascending order, then sweep 2 in descending order (the
  // tiles read last are the likeliest to still be cached).  m is the position in the plan, kc the
  // number of tiles consumed so far; tile position m lives in stage (kc % ST) when it is consumed
  // and positions m+1 .. m+ST-2 are in flight meanwhile.
  auto plan_tile = [&](int pos) {
    if (MODE == 1) return tb + pos;        // ascending
    if (MODE == 2) return te - 1 - pos;    // descending
    return pos < T ? pos : 2 * T - 1 - pos;
  };
  unsigned kc = 0;   // unsigned: kc % ST is a mask for ST = 4
  int m = 0;
  auto prologue = [&](int first) {   // first = 0: both sweeps; first = T: the second sweep alone
    m = first;
    for (int i = 0; i < ST - 1 && first + i < P; ++i) issue(plan_tile(first + i), (int)((kc + (unsigned)i) % ST));
  };
  // top of a tile iteration: tile position m has landed for every wave, the stage consumed by the
  // previous iteration is free and receives position m+ST-1; returns the stage to read
  auto acquire = [&]() {
    if (m + ST - 2 < P) fc_wait_barrier<LPW*(ST - 2)>(); else fc_wait_barrier<0>();
    const int nx = m + ST - 1;
    if (nx < P) issue(plan_tile(nx), (int)((kc + ST - 1) % ST));
    return (int)(kc % ST);
  };

  const bool always_general = SW < SK_KT;
  const int swz = lrow & 15;

  // LDS address of the lane's fragment of k-slice ks of a 32-key block: the row base plus the
  // swizzled chunk ((ks*2 + lhalf) ^ swz) * 16.  ks*32, lhalf*16 and the row base occupy disjoint
  // bits, so this is (row base + xs) ^ (ks*32).
  const unsigned xs = (unsigned)((lhalf ^ swz) << 4) + lrow * 256 + kbuf_lds;   // an absolute LDS address
  // 32 keys x 32 queries of logits.  KEYS_ROWS: C[key][query] (the lane owns one query and 16
  // keys), otherwise C[query][key] (the lane owns one key and 16 queries).
  auto mfma_block = [&](bool keys_rows, int stage, int cb, f32x16& acc) {
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.f;
    const unsigned a0 = (unsigned)(stage * SK_TILEB + cb * 8192) + xs;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      const uint4 kf = fc_lds_read128(a0 ^ (unsigned)(ks * 32));
      #ifdef FC_ABLATE_MFMA16
      acc = keys_rows ? fc_mfma<DTYPE>(kf, qf[ks], acc, ks) : fc_mfma<DTYPE>(qf[ks], kf, acc, ks);
#else
      acc = keys_rows ? fc_mfma<DTYPE>(kf, qf[ks], acc) : fc_mfma<DTYPE>(qf[ks], kf, acc);
#endif
    }
  };
  // The same for the loops that walk whole tiles: the eight fragment addresses of a tile's first block are
  // formed once per tile (tile_addr) and the second block reads 8192 bytes further, which the read instruction
  // adds by itself.
  unsigned adr[8];
  auto tile_addr = [&](int stage) {
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) adr[ks] = ((unsigned)(stage * SK_TILEB) + xs) ^ (unsigned)(ks * 32);
  };
  auto mfma_tile_block = [&](bool keys_rows, int cb, f32x16& acc) {
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.f;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      const uint4 kf = fc_lds_read128(adr[ks] + (unsigned)(cb * 8192));
      #ifdef FC_ABLATE_MFMA16
      acc = keys_rows ? fc_mfma<DTYPE>(kf, qf[ks], acc, ks) : fc_mfma<DTYPE>(qf[ks], kf, acc, ks);
#else
      acc = keys_rows ? fc_mfma<DTYPE>(kf, qf[ks], acc) : fc_mfma<DTYPE>(qf[ks], kf, acc);
#endif
    }
  };
  // ask the scheduler to spread the VALU work of one block between the MFMAs of the next
  auto interleave = [&]() {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // one MFMA
      __builtin_amdgcn_sched_group_barrier(0x002, 7, 0);   // seven VALU
    }
  };

  // ================= sweep 1: softmax statistics ==============================================
  // C[key][query]: lane (lrow, lhalf) owns query qi + lrow and, per 32-key block, the 16 keys
  // (i/4)*8 + lhalf*4 + i%4.  Its state is (mref, lsq): the largest raw logit seen and the sum of
  // exp2((logit - mref) * c).  The first tile uses the online update; later tiles only add
  // exp2(logit * c - mref * c): any fixed offset is mathematically valid, it merely has to keep the
  // sums inside the fp32 range.  A sum that overflows (logits rising by more than ~2^7 in log2
  // units above the first tile's) is detected afterwards and the sweep is redone with the online
  // update on every tile.  Masked logits are SK_NEG; differences are formed before scaling so that
  // SK_NEG - SK_NEG is exactly 0 and nothing overflows.
  float mref = SK_NEG, lsq = 0.f, nmq = 0.f;
  const int klim = causal ? min(S, SW + qi + lrow + 1) : S;   // first masked key of this lane's query
  auto stats_general = [&](f32x16& acc, int t, int cb) {
    const int sb = t * SK_KT + cb * 32 + lhalf * 4;
#pragma unroll
    for (int i = 0; i < 16; ++i)
      if (sb + (i >> 2) * 8 + (i & 3) >= klim) acc[i] = SK_NEG;
    float mx = acc[0];
#pragma unroll
    for (int i = 1; i < 16; ++i) mx = fmaxf(mx, acc[i]);
    float bs = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) bs += sk_exp2((acc[i] - mx) * c);
    const float mnew = fmaxf(mref, mx);
    lsq = lsq * sk_exp2((mref - mnew) * c) + bs * sk_exp2((mx - mnew) * c);
    mref = mnew;
  };
  auto stats_fast = [&](const f32x16& acc) {
#pragma unroll
    for (int i = 0; i < 16; ++i) lsq += sk_exp2(fmaf(acc[i], c, nmq));
  };
  // tiles [t0, t1) one block at a time, with masking; fixed offset unless `general`
  auto sweep1_plain = [&](int t0, int t1, bool general) {
    for (int t = t0; t < t1; ++t) {
      const int stage = acquire();
#pragma unroll
      for (int cb = 0; cb < 2; ++cb) {
        f32x16 acc;
        mfma_block(true, stage, cb, acc);
        if (general) {
          stats_general(acc, t, cb);
        } else {
          const int sb = t * SK_KT + cb * 32 + lhalf * 4;
#pragma unroll
          for (int i = 0; i < 16; ++i)
            if (sb + (i >> 2) * 8 + (i & 3) >= klim) acc[i] = SK_NEG;
          stats_fast(acc);
        }
      }
      ++m;
      ++kc;
    }
  };
  // unmasked tiles [t0, t1), t1 > t0, fixed offset: the MFMAs of each block are issued together
  // with the exponentials of the block before it
  auto sweep1_piped = [&](int t0, int t1) {
    f32x16 acc_a, acc_b;
    tile_addr(acquire());
    mfma_tile_block(true, 0, acc_a);
    for (int t = t0; t < t1 - 1; ++t) {
      mfma_tile_block(true, 1, acc_b);
      stats_fast(acc_a);
      interleave();
      asm volatile("" : "+v"(lsq));   // ... nor sink acc_a's exponentials below it
      ++m;
      ++kc;
      tile_addr(acquire());
      // acc_b's exponentials are pure register arithmetic, which the compiler would otherwise move ahead of the
      // barrier in acquire() and leave the MFMAs below without vector work to overlap
      asm volatile("" : "+v"(acc_b));
      mfma_tile_block(true, 0, acc_a);
      stats_fast(acc_b);
      interleave();
    }
    mfma_tile_block(true, 1, acc_b);
    stats_fast(acc_a);
    interleave();
    stats_fast(acc_b);
    ++m;
    ++kc;
  };
  // leading tiles without any masked key
  const int TF = causal ? min(S, SW + 1) / SK_KT : S / SK_KT;
  // With the log-sum-exp of every window query given (the attention kernel of the prefill has it), the
  // first sweep is not needed at all.
  const bool skip_sweep1 = MODE == 2 || (MODE == 0 && lse != nullptr);
  if (skip_sweep1) prologue(MODE == 2 ? 0 : T);
  for (int attempt = 0; attempt < 2 && !skip_sweep1; ++attempt) {
    prologue(0);
    if (always_general || attempt == 1) {
      sweep1_plain(tb, te, true);
    } else {
      sweep1_plain(tb, tb + 1, true);
      nmq = -mref * c;
      const int tf_end = min(TF, te);
      if (tf_end > tb + 1) sweep1_piped(tb + 1, tf_end);
      sweep1_plain(max(tf_end, tb + 1), te, false);
    }
    const bool bad = !(lsq <= 3.0e38f);   // inf or NaN
    if (attempt == 1) break;
    // Did any lane of the workgroup overflow?  Through the (still unused) per-key sum area rather than
    // __syncthreads_or, whose static LDS word would move the key tiles off LDS address 0 and cost every
    // operand read an extra address addition.
    const bool wave_bad = __any(bad);
    if (lane == 0) vpart[0][wave][0] = wave_bad ? 1.f : 0.f;
    __syncthreads();
    float any_bad = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) any_bad += vpart[0][w][0];
    if (!__builtin_amdgcn_readfirstlane(any_bad > 0.f)) break;
    fc_wait_barrier<0>();   // the tiles prefetched for sweep 2 land before their stages are reused
    mref = SK_NEG;
    lsq = 0.f;
  }

  // merge the two half-waves' states of each query and fold the normaliser into the offset:
  // p = exp2(logit * c + nmfin), nmfin = -(max * c) - log2(sum).  Then hand every lane the offsets
  // of the 16 queries it owns in the C[query][key] orientation of sweep 2.
  float nm[16];
  {
    const float m2 = __shfl_xor(mref, 32, 64), l2 = __shfl_xor(lsq, 32, 64);
    const float mnew = fmaxf(mref, m2);
    const float ll = lsq * sk_exp2((mref - mnew) * c) + l2 * sk_exp2((m2 - mnew) * c);
    const bool ok = rb_valid && qi + lrow < W;
    if constexpr (MODE == 1) {   // this piece's statistics of the query, in log2 units; done
      if (ok && lhalf == 0) {
        float* pp = part + (((((long long)l * kv.batch + b) * Hq + (h * G + qg)) * W + qi + lrow) * nsplit + split) * 2;
        pp[0] = mnew * c;
        pp[1] = ll;
      }
      return;
    }
    float nmfin = ok ? -mnew * c - __builtin_amdgcn_logf(ll) : SK_NEG;   // v_log_f32 is log2
    if (lse && ok)   // natural-log sum of exp(scale * q.k) over the keys the query sees
      nmfin = -1.4426950408889634f *
              lse[((((long long)l * kv.batch + b) * Hq + (h * G + qg)) * W + qi + lrow)];
#pragma unroll
    for (int i = 0; i < 16; ++i) nm[i] = __shfl(nmfin, (i >> 2) * 8 + lhalf * 4 + (i & 3), 64);
  }

  // ================= sweep 2: probabilities, per-key sums, moving average ======================
  // C[query][key], tiles in descending order.  Every wavefront leaves its per-key sums of a tile in
  // vpart (four tiles deep); one iteration later the sums are folded (fixed order) into vraw, a ring
  // of four tiles, each wavefront taking 64/NW keys; the moving average of a tile is written two
  // iterations after its own fold, when both neighbours are in the ring.
  const int hw = ksz >> 1;
  // Every wavefront folds and emits 64/NW keys of a tile with NW lanes per key.
  constexpr int KPW = SK_KT / NW;
  const int fkey = wave * KPW + lane / NW, fp = lane % NW;
  const int tend = MODE == 2 ? te : T;          // sweep 2 walks tiles tend-1, tend-2, ...
  const int P2 = MODE == 2 ? te - tb : T;       // ... P2 of them
  auto fold = [&](int u) {   // tile processed u-th (tile tend-1-u): sum the wavefronts' partial sums per key
    const float v = fc_group_sum<NW>(vpart[u & 3][fp][fkey]);
    if constexpr (MODE == 2) {
      const int s = (tend - 1 - u) * SK_KT + fkey;
      if (fp == 0 && s < SW) raw[(((long long)l * kv.batch + b) * Hkv + h) * (long long)score_stride + s] = v;
    } else {
      if (fp == 0) vraw[(T - 1 - u) & 3][fkey] = v;
    }
  };
  auto emit_tile = [&](int e) {   // moving average of tile e, whose neighbours are folded
    const int s = e * SK_KT + fkey;
    float a = 0.f;
    if (ksz <= NW) {   // the usual case: at most one term per lane, no loop
      const int x = s + fp - hw;
      if (fp < ksz && x >= 0 && x < SW) a = vraw[(x >> 6) & 3][x & (SK_KT - 1)];
    } else {
      for (int j = fp; j < ksz; j += NW) {
        const int x = s + j - hw;
        if (x >= 0 && x < SW) a += vraw[(x / SK_KT) & 3][x % SK_KT];
      }
    }
    a = fc_group_sum<NW>(a);
    if (fp == 0 && s < SW) out_row[s] = a * out_mul;
  };
  auto probs = [&](const f32x16& acc, int u, int cb) {
    float vs = sk_exp2(fmaf(acc[0], c, nm[0]));
#pragma unroll
    for (int i = 1; i < 16; ++i) vs += sk_exp2(fmaf(acc[i], c, nm[i]));
    vs += __shfl_xor(vs, 32, 64);
    if (lane < 32) vpart[u & 3][wave][cb * 32 + lane] = vs;
  };
  {
    f32x16 acc_a, acc_b;
    tile_addr(acquire());
    mfma_tile_block(false, 0, acc_a);
    for (int u = 0; u < P2 - 1; ++u) {
      mfma_tile_block(false, 1, acc_b);
      probs(acc_a, u, 0);
      interleave();
      ++m;
      ++kc;
      tile_addr(acquire());
      // the sums of the tile processed before this one are complete: fold them; tile T-u+2 had
      // both neighbours folded (by other wavefronts) before the barrier just passed
      if (u >= 1) fold(u - 1);
      if (MODE == 0 && u >= 3) emit_tile(T - u + 2);
      mfma_tile_block(false, 0, acc_a);
      probs(acc_b, u, 1);
      interleave();
    }
    mfma_tile_block(false, 1, acc_b);
    probs(acc_a, P2 - 1, 0);
    interleave();
    probs(acc_b, P2 - 1, 1);
    ++m;
    ++kc;
  }
  if constexpr (MODE == 2) {   // the last two tiles' sums; pooling, tail and row maximum are the pooling kernel's
    __syncthreads();
    if (P2 >= 2) fold(P2 - 2);
    fold(P2 - 1);
    return;
  }

  // ---- drain: fold the last two tiles processed (tiles 1 and 0) and write tiles 3, 2, 1, 0.  Tile 3 needs
  // tile 4, whose ring slot tile 0 takes over, so tile 0 is folded after tiles 3 and 2 are written.
  __syncthreads();
  if (T >= 2) fold(T - 2);
  __syncthreads();
  emit_tile(3);
  emit_tile(2);
  __syncthreads();
  fold(T - 1);
  __syncthreads();
  emit_tile(1);
  emit_tile(0);
  for (int s = S + tid; s < score_stride; s += THREADS) out_row[s] = -INFINITY;
  if (row_max) {   // maximum of this row's scores, for the window fill: re-read what this workgroup wrote
    __syncthreads();
    float rmax = -INFINITY;
    for (int s = tid; s < SW; s += THREADS) rmax = fmaxf(rmax, out_row[s]);
    rmax = fc_wave_max(rmax);
    if (lane == 0) vpart[0][wave][0] = rmax;
    __syncthreads();
    if (tid == 0) {
      float mx = vpart[0][0][0];
#pragma unroll
      for (int w = 1; w < NW; ++w) mx = fmaxf(mx, vpart[0][w][0]);
      row_max[((long long)l * kv.batch + b) * Hkv + h] = mx;
    }
  }
  // ---- press: select and compact this column --------------------------------------------------------------
  // The window positions rank above every scored key (the caller fills them with the layer's largest score
  // afterwards), so with more kept positions than window positions the selection over the filled row is: the window,
  // plus the kk - W best of the scored keys; only those enter the selection.  The score row is read back from memory (this workgroup wrote it; its stores are waited for) into the
  // LDS that held the key tiles.
  if constexpr (PRESS) {
    static_assert(MODE == 0 && NW >= 4, "the press tail needs a whole column and at least 256 threads");
    int kk = press.n_kept ? press.n_kept[b] : press.k;
    kk = min(min(kk, S), press.index_stride);
    if (kk <= W) return;   // not a selection this tail can make; the host does not ask for it
    fc_wait_vm<0>();
    __syncthreads();
    float* sc = reinterpret_cast<float*>(smem);
    int* sel = reinterpret_cast<int*>(smem) + S;
    int* vtbl = sel + press.index_stride;
    TkArea<THREADS>& sh = *reinterpret_cast<TkArea<THREADS>*>(vtbl + SK_TBL);
    static_assert(sizeof(TkArea<THREADS>) <= 4096 - 8, "the selection's counters outgrew their share of the LDS budget");
    // page addresses of the column for the compaction: 8-byte words behind the counters (smem is 16-byte aligned)
    const int ptbl_word = (S + press.index_stride + SK_TBL + (int)(sizeof(TkArea<THREADS>) / 4) + 1) & ~1;
    unsigned long long* ptbl = reinterpret_cast<unsigned long long*>(reinterpret_cast<int*>(smem) + ptbl_word);
    for (int s = tid; s < SW; s += THREADS) sc[s] = out_row[s];
    const KvView& vv = press.vv;
    const int nblk_v = vv.block_shift >= 0 ? ((S - 1) >> vv.block_shift) + 1 : 0;
    const bool v_lds = vv.block_tables && vv.block_shift >= 0 && nblk_v <= SK_TBL;
    if (v_lds)
      for (int i = tid; i < nblk_v; i += THREADS) vtbl[i] = vv.block_tables[(long long)b * vv.table_stride + i];
    __syncthreads();
    int* idx_row = press.indices + (((long long)l * kv.batch + b) * Hkv + h) * (long long)press.index_stride;
    kp_select_and_move<2, THREADS, true>(kv, vv, tbl, tbl_lds, vtbl, v_lds, sc, sel, sh, ptbl, l, b, h, S, kk, W, idx_row);
  }
}

// Split columns: the pieces' (max, sum) per window query -> natural-log sum of exponentials.
__global__ __launch_bounds__(256) void snapkv_merge_stats_kernel(const float* __restrict__ part, long long queries_total,
                                                                 int queries_per_seq, int batch,
                                                                 const int* __restrict__ seq_lens, int max_seq_len,
                                                                 int nsplit, float* __restrict__ lse) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;   // (layer, b, hq, w) flattened
  if (i >= queries_total) return;
  const int b = (int)((i / queries_per_seq) % batch);
  int S = seq_lens ? seq_lens[b] : max_seq_len;
  S = S < max_seq_len ? (S < 0 ? 0 : S) : max_seq_len;
  const int T = (S + SK_KT - 1) / SK_KT;
  if (T == 0) return;
  const int tps = (T + nsplit - 1) / nsplit;
  const int used = (T + tps - 1) / tps;                            // pieces that had tiles
  const float* pp = part + i * nsplit * 2;
  float M = SK_NEG;
  for (int s = 0; s < used; ++s) M = fmaxf(M, pp[2 * s]);
  float L = 0.f;
  for (int s = 0; s < used; ++s) L += pp[2 * s + 1] * sk_exp2(pp[2 * s] - M);
  lse[i] = (M + __builtin_amdgcn_logf(L)) * 0.6931471805599453f;   // log2 units -> natural log
}

// Split columns: zero-padded moving average of the raw per-key sums, the tail past the sequence, the row maximum.
__global__ __launch_bounds__(256) void snapkv_pool_kernel(const float* __restrict__ raw, float* __restrict__ scores,
                                                          int score_stride, const int* __restrict__ seq_lens,
                                                          int max_seq_len, int W, int ksz, float out_mul,
                                                          float* __restrict__ row_max) {
  __shared__ float red[4];
  const int h = blockIdx.x, b = blockIdx.y, l = blockIdx.z;
  const long long row = ((long long)l * gridDim.y + b) * gridDim.x + h;
  int S = seq_lens ? seq_lens[b] : max_seq_len;
  S = S < max_seq_len ? (S < 0 ? 0 : S) : max_seq_len;
  const float* in = raw + row * score_stride;
  float* out = scores + row * score_stride;
  const int tid = threadIdx.x;
  if (S <= W) {
    for (int s = tid; s < score_stride; s += 256) out[s] = s < S ? 0.f : -INFINITY;
    if (row_max && tid == 0) row_max[row] = -INFINITY;
    return;
  }
  const int SW = S - W, hw = ksz >> 1;
  float mx = -INFINITY;
  for (int s = tid; s < score_stride; s += 256) {
    if (s < SW) {
      float a = 0.f;
      for (int x = max(s - hw, 0); x <= min(s + hw, SW - 1); ++x) a += in[x];
      a *= out_mul;
      out[s] = a;
      mx = fmaxf(mx, a);
    } else if (s >= S) {
      out[s] = -INFINITY;
    }
  }
  if (row_max) {
    mx = fc_wave_max(mx);
    if ((tid & 63) == 0) red[tid >> 6] = mx;
    __syncthreads();
    if (tid == 0) row_max[row] = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
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

static int snapkv_score_impl(const char* who, const fc_kv_view* keys, const void* queries, int32_t num_q_heads,
                             int32_t window, int32_t kernel_size, int32_t causal_window, float scale, float out_scale,
                             float* scores, int32_t score_stride, float* row_max, const float* lse, void* stream,
                             const fc_kv_view* press_values = nullptr, int32_t press_k = 0,
                             const int32_t* press_n_kept = nullptr, int32_t* press_indices = nullptr,
                             int32_t press_index_stride = 0) {
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
  const int waves = rbt;
  FC_REQUIRE(waves <= 16, FC_EUNSUPPORTED, "%s: group of %d heads x window %d needs %d wavefronts (max 16)", who, G,
             window, waves);
  if (keys->max_seq_len == 0) return FC_OK;
  KvView kv = fc_make_view(keys);
  dim3 grid(keys->num_kv_heads, keys->batch, keys->num_layers);
  hipStream_t st = (hipStream_t)stream;
  const float c = scale * 1.4426950408889634f;
  const float out_mul = out_scale / (float)kernel_size;
  const char* q = (const char*)queries;
  // a key tile lies inside one page (whose table row fits the LDS copy), or the view is dense
  const bool fast = keys->stride_token >= 0 && keys->stride_token < (1 << 24) &&   // a tile's byte offsets fit 32 bits
                    (!keys->block_tables ||
                     (kv.block_shift >= 6 && ((keys->max_seq_len - 1) >> kv.block_shift) < SK_TBL));
  if (press_values) {   // scoring, selection and compaction of every column by its workgroup
    const fc_kv_view* values = press_values;
    if ((rc = fc_check_view(values, who))) return rc;
    FC_REQUIRE(keys->dtype == values->dtype && keys->num_layers == values->num_layers &&
                   keys->batch == values->batch && keys->num_kv_heads == values->num_kv_heads &&
                   keys->max_seq_len == values->max_seq_len,
               FC_EINVAL, "%s: key and value views disagree on dtype/layers/batch/heads/length", who);
    FC_REQUIRE(press_indices, FC_EINVAL, "%s: null indices", who);
    FC_REQUIRE(press_index_stride >= 0 && press_index_stride <= keys->max_seq_len, FC_EINVAL,
               "%s: index_stride %d exceeds max_seq_len %d", who, press_index_stride, keys->max_seq_len);
    FC_REQUIRE(press_n_kept != nullptr || (press_k > window && press_k <= press_index_stride), FC_EINVAL,
               "%s: k=%d must exceed the window (%d) and fit index_stride=%d", who, press_k, window,
               press_index_stride);
    const int nw = waves <= 4 ? 4 : (waves <= 8 ? 8 : 16);
    const int room = nw == 4 ? sk_press_room<4>() : (nw == 8 ? sk_press_room<8>() : sk_press_room<16>());
    FC_REQUIRE(fast && sk_press_need(keys->max_seq_len, press_index_stride) <= room, FC_EUNSUPPORTED,
               "%s: the one-launch press takes dense views or pages of 64*2^n tokens and 4*(max_seq_len + "
               "index_stride) + 12288 <= %d bytes (got max_seq_len %d, index_stride %d); use fc_snapkv_score and "
               "fc_select_compact", who, room, keys->max_seq_len, press_index_stride);
    SkPress press;
    press.vv = fc_make_view(values);
    press.k = press_k;
    press.n_kept = press_n_kept;
    press.indices = press_indices;
    press.index_stride = press_index_stride;
#define SK_PRESS(DT, NWV)                                                                                        \
  do {                                                                                                         \
    FC_ALLOW_LDS((snapkv_kernel<DT, NWV, true, 0, true>), SkCfg<NWV>::LDS);                                     \
    hipLaunchKernelGGL((snapkv_kernel<DT, NWV, true, 0, true>), grid, dim3(NWV * 64), SkCfg<NWV>::LDS, st, kv, \
                       q, num_q_heads, window, kernel_size, causal_window, c, out_mul, scores, score_stride,   \
                       row_max, lse, 1, (float*)nullptr, (float*)nullptr, press);                              \
  } while (0)
#define SK_PRESS_NW(DT)                 \
  if (nw == 4) SK_PRESS(DT, 4);         \
  else if (nw == 8) SK_PRESS(DT, 8);    \
  else SK_PRESS(DT, 16)
    if (keys->dtype == FC_BF16) { SK_PRESS_NW(FC_BF16); } else { SK_PRESS_NW(FC_F16); }
#undef SK_PRESS_NW
#undef SK_PRESS
    FC_CHECK_LAUNCH(who);
    return FC_OK;
  }
#define SK_LAUNCH(DT, NWV, FA)                                                                                  \
  do {                                                                                                       \
    FC_ALLOW_LDS((snapkv_kernel<DT, NWV, FA, 0>), SkCfg<NWV>::LDS);                                           \
    hipLaunchKernelGGL((snapkv_kernel<DT, NWV, FA, 0>), grid, dim3(NWV * 64), SkCfg<NWV>::LDS, st, kv, q,    \
                       num_q_heads, window, kernel_size, causal_window, c, out_mul, scores, score_stride,    \
                       row_max, lse, 1, (float*)nullptr, (float*)nullptr, SkPress{});                        \
  } while (0)
  // One wavefront per 32-row block of window queries, but never fewer than four: a lone wavefront has to fetch a whole
  // key tile by itself between two barriers (one block of queries: 7.2 ms with one wavefront, 0.87 ms with four of
  // which three only fetch, 2048 columns of 4096 keys); two blocks score 2-7 % slower with four wavefronts than with
  // two, but four is what the press tail needs, and scoring and press must sum in the same order to agree bit for bit
  // (whole pass, 2048 columns of 4096 keys and 8192 of 1024: 1.37 -> 1.34 ms and 1.41 -> 1.27 ms in one launch).
#define SK_DISPATCH2(DT, FA)                 \
  if (waves <= 4) SK_LAUNCH(DT, 4, FA);      \
  else if (waves <= 8) SK_LAUNCH(DT, 8, FA); \
  else SK_LAUNCH(DT, 16, FA)
#define SK_DISPATCH(DT) \
  if (fast) { SK_DISPATCH2(DT, true); } else { SK_DISPATCH2(DT, false); }
  if (keys->dtype == FC_BF16) { SK_DISPATCH(FC_BF16); } else { SK_DISPATCH(FC_F16); }
#undef SK_DISPATCH2
#undef SK_DISPATCH
#undef SK_LAUNCH
  FC_CHECK_LAUNCH(who);
  return FC_OK;
}

extern "C" int fc_snapkv_score(const fc_kv_view* keys, const void* queries, int32_t num_q_heads, int32_t window,
                               int32_t kernel_size, int32_t causal_window, float scale, float out_scale,
                               float* scores, int32_t score_stride, float* row_max, void* stream) {
  return snapkv_score_impl("fc_snapkv_score", keys, queries, num_q_heads, window, kernel_size, causal_window, scale,
                           out_scale, scores, score_stride, row_max, nullptr, stream);
}

extern "C" int fc_snapkv_score_lse(const fc_kv_view* keys, const void* queries, const float* lse, int32_t num_q_heads,
                                   int32_t window, int32_t kernel_size, int32_t causal_window, float scale,
                                   float out_scale, float* scores, int32_t score_stride, float* row_max,
                                   void* stream) {
  const char* who = "fc_snapkv_score_lse";
  FC_REQUIRE(lse, FC_EINVAL, "%s: null log-sum-exp pointer", who);
  return snapkv_score_impl(who, keys, queries, num_q_heads, window, kernel_size, causal_window, scale, out_scale,
                           scores, score_stride, row_max, lse, stream);
}

extern "C" int fc_snapkv_press(const fc_kv_view* keys, const fc_kv_view* values, const void* queries, const float* lse,
                               int32_t num_q_heads, int32_t window, int32_t kernel_size, int32_t causal_window,
                               float scale, float out_scale, float* scores, int32_t score_stride, float* row_max,
                               int32_t k, const int32_t* n_kept, int32_t* indices, int32_t index_stride,
                               void* stream) {
  const char* who = "fc_snapkv_press";
  FC_REQUIRE(values && row_max, FC_EINVAL, "%s: null value view or row_max", who);
  return snapkv_score_impl(who, keys, queries, num_q_heads, window, kernel_size, causal_window, scale, out_scale,
                           scores, score_stride, row_max, lse, stream, values, k, n_kept, indices, index_stride);
}

// ---- split columns ------------------------------------------------------------------------------------
extern "C" int64_t fc_snapkv_split_workspace_bytes(int32_t num_layers, int32_t batch, int32_t num_q_heads,
                                                   int32_t num_kv_heads, int32_t window, int32_t score_stride,
                                                   int32_t nsplit) {
  if (num_layers <= 0 || batch <= 0 || num_q_heads <= 0 || num_kv_heads <= 0 || window <= 0 || score_stride < 0 ||
      nsplit <= 0)
    return -1;
  const int64_t nq = (int64_t)num_layers * batch * num_q_heads * window;
  return (nq * nsplit * 2 + nq + (int64_t)num_layers * batch * num_kv_heads * score_stride + 64) * (int64_t)sizeof(float);
}

extern "C" int fc_snapkv_score_split(const fc_kv_view* keys, const void* queries, const float* lse, int32_t num_q_heads,
                                     int32_t window, int32_t kernel_size, int32_t causal_window, float scale,
                                     float out_scale, float* scores, int32_t score_stride, float* row_max,
                                     int32_t nsplit, void* workspace, int64_t workspace_bytes, void* stream) {
  const char* who = "fc_snapkv_score_split";
  int rc = fc_check_view(keys, who);
  if (rc) return rc;
  FC_REQUIRE(queries && scores && workspace, FC_EINVAL, "%s: null pointer", who);
  FC_REQUIRE(((uintptr_t)queries & 15) == 0 && ((uintptr_t)workspace & 15) == 0, FC_EINVAL,
             "%s: queries / workspace not 16-byte aligned", who);
  FC_REQUIRE(keys->dtype == FC_F16 || keys->dtype == FC_BF16, FC_EUNSUPPORTED,
             "%s: fp16/bf16 caches only (got dtype %d)", who, keys->dtype);
  FC_REQUIRE(num_q_heads > 0 && num_q_heads % keys->num_kv_heads == 0, FC_EINVAL,
             "%s: num_q_heads %d not a multiple of num_kv_heads %d", who, num_q_heads, keys->num_kv_heads);
  FC_REQUIRE(window > 0, FC_EINVAL, "%s: window must be positive", who);
  FC_REQUIRE(kernel_size >= 1 && (kernel_size & 1) && kernel_size <= 63, FC_EINVAL,
             "%s: kernel_size %d must be odd and <= 63", who, kernel_size);
  FC_REQUIRE(score_stride >= keys->max_seq_len, FC_EINVAL, "%s: score_stride %d < max_seq_len %d", who,
             score_stride, keys->max_seq_len);
  FC_REQUIRE(nsplit >= 1 && nsplit <= 256, FC_EINVAL, "%s: nsplit %d out of range [1, 256]", who, nsplit);
  const int L = keys->num_layers, B = keys->batch, Hkv = keys->num_kv_heads;
  const int G = num_q_heads / Hkv;
  const int waves = G * ((window + 31) / 32);
  KvView kv = fc_make_view(keys);
  const bool fast = keys->stride_token >= 0 && keys->stride_token < (1 << 24) &&   // a tile's byte offsets fit 32 bits
                    (!keys->block_tables ||
                     (kv.block_shift >= 6 && ((keys->max_seq_len - 1) >> kv.block_shift) < SK_TBL));
  FC_REQUIRE(waves <= 16 && fast, FC_EUNSUPPORTED,
             "%s: split columns need a query group of at most 16 row blocks (got %d) and pages of 64*2^n tokens or a "
             "dense view", who, waves);
  const int64_t need = fc_snapkv_split_workspace_bytes(L, B, num_q_heads, Hkv, window, score_stride, nsplit);
  FC_REQUIRE(workspace_bytes >= need, FC_EINVAL, "%s: workspace of %lld bytes, %lld needed", who,
             (long long)workspace_bytes, (long long)need);
  FC_REQUIRE((long long)Hkv * nsplit <= 2147483647LL && B <= 65535 && L <= 65535, FC_EUNSUPPORTED, "%s: grid too large",
             who);
  if (keys->max_seq_len == 0) return FC_OK;
  const long long nq = (long long)L * B * num_q_heads * window;
  float* part = (float*)workspace;
  float* lse_ws = part + nq * nsplit * 2;
  float* raw = lse_ws + nq;
  hipStream_t st = (hipStream_t)stream;
  const float c = scale * 1.4426950408889634f;
  const float out_mul = out_scale / (float)kernel_size;
  const char* q = (const char*)queries;
  dim3 grid(Hkv * nsplit, B, L);
  const float* lse_use = lse;
#define SK_SPLIT(DT, NWV, MD)                                                                                      \
  do {                                                                                                           \
    FC_ALLOW_LDS((snapkv_kernel<DT, NWV, true, MD>), SkCfg<NWV>::LDS);                                            \
    hipLaunchKernelGGL((snapkv_kernel<DT, NWV, true, MD>), grid, dim3(NWV * 64), SkCfg<NWV>::LDS, st, kv, q,     \
                       num_q_heads, window, kernel_size, causal_window, c, out_mul, scores, score_stride,        \
                       row_max, lse_use, nsplit, part, raw, SkPress{});                                          \
  } while (0)
#define SK_SPLIT_NW(DT, MD)                     \
  if (waves <= 4) SK_SPLIT(DT, 4, MD);          \
  else if (waves <= 8) SK_SPLIT(DT, 8, MD);     \
  else SK_SPLIT(DT, 16, MD)
  if (!lse) {   // pieces' statistics, then their merge into the log-sum-exp
    if (keys->dtype == FC_BF16) { SK_SPLIT_NW(FC_BF16, 1); } else { SK_SPLIT_NW(FC_F16, 1); }
    hipLaunchKernelGGL(snapkv_merge_stats_kernel, dim3((unsigned)((nq + 255) / 256)), dim3(256), 0, st,
                       (const float*)part, nq, num_q_heads * window, B, keys->seq_lens, keys->max_seq_len, nsplit,
                       lse_ws);
    lse_use = lse_ws;
  }
  if (keys->dtype == FC_BF16) { SK_SPLIT_NW(FC_BF16, 2); } else { SK_SPLIT_NW(FC_F16, 2); }
#undef SK_SPLIT_NW
#undef SK_SPLIT
  hipLaunchKernelGGL(snapkv_pool_kernel, dim3(Hkv, B, L), dim3(256), 0, st, (const float*)raw, scores, score_stride,
                     keys->seq_lens, keys->max_seq_len, window, kernel_size, out_mul, row_max);
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
