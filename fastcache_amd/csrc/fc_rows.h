// Ordered movement of token rows of one (layer, sequence, head) column by one workgroup, shared by the kernels that
// compact a cache in place.
//
// A token row of one head is 128 elements (256 or 512 bytes) and is moved by 16 or 32 lanes with 16-byte accesses.
// The column is walked in ascending chunks: all source rows of a chunk are loaded into registers, the workgroup waits
// for the loads and synchronises, and only then are the chunk's destination rows stored (while the next chunk's loads
// are already in flight).  With ascending unique source positions (dst j <= src of j) this makes the in-place case
// (dst aliases src) safe: a chunk's stores can only hit rows whose reads have already completed, and later chunks
// read rows that no earlier chunk writes.
#pragma once
#include "fc_common.h"

typedef unsigned cp_u32x4 __attribute__((ext_vector_type(4)));   // native vector: arrays of it stay in registers

#ifndef CP_R
#define CP_R 8      // 16-byte loads in flight per lane and chunk
#endif
#define CP_TBL 1024 // block-table entries of one sequence cached in LDS (per view)

// The loaded registers are not consumed before the barrier, so wait for them explicitly.  The stores
// of the previous chunk were issued AFTER these loads; when every lane of the wavefront issued all
// CP_R of them (stores_behind), the loads are complete as soon as at most CP_R operations are still
// outstanding, and the stores' completion is not waited for.
__device__ __forceinline__ void cp_wait_then_barrier(bool stores_behind) {
  if (stores_behind)
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(CP_R) : "memory");
  else
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// Element offset of token s of sequence b (-1: its page is not allocated).  With the table row in LDS the page offset is
// two 32 x 32 -> 64 bit multiply-adds when both strides fit 32 bits (which the workgroup tests once, on scalars), and
// the unallocated page is a select, not a branch: this sits in front of every row load and store.
__device__ __forceinline__ long long cp_offset(const KvView& v, const int* tbl, bool tbl_lds, int b, int s) {
  if (tbl_lds) {
    const int blk = tbl[s >> v.block_shift];
    const unsigned page = (unsigned)max(blk, 0), slot = (unsigned)s & (unsigned)(v.block_size - 1);
    long long off;
    if ((((unsigned long long)v.stride_block | (unsigned long long)v.stride_token) >> 32) == 0ull)
      off = (long long)((unsigned long long)page * (unsigned)v.stride_block +
                        (unsigned long long)slot * (unsigned)v.stride_token);
    else
      off = (long long)page * v.stride_block + (long long)slot * v.stride_token;
    return blk < 0 ? -1ll : off;
  }
  return fc_token_offset(v, b, s);
}

// Rows j = 0 .. n-1 of a column: destination token dst_start + j <- source token src_of(j).  The workgroup (THREADS
// threads, all of which call this) moves HG adjacent heads at once: lane group rg handles head rg % HG of token
// rg / HG of a pass, so that the HG head rows of a token (contiguous in memory) are moved by neighbouring lanes;
// sbase / dbase point at the lane's 16 bytes of its head's row of token offset 0 and `safe` at 16 readable bytes
// (read in place of rows that do not exist, so that every lane always loads).  stbl / dtbl: the sequence's block-table
// rows in LDS when s_lds / d_lds.  Two register buffers: the loads of chunk c+1 are issued right after the barrier that
// releases the stores of chunk c, so loads and stores overlap.
template <int EB, int HG, int THREADS, typename SrcOf>
__device__ __forceinline__ void cp_walk(const KvView& src, const KvView& dst, const int* stbl, bool s_lds,
                                        const int* dtbl, bool d_lds, int b, int S, int n, const char* sbase,
                                        char* dbase, const char* safe, int dst_start, SrcOf src_of) {
  constexpr int LPR = FC_HEAD_DIM * EB / 16;
  constexpr int RPP = THREADS / LPR;
  constexpr int CH = RPP * CP_R / HG;   // tokens per chunk
  constexpr int TPP = RPP / HG;         // tokens per pass
  const int tg = ((int)threadIdx.x / LPR) / HG;

  auto load_idx = [&](int (&si)[CP_R], int j0) {
#pragma unroll
    for (int u = 0; u < CP_R; ++u) {
      const int j = j0 + u * TPP + tg;
      si[u] = j < n ? src_of(j) : -1;
    }
  };
  // Every lane always loads and the validity goes into a bit mask: with no control flow around the buffer
  // elements they stay in registers.
  auto load_rows = [&](cp_u32x4 (&buf)[CP_R], unsigned& ok, const int (&si)[CP_R]) {
    ok = 0;
#pragma unroll
    for (int u = 0; u < CP_R; ++u) {
      const int s = si[u];
      long long off = -1;
      if (s >= 0 && s < S) off = cp_offset(src, stbl, s_lds, b, s);
      const bool valid = off >= 0;
      const char* p = valid ? sbase + off * EB : safe;
      buf[u] = *reinterpret_cast<const cp_u32x4*>(p);
      ok |= valid ? (1u << u) : 0u;
    }
  };
  // returns whether every lane of this wavefront stored all CP_R rows
  auto store_rows = [&](const cp_u32x4 (&buf)[CP_R], unsigned ok, int j0) {
    bool all = true;
#pragma unroll
    for (int u = 0; u < CP_R; ++u) {
      const int j = j0 + u * TPP + tg;
      long long off = -1;
      if (ok & (1u << u)) off = cp_offset(dst, dtbl, d_lds, b, dst_start + j);
      if (off >= 0) *reinterpret_cast<cp_u32x4*>(dbase + off * EB) = buf[u];
      all &= off >= 0;
    }
    return (bool)__all(all);
  };

  cp_u32x4 bufa[CP_R], bufb[CP_R];
  unsigned oka, okb;
  int sia[CP_R], sib[CP_R];
  load_idx(sia, 0);
  load_rows(bufa, oka, sia);
  load_idx(sib, CH);
  bool behind = false;   // the newest operations in flight are exactly CP_R stores of this wavefront
  for (int j0 = 0; j0 < n; j0 += 2 * CH) {
    // chunk j0 is in flight in buffer a; the indices of chunk j0 + CH are in sib
    cp_wait_then_barrier(behind);
    if (j0 + CH < n) load_rows(bufb, okb, sib);
    load_idx(sia, j0 + 2 * CH);
    behind = store_rows(bufa, oka, j0);
    if (j0 + CH >= n) break;
    cp_wait_then_barrier(behind);
    if (j0 + 2 * CH < n) load_rows(bufa, oka, sia);
    load_idx(sib, j0 + 3 * CH);
    behind = store_rows(bufb, okb, j0 + CH);
  }
}

// ---- the in-place walk of a paged column over precomputed page addresses ---------------------------------------------
// cp_walk computes every row's address from the view (table look-up, two 64-bit multiply-adds, the unallocated-page
// select), about thirty vector instructions per row and lane for source and destination together.  A press that
// compacts a column onto itself can do with far fewer: the address of (page i, slot 0) of this column's layer and head
// is put in LDS once per page (ptbl), a source row then costs one table read, one 24-bit multiply-add and a 64-bit
// add, and a chunk's destination rows share one page, so their address is a scalar base plus a per-lane offset that
// never changes.  Conditions (cp_pages_ok, and every page of the sequence allocated): power-of-two pages that hold a
// whole chunk, at most CP_PT pages, a token stride below 2^24 bytes.
#define CP_PT 256

template <int EB, int THREADS>
__device__ __forceinline__ bool cp_pages_ok(const KvView& v, int S) {
  constexpr int CH = (THREADS / (FC_HEAD_DIM * EB / 16)) * CP_R;
  return v.block_tables != nullptr && v.block_shift >= 0 && v.block_size >= CH && S > 0 &&
         ((S - 1) >> v.block_shift) < CP_PT && v.stride_token > 0 && v.stride_token * EB < (1ll << 24);
}

// ptbl[i] = address of token 0 of page i of the column whose (layer, head) offset `colbase` carries; tbl = the
// sequence's block-table row in LDS.  Returns (to every thread, behind a barrier) whether all pages are allocated.
template <int EB, int THREADS>
__device__ __forceinline__ bool cp_fill_pages(const KvView& v, const int* tbl, char* colbase, int S,
                                              unsigned long long* ptbl) {
  int bad = 0;
  for (int i = threadIdx.x; i <= ((S - 1) >> v.block_shift); i += THREADS) {
    const int blk = tbl[i];
    bad |= blk < 0;
    ptbl[i] = (unsigned long long)(uintptr_t)(colbase + (long long)max(blk, 0) * v.stride_block * EB);
  }
  return !__syncthreads_or(bad);
}

// One plane's page addresses and geometry for the walks below.
struct CpPages {
  const unsigned long long* ptbl;   // LDS: address of token 0 of page i (layer and head applied)
  int shift;                        // log2 of the page size
  unsigned tok_bytes;               // bytes between consecutive tokens of a page
};

// Rows j = 0 .. n-1 of BOTH planes: token j <- token sel[j] (ascending, sel[j] >= j, all below the sequence length; sel
// in LDS), in place.  A chunk's K and V rows are loaded together, the workgroup waits for them and synchronises, and
// only then are they stored; the next chunk's loads follow the stores at once (the stores are not waited for).
template <int EB, int THREADS>
__device__ __forceinline__ void cp_walk_pages(const CpPages& kp, const CpPages& vp, int n, const int* sel) {
  constexpr int LPR = FC_HEAD_DIM * EB / 16;
  constexpr int RPP = THREADS / LPR;
  constexpr int CH = RPP * CP_R;   // tokens per chunk
  const int tid = threadIdx.x;
  const int tg = tid / LPR;
  const unsigned lane_b = (unsigned)(tid % LPR) * 16u;

  auto load_rows = [&](const CpPages& pl, cp_u32x4 (&buf)[CP_R], int j0) {
    const unsigned slot_mask = (1u << pl.shift) - 1u;
#pragma unroll
    for (int u = 0; u < CP_R; ++u) {
      const int j = min(j0 + u * RPP + tg, n - 1);   // rows past the end re-read the last one and are not stored
      const unsigned s = (unsigned)sel[j];
      const char* page = reinterpret_cast<const char*>((uintptr_t)pl.ptbl[s >> pl.shift]);
      buf[u] = *reinterpret_cast<const cp_u32x4*>(page + (__umul24(s & slot_mask, pl.tok_bytes) + lane_b));
    }
  };
  auto store_rows = [&](const CpPages& pl, const cp_u32x4 (&buf)[CP_R], int j0) {
    // the chunk lies in one page (CH divides the page size): a wave-uniform base, a per-lane offset
    const unsigned slot_mask = (1u << pl.shift) - 1u;
    const unsigned long long pg = pl.ptbl[j0 >> pl.shift];
    const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)pg);
    const unsigned hi = __builtin_amdgcn_readfirstlane((unsigned)(pg >> 32));
    char* base = reinterpret_cast<char*>((uintptr_t)(((unsigned long long)hi << 32) | lo)) +
                 (unsigned long long)((unsigned)j0 & slot_mask) * pl.tok_bytes;
    const unsigned dlane = (unsigned)tg * pl.tok_bytes + lane_b;
#pragma unroll
    for (int u = 0; u < CP_R; ++u) {
      char* row = base + (unsigned long long)(unsigned)(u * RPP) * pl.tok_bytes;   // wave-uniform
      if (j0 + u * RPP + tg < n) *reinterpret_cast<cp_u32x4*>(row + dlane) = buf[u];
    }
  };

  cp_u32x4 kb[CP_R], vb[CP_R];
  for (int j0 = 0; j0 < n; j0 += CH) {
    load_rows(kp, kb, j0);
    load_rows(vp, vb, j0);
    // The loads follow the previous chunk's stores in issue order, so waiting for them waits for those stores as
    // well; a store is acknowledged long before a load that misses the caches returns, so that costs nothing.
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    store_rows(kp, kb, j0);
    store_rows(vp, vb, j0);
  }
}
