/*
 * fastcache_hip.h — C ABI of libfastcache_hip.so (gfx950 / MI355X).
 *
 * The reference (Ringssss/Fastcache) has no FFI for its KV-cache compression
 * path: its boundary is a set of Python call signatures that end in torch ops,
 * Triton kernels and two third-party wheels (kvpress, flash-attn).  Each entry
 * point below names the reference call it stands in for (paths are relative to
 * the reference root).
 *
 * Conventions (all entry points):
 *   - every pointer is a DEVICE pointer owned by the caller, except the
 *     descriptor structs themselves (fc_kv_view, fc_mlp_weights), which are
 *     read on the host during the call and may be freed after it returns;
 *   - the call only ENQUEUES work on `stream` (a hipStream_t passed as void*;
 *     NULL = the default stream): no allocation and no synchronisation, so it
 *     may be recorded into a HIP graph.  What the library keeps between calls
 *     is small and per process: the calling thread's last error text; for each
 *     kernel that needs more than 64 KB of dynamic LDS, one bit per device
 *     saying that its limit has been raised (hipFuncSetAttribute on the first
 *     launch on a device; unsynchronised, setting it twice is harmless); the
 *     compute-unit count of each device; and, for fc_decode_attn_static only,
 *     the device address of its built-in buffer (and, with FC_STATIC_GUARD=1 in the
 *     environment, the stream of the previous call on each device).  The first launch of a kernel
 *     on a device therefore does host-side work: make it outside a graph
 *     capture;
 *   - return value: FC_OK (0) or a negative FC_E* code; nothing is enqueued
 *     when an error is returned; fc_last_error() gives a message for the
 *     calling thread;
 *   - head_dim must be 128 (every model family of the reference path);
 *   - element types: FC_F32, FC_F16, FC_BF16.
 */
#ifndef FASTCACHE_HIP_H
#define FASTCACHE_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/*
 * Version of the SIGNATURES and STRUCT LAYOUTS below, returned by fc_abi_version().  The policy is additive: a
 * release may add entry points and error codes without changing the number (a binding looks an optional entry point
 * up by name and does without it when the look-up fails); the number changes only when an existing entry point's
 * arguments or meaning, or a struct's layout, change, and a binding that was written for another number must refuse
 * to run.  Everything added since the first release (the one-launch presses, the ragged MLP, the entry point with a
 * built-in buffer, the optional FC_STATIC_GUARD check) left the existing signatures as they were: still 1.
 */
#define FC_ABI_VERSION 1

enum { FC_F32 = 0, FC_F16 = 1, FC_BF16 = 2 };

enum {
  FC_OK = 0,
  FC_EINVAL = -1,      /* bad argument (null pointer, non-positive size, unsupported dtype/head_dim) */
  FC_EUNSUPPORTED = -2,/* shape outside what the kernels were built for */
  FC_ELAUNCH = -3      /* hipLaunchKernel reported an error */
};

/*
 * A strided view of one K (or V) cache, either
 *   paged  (block_tables != NULL): nano-vllm pool kv_cache[kv][layer][block][slot][kv_head][d]
 *          (nanovllm/engine/llava_model_runner.py:526-529); token s of sequence b lives in
 *          block block_tables[b*table_stride + s/block_size], slot s%block_size;
 *   dense  (block_tables == NULL): a HuggingFace-layout tensor [B, Hkv, S, D], possibly a
 *          permuted view (llava_model_runner.py:863-868).
 * Element address (in elements of `dtype` from `base`):
 *   paged: layer*stride_layer + block*stride_block + slot*stride_token + head*stride_head + d
 *   dense: layer*stride_layer + b*stride_batch     + s*stride_token    + head*stride_head + d
 * The d axis is contiguous.  seq_lens[b] gives each sequence's token count (NULL in dense
 * mode = every sequence has max_seq_len tokens).
 */
typedef struct fc_kv_view {
  void* base;
  int64_t stride_layer;
  int64_t stride_block;
  int64_t stride_batch;
  int64_t stride_token;
  int64_t stride_head;
  const int32_t* block_tables;
  int32_t table_stride;   /* entries per row of block_tables */
  int32_t block_size;     /* 256 in the reference (nanovllm/engine/sequence.py:15) */
  int32_t dtype;
  int32_t num_layers;
  int32_t batch;
  int32_t num_kv_heads;
  int32_t head_dim;
  int32_t max_seq_len;
  const int32_t* seq_lens;
} fc_kv_view;

int fc_abi_version(void);
const char* fc_last_error(void);

/*
 * Knorm scoring.  scores[l][b][h][s] = -||K[l][b][h][s][:]||_2, fp32 accumulation, for
 * s < seq_lens[b]; entries s >= seq_lens[b] are set to -inf.
 * Replaces kvpress.KnormPress.score (third-party; reference call sites
 * utils_ccm/utils_compress.py:22-24, 318-320, 347-348) evaluated per layer inside the
 * attention forward hook (utils_compress.py:209-270).
 * scores: float[num_layers][batch][num_kv_heads][score_stride].
 */
int fc_knorm_score(const fc_kv_view* keys, float* scores, int32_t score_stride, void* stream);

/*
 * Head-averaged key norms of the in-tree adapter: mean_norm[l][b][s] = mean_h ||K[l][b][h][s]||_2
 * (nanovllm/kernels/kvpress_compressor.py:220-223).  Entries s >= seq_lens[b] are -inf.
 * out: float[num_layers][batch][score_stride].
 */
int fc_knorm_mean_score(const fc_kv_view* keys, float* out, int32_t score_stride, void* stream);

/*
 * SnapKV scoring over an observation window.
 *   queries: [num_layers][batch][num_q_heads][window][head_dim] (contiguous, dtype of keys) —
 *            the already-rotated last `window` query positions;
 *   A = softmax_fp32(Q K^T * scale) over all keys of kv head hq / (num_q_heads/num_kv_heads),
 *       with (causal_window != 0) key position S-W+j masked for window query i when j > i;
 *   v[hq][s] = sum_i A[hq][i][s] for s < S-W;  pooled = avg_pool1d(v, kernel, stride 1,
 *   pad kernel/2, zeros counted);  scores[l][b][hkv][s] = out_scale * sum_{hq in group} pooled.
 *   Entries S-W <= s < S are left for fc_snapkv_fill_window; entries s >= S are -inf.
 *   row_max (optional, float[num_layers][batch][num_kv_heads]) receives each row's largest score.
 * Replaces kvpress.SnapKVPress.score / compute_window_attention (third-party; reference
 * call sites utils_ccm/utils_compress.py:310-312, 335-337; bench_kvpress_native.py:137-147;
 * nanovllm/kernels/kvpress_compressor.py:139-143).
 * Every sequence must have seq_len > window.  kernel_size must be odd and <= 63.
 */
int fc_snapkv_score(const fc_kv_view* keys, const void* queries, int32_t num_q_heads,
                    int32_t window, int32_t kernel_size, int32_t causal_window,
                    float scale, float out_scale,
                    float* scores, int32_t score_stride, float* row_max, void* stream);

/*
 * The same scores when the caller already has the log-sum-exp of every window query,
 *   lse[layer][b][hq][w] = ln sum_s exp(scale * q . k_s)   over the keys the query sees
 * (fp32, contiguous; with causal_window the keys up to the query's own position) -- what a fused
 * attention kernel returns for its rows (flash-attn's softmax_lse for the last `window` positions of the
 * prefill).  The kernel then needs a single pass over K instead of two.  The reference has no
 * counterpart: its SnapKVPress recomputes the window attention from scratch (call sites as above).
 */
int fc_snapkv_score_lse(const fc_kv_view* keys, const void* queries, const float* lse, int32_t num_q_heads,
                        int32_t window, int32_t kernel_size, int32_t causal_window, float scale,
                        float out_scale, float* scores, int32_t score_stride, float* row_max, void* stream);

/*
 * SnapKV press in one launch: fc_snapkv_score (or fc_snapkv_score_lse when `lse` is not NULL) and, by the same
 * workgroup that scored a (layer, b, kv head) column, the selection of the column's kept positions and the compaction
 * of `keys` and `values` onto themselves.  Kept counts (k, or n_kept[b] in device memory) include the window and must
 * exceed it: the window positions rank first, so the indices and cache bytes are those of fc_snapkv_score +
 * fc_snapkv_fill_window + fc_topk_select + fc_compact, except where scored keys tie EXACTLY with the layer's largest
 * score and are more than the row keeps outside the window (after the fill such keys tie with the window positions and
 * the lower index wins; here the window wins).  `scores` receives the scored
 * positions and `row_max` (required) the per-row maxima; the caller runs fc_snapkv_fill_window afterwards if it wants
 * the window entries of `scores` filled.  Rows of sequences no longer than the window keep their first positions.
 * Takes dense views or pages of 64*2^n tokens and sequences short enough for the score row and the kept positions to
 * fit the LDS of the key tiles: 4 * (max_seq_len + index_stride) + 12288 bytes within 54272 (up to four 32-row query
 * blocks per kv head) or 74752 (more), e.g. 12 000 tokens of which a quarter is kept; refused with FC_EUNSUPPORTED
 * otherwise.  A row whose kept count does not exceed the window (n_kept comes from device memory) is left untouched.  Replaces, for SnapKVPress, the per-sequence loop of
 * LlavaModelRunner.compress_kv_cache_batch (nanovllm/engine/llava_model_runner.py:745-786).
 */
int fc_snapkv_press(const fc_kv_view* keys, const fc_kv_view* values, const void* queries, const float* lse,
                    int32_t num_q_heads, int32_t window, int32_t kernel_size, int32_t causal_window, float scale,
                    float out_scale, float* scores, int32_t score_stride, float* row_max, int32_t k,
                    const int32_t* n_kept, int32_t* indices, int32_t index_stride, void* stream);

/*
 * The same scores with every (layer, sequence, kv head) column cut into `nsplit` key ranges, one workgroup each:
 * statistics of the pieces, their merge, per-key sums of the pieces, then the moving average across the pieces'
 * borders.  For launches with too few columns to fill the GPU (one long prompt of a model with few kv heads:
 * 288 columns of 32768 keys -32 % with 8 pieces); with 1000 or more columns one workgroup per column is faster.
 * lse: optional log-sum-exp of the window queries as for fc_snapkv_score_lse (NULL = computed here).
 * Needs a dense view or pages of 64*2^n tokens.
 * workspace: fc_snapkv_split_workspace_bytes bytes.  No counterpart in the reference (same call sites as
 * fc_snapkv_score).
 */
int64_t fc_snapkv_split_workspace_bytes(int32_t num_layers, int32_t batch, int32_t num_q_heads,
                                        int32_t num_kv_heads, int32_t window, int32_t score_stride, int32_t nsplit);
int fc_snapkv_score_split(const fc_kv_view* keys, const void* queries, const float* lse, int32_t num_q_heads,
                          int32_t window, int32_t kernel_size, int32_t causal_window, float scale, float out_scale,
                          float* scores, int32_t score_stride, float* row_max, int32_t nsplit, void* workspace,
                          int64_t workspace_bytes, void* stream);

/*
 * Sets the window entries scores[l][b][h][S_b-W .. S_b) to the maximum over
 * scores[l][:, :, :S_b-W] of the same layer, the way kvpress pads the observation window
 * back in (F.pad(value=scores.max())) so that it always survives selection.
 * row_max (optional): the per-row maxima written by fc_snapkv_score, which save the scan.
 */
int fc_snapkv_fill_window(float* scores, int32_t score_stride, int32_t num_layers, int32_t batch,
                          int32_t num_kv_heads, const int32_t* seq_lens, int32_t max_seq_len,
                          int32_t window, const float* row_max, void* stream);

/*
 * Row-wise top-k with a defined order.  Row r of `rows` score rows has
 * row_lens[(r / rows_per_len) % row_lens_mod] valid entries (row_lens == NULL: `len`) and keeps
 * n_kept[(r / rows_per_len) % row_lens_mod] of them (n_kept == NULL: `k`); for rows ordered
 * (layer, b, head) that is rows_per_len = heads, row_lens_mod = batch.  The kept scores are the
 * largest ones, ties broken towards the lowest index; their indices are written in ASCENDING
 * index order to indices[r*index_stride ...].  NaN sorts above +inf, -0 equals +0 (torch.topk's order).
 * Replaces scores.topk(n_kept).indices of kvpress.ScorerPress.compress (third-party) and
 * topk + sort of nanovllm/kernels/kvpress_compressor.py:225-226.
 */
int fc_topk_select(const float* scores, int32_t score_stride, int32_t rows, int32_t len,
                   const int32_t* row_lens, int32_t rows_per_len, int32_t row_lens_mod,
                   int32_t k, const int32_t* n_kept,
                   int32_t* indices, int32_t index_stride, void* stream);

/*
 * Knorm press in one launch: fc_knorm_score, fc_topk_select (rows of one sequence keep n_kept[b] of their
 * seq_lens[b] scores, or `k` when n_kept is NULL) and fc_compact of `keys` and `values` onto themselves, for every
 * (layer, b, kv head) column, with the same scores, indices (entries past a row's kept count are left as they are)
 * and cache bytes as those three calls.  A column's scores and kept positions stay in LDS: views with
 * 4 * (max_seq_len + index_stride) > 147456 bytes are refused with FC_EUNSUPPORTED and take the three calls.
 * Replaces, for KnormPress, the per-sequence loop extract -> press -> write back of
 * LlavaModelRunner.compress_kv_cache_batch (nanovllm/engine/llava_model_runner.py:745-786) with
 * kvpress KnormPress.score + ScorerPress.compress (third-party) inside.
 */
int fc_knorm_press(const fc_kv_view* keys, const fc_kv_view* values, float* scores, int32_t score_stride, int32_t k,
                   const int32_t* n_kept, int32_t* indices, int32_t index_stride, void* stream);

/*
 * Selection and in-place compaction in one launch, from scores that a scoring entry point wrote: for every
 * (layer, b, kv head) row of scores[.., score_stride], fc_topk_select over the row's first seq_lens[b] entries
 * (keeping n_kept[b], or `k` when n_kept is NULL) and fc_compact of `keys` and `values` onto themselves with the row's
 * own indices, with the same indices (entries past a row's kept count are left as they are) and cache bytes as those
 * two calls.  Views with 4 * (max_seq_len + index_stride) > 147456 bytes (the column's scores and kept positions stay
 * in LDS) are refused with FC_EUNSUPPORTED and take the two calls.
 * Replaces scores.topk + gather of kvpress ScorerPress.compress (third-party) together with
 * LlavaModelRunner._write_compressed_kv_cache_fast (nanovllm/engine/llava_model_runner.py:874-912).
 */
int fc_select_compact(const fc_kv_view* keys, const fc_kv_view* values, const float* scores, int32_t score_stride,
                      int32_t k, const int32_t* n_kept, int32_t* indices, int32_t index_stride, void* stream);

/*
 * Gather + compaction.  For each (layer, b, kv head): dst token j <- src token
 * indices[(l*batch + b)*heads_in_index + (h % heads_in_index)][j] for j < n_kept[b] (or k).
 * `dst` may alias `src` (same pool, same tables): indices must then be ascending, and the
 * copy is ordered so that no source row is overwritten before it is read.  When no destination view can overlap a
 * source view (one paged and one dense, or dense views with disjoint byte ranges) the rows move in no particular order.
 * Replaces keys.gather(2, idx) (nanovllm/kernels/kvpress_compressor.py:241-249) followed by
 * LlavaModelRunner._write_compressed_kv_cache_fast (llava_model_runner.py:874-912), and the
 * generated sparse_gather kernel (nanovllm/autocompress/kernels.py:321-346).
 * Slots at and beyond n_kept keep their previous contents, as in the reference.
 */
int fc_compact(const fc_kv_view* src_k, const fc_kv_view* src_v,
               const fc_kv_view* dst_k, const fc_kv_view* dst_v,
               const int32_t* indices, int32_t index_stride, int32_t heads_in_index,
               int32_t k, const int32_t* n_kept, void* stream);

/*
 * CCM three-layer MLP compressor over one token segment.
 *   y = W3 relu(W2 relu(W1 x + b1) + b2) + b3,  x = concat of `cf` consecutive tokens of one head,
 *   rounded to the storage dtype after every Linear (fp32 accumulation).
 * Weights are nn.Linear layout [out][in] in the storage dtype, stacked over layers:
 *   w1 [L][128][cf*128], w2/w3 [L][128][128], b1/b2/b3 [L][128].
 * For each (layer, b, head): rows j < c = seg_len/cf read src tokens [seg_start + cf*j, +cf)
 * and write dst token dst_start + j; the seg_len - c*cf remainder tokens are copied to
 * dst_start + c + i.  `dst` may alias `src` when dst_start <= seg_start.
 * Replaces KVCacheLinearDecoupleCompressor.compress_layer (utils_ccm/module_ccm_v11.py:666-694),
 * KVCacheHybridCompressor.compress_layer (:883-925), BatchedGEMMCompressor._compress_batched
 * (nanovllm/kernels/batched_compress.py:361-440) and its Triton kernel (:31-122).
 */
typedef struct fc_mlp_weights {
  const void* w1; const void* b1;
  const void* w2; const void* b2;
  const void* w3; const void* b3;
} fc_mlp_weights;

int fc_ccm_mlp(const fc_kv_view* src, const fc_kv_view* dst, const fc_mlp_weights* w,
               int32_t cf, int32_t seg_start, int32_t seg_len, int32_t dst_start, void* stream);

/*
 * The same compressor when every sequence has its own segment (a batch of prompts of different lengths compressed in
 * one pass instead of the reference's per-sequence loop, nanovllm/engine/llava_model_runner.py:745-786):
 * seg_start[b], seg_len[b], dst_start[b] are int32 arrays of `batch` entries in DEVICE memory.  Per sequence:
 * c = seg_len[b] / cf rows; with c < min_rows the segment is copied through unchanged (the min_seq_len guard of
 * compress_layer, module_ccm_v11.py:674-675), otherwise rows j < c go to dst_start[b] + j and the remainder tokens
 * behind them.  max_seg_len bounds every seg_len[b] (it sizes the launch); values read from the arrays are cut to
 * the views' max_seq_len on the device.  `dst` may alias `src` when dst_start[b] <= seg_start[b] for every b.
 */
int fc_ccm_mlp_ragged(const fc_kv_view* src, const fc_kv_view* dst, const fc_mlp_weights* w, int32_t cf,
                      const int32_t* seg_start, const int32_t* seg_len, const int32_t* dst_start,
                      int32_t max_seg_len, int32_t min_rows, void* stream);

/*
 * Expected-attention scores: attention each key can expect from future queries whose distribution is
 * Gaussian with mean mean_query[layer][b][hq][128] and covariance cov_query[layer][b][hq][128][128]
 * (fp32, contiguous; cov_query may be NULL = mean only).  For the keys past the first n_sink of a sequence
 *   z[hq][s] = mean . k_s / sqrt(128) + k_s^T cov k_s / (2 * 128),   p = softmax over those keys,
 *   scores[layer][b][hk][s] = (mean over the query heads of group hk of p[.][s] + epsilon) * ||v_s||_2
 * (without use_vnorm: the group mean alone); the first n_sink keys get the largest score of their layer;
 * entries past a sequence's length are -inf.  fp16 / bf16 caches; scores fp32 with row stride
 * score_stride >= max_seq_len.  workspace: fc_expected_attention_workspace_bytes bytes.
 * Replaces ExpectedAttentionPress.score of the kvpress package as the reference uses it
 * (utils_ccm/utils_compress.py:22-24, 315-316, 338-340); the query statistics themselves are computed by
 * the host from the attention module's q_proj (model code, not part of the library).
 */
int64_t fc_expected_attention_workspace_bytes(int32_t num_layers, int32_t batch, int32_t num_q_heads,
                                              int32_t max_seq_len);
int fc_expected_attention_score(const fc_kv_view* keys, const fc_kv_view* values, const float* mean_query,
                                const float* cov_query, int32_t num_q_heads, int32_t n_sink, int32_t use_vnorm,
                                float epsilon, float* scores, int32_t score_stride, void* workspace,
                                int64_t workspace_bytes, void* stream);

/*
 * Observed-attention scores from a materialised attention matrix attn[batch][num_q_heads][sq][sk]
 * (fp32 / fp16 / bf16, contiguous):
 *   scores[b][hk][s] = mean over the query heads of kv group hk of (sum_q attn[b][h][q][s]) / (sk - s),
 * fp32, contiguous [batch][num_kv_heads][sk].  workspace: fc_observed_attention_workspace_bytes bytes.
 * Replaces ObservedAttentionPress.score of the kvpress package as the reference uses it
 * (utils_ccm/utils_compress.py:22-24, 302-349).
 */
int64_t fc_observed_attention_workspace_bytes(int32_t batch, int32_t num_kv_heads, int32_t sk);
int fc_observed_attention_score(const void* attn, int32_t batch, int32_t num_q_heads,
                                int32_t num_kv_heads, int32_t sq, int32_t sk, int32_t dtype,
                                float* scores, void* workspace, int64_t workspace_bytes, void* stream);

/*
 * One Linear layer on dense row-major matrices: y[m][n] = act(x[m][k] * weight^T + bias), weight
 * in nn.Linear layout [n][k], fp16 or bf16 throughout, fp32 accumulation, one rounding to the
 * storage dtype.  bias may be NULL; apply_relu != 0 clamps at zero.  k must be a multiple of 16,
 * n of 32, ldx (row stride of x in elements) of 8; x and weight 16-byte aligned.
 * Replaces fused_linear_relu_dropout in inference mode (nanovllm/kernels/fused_compress.py:21-178)
 * and the generated per-layer kernel mlp_layer_kernel (nanovllm/autocompress/kernels.py:177-222).
 */
int fc_linear_act(const void* x, int64_t ldx, const void* weight, const void* bias, void* y,
                  int64_t ldy, int64_t m, int32_t n, int32_t k, int32_t dtype, int32_t apply_relu,
                  void* stream);

/*
 * Symmetric per-row quantisation: for each of `rows` rows of `d` elements,
 *   scale = clamp(max|x| / qmax, min=1e-8), q = clamp(round_half_even(x / scale), -qmax-1, qmax),
 * qmax = 2^(bits-1) - 1, q stored as int8 (also for bits = 4), scale in the dtype of x; every
 * intermediate is rounded to that dtype as an eager tensor expression would.  And the inverse,
 * out = q * scale rounded to out_dtype (= scale_dtype, or fp32 for an fp16/bf16 scale).
 * Replaces the quantize / dequantize pair of nanovllm/autocompress/kernels.py:387-421.
 */
int fc_quantize_rows(const void* x, int64_t rows, int32_t d, int32_t dtype, int32_t bits,
                     int8_t* q, void* scale, void* stream);
int fc_dequantize_rows(const int8_t* q, const void* scale, int64_t rows, int32_t d,
                       int32_t scale_dtype, int32_t out_dtype, void* out, void* stream);

/* Quantise and dequantise in one pass ("fake quantisation"), x and y [rows][d] contiguous in `dtype`:
 *   scale = max|x| / (2^(bits-1) - 1), per row or (per_tensor != 0) over the whole tensor;
 *   y = clamp(round(x / scale), -2^(bits-1), 2^(bits-1) - 1) * scale,
 * every step rounded to `dtype` as the eager tensor expression does, no floor on the scale (a zero
 * row gives NaN, as there).  scale / absmax: optional outputs in `dtype`, [rows] or [1].  The
 * whole-tensor form needs a workspace of fc_fake_quantize_workspace_bytes().  x == y is allowed.
 * Replaces SimpleKVQuantizer._quantize_tensor (utils_ccm/utils_compress.py:144-154, whole-tensor
 * scale) and ImprovedKVQuantizer._quantize_tensor_with_params (utils_compress.py:51-70, per row). */
int64_t fc_fake_quantize_workspace_bytes(void);
int fc_fake_quantize(const void* x, void* y, int64_t rows, int32_t d, int32_t dtype, int32_t bits,
                     int32_t per_tensor, void* scale, void* absmax, void* workspace, int64_t workspace_bytes,
                     void* stream);

/*
 * Key-channel statistics and pruning for the ThinK press (kvpress.ThinKPress, which the reference registers at
 * nanovllm/autocompress/methods.py:422 and constructs at :432-436):
 *   energy[l][b][h][d] = sum over the tokens s < len(b) of keys[l][b][h][s][d]^2   (fp32, [L][B][Hkv][128]);
 *   fc_key_channel_zero sets keys[l][b][h][s][d] = 0 for every token of the sequence and every channel d with
 *   prune[l][b][h][d] != 0 (uint8, [L][B][Hkv][128]), in place.
 * The press multiplies the energies with those of the window queries, picks the channels and calls the second.
 */
int fc_key_channel_energy(const fc_kv_view* keys, float* energy, void* stream);
int fc_key_channel_zero(const fc_kv_view* keys, const uint8_t* prune, void* stream);

/*
 * 8-bit floating point codes with one scale for the whole tensor of n elements:
 *   scale = clamp(max|x| / 448, min=1e-8) (448 for both formats, as the reference has it), code = fp8(x / scale),
 * e5m2 == 0: E4M3, finite-only variant (largest value 448, 0x7f = NaN); e5m2 != 0: E5M2; conversion rounds to
 * nearest even from the quotient rounded to `dtype`.  scale: one element in `dtype`.  Workspace as for
 * fc_fake_quantize.  And the inverse, out = float(code) * scale rounded to out_dtype (dtype rules of
 * fc_dequantize_rows).  Replaces QuantizationMethod._quantize_fp8 and the fp8 branch of dequantize
 * (nanovllm/autocompress/methods.py:671-680, 735-736).
 */
int fc_quantize_fp8(const void* x, int64_t n, int32_t dtype, int32_t e5m2, uint8_t* q, void* scale,
                    void* workspace, int64_t workspace_bytes, void* stream);
int fc_dequantize_fp8(const uint8_t* q, const void* scale, int64_t n, int32_t e5m2, int32_t scale_dtype,
                      int32_t out_dtype, void* out, void* stream);

/*
 * Asymmetric 8-bit quantisation of rows of `d` elements:
 *   scale = clamp((max - min) / 255, min=1e-8), zero = clamp(round(-min / scale), 0, 255),
 *   q = clamp(round((x - min) / scale), 0, 255) as uint8; params[row] = (scale, zero) in the dtype of x;
 * every intermediate rounded to that dtype.  Replaces the symmetric=False branch of
 * QuantizationMethod._quantize_int8 (nanovllm/autocompress/methods.py:644-651).
 */
int fc_quantize_rows_asym(const void* x, int64_t rows, int32_t d, int32_t dtype, uint8_t* q, void* params,
                          void* stream);

/*
 * 4-bit quantisation of groups of `group_size` consecutive elements, two codes per byte (element 2j in
 * the low nibble), one scale per group in the dtype of x.
 *   nf4 == 0: scale = clamp(max|x| / 7, 1e-8), code = clamp(round(x / scale), -8, 7) + 8;
 *   nf4 != 0: scale = clamp(max|x|, 1e-8), code = index of the nearest of the 16 NF4 levels.
 * De-quantisation: out = level * scale with level = code - 8, or the NF4 level rounded to table_dtype;
 * the output dtype is the promotion of table_dtype and scale_dtype.
 * Replaces QuantizationMethod._quantize_int4 / _quantize_nf4 / dequantize
 * (nanovllm/autocompress/methods.py:654-734).
 */
int fc_quantize_group4(const void* x, int64_t groups, int32_t group_size, int32_t dtype, int32_t nf4,
                       uint8_t* packed, void* scale, void* stream);
int fc_dequantize_group4(const uint8_t* packed, const void* scale, int64_t groups, int32_t group_size,
                         int32_t scale_dtype, int32_t table_dtype, int32_t nf4, void* out, void* stream);

/*
 * Plain ordered token copy src[seg_start + i] -> dst[dst_start + i], i < count, per
 * (layer, b, head); the pass-through branch of compress_layer when seg_len/cf < min_seq_len
 * (module_ccm_v11.py:674-675).  dst may alias src when dst_start <= seg_start and both views are of one kind
 * (both paged or both dense): the rows then move in ascending order.  A paged and a dense view must not overlap; they,
 * and two dense views whose byte ranges are disjoint, are copied in no particular order (short-lived workgroups, the
 * fastest form of a copy on this part).
 */
int fc_copy_tokens(const fc_kv_view* src, const fc_kv_view* dst,
                   int32_t seg_start, int32_t count, int32_t dst_start, void* stream);

/*
 * The same copy from a source whose layers are tensors of their own (the list of per-layer (K, V) tensors a
 * HuggingFace-style compressor returns): src_layers[l] (a table of src->num_layers addresses in DEVICE memory) is the
 * address of layer l's tensor, all of the one geometry `src` describes (dense, its base = the address of layer 0, its
 * stride_layer unused).  Replaces the per-layer loop of LlavaModelRunner._write_compressed_kv_cache_fast
 * (nanovllm/engine/llava_model_runner.py:874-912) without first stacking the layers into one tensor.
 */
int fc_copy_tokens_from_layers(const void* const* src_layers, const fc_kv_view* src, const fc_kv_view* dst,
                               int32_t seg_start, int32_t count, int32_t dst_start, void* stream);

/*
 * Append one new K/V row per sequence: cache[block_tables[b][len_b / bs]][len_b % bs] <- k_new[b], v_new[b]
 * for every layer in the views (k_new/v_new: [num_layers][batch][num_kv_heads][head_dim]).
 * The slot is computed on the device from context_lens so that the call can be replayed in a graph.
 * Replaces store_kvcache (nanovllm/layers/attention.py:10-39) + the slot computation of
 * LlavaModelRunner.prepare_decode (llava_model_runner.py:655-665).
 * Rows with context_lens[b] < 0 are skipped.
 */
int fc_store_kv(const fc_kv_view* k_cache, const fc_kv_view* v_cache,
                const void* k_new, const void* v_new, const int32_t* context_lens, void* stream);

/*
 * The same append with host-computed slots: for token i < num_tokens,
 *   k_cache[slot_mapping[i]] <- key[i], v_cache[slot_mapping[i]] <- value[i],
 * a row being row_elems = num_kv_heads*head_dim contiguous elements; key/value rows are
 * key_stride/value_stride elements apart; k_cache/v_cache are one layer's planes viewed as
 * [num_blocks*block_size][row_elems].  Negative slots are skipped.
 * Replaces store_kvcache(key, value, k_cache, v_cache, slot_mapping) (nanovllm/layers/attention.py:32-39).
 */
int fc_store_kv_slots(const void* key, int64_t key_stride, const void* value, int64_t value_stride,
                      void* k_cache, void* v_cache, const int32_t* slot_mapping, int32_t num_tokens,
                      int32_t row_elems, int32_t dtype, void* stream);

/* context_lens[b] += delta for b < batch where context_lens[b] >= 0 (device side, graph-replayable). */
int fc_advance_lens(int32_t* context_lens, int32_t batch, int32_t delta, void* stream);

/*
 * Decode paged attention, one query token per sequence, for ONE layer `layer` of the views:
 *   o[b][hq] = softmax_fp32(q[b][hq] . K[b][:len_b][hq/G]^T * scale) V[b][:len_b][hq/G]
 * q, out: [batch][num_q_heads][head_dim] in the cache dtype (fp16/bf16).  context_lens[b] is the number
 * of cached tokens attended (rows with context_lens[b] <= 0 produce zeros).
 * Replaces flash_attn_with_kvcache(q, k_cache, v_cache, cache_seqlens, block_table, softmax_scale,
 * causal=True) at nanovllm/layers/attention.py:75-77.
 * workspace: fc_decode_attn_workspace_bytes(batch, num_q_heads, max_splits) bytes, 256-byte aligned.
 */
int64_t fc_decode_attn_workspace_bytes(int32_t batch, int32_t num_q_heads, int32_t max_seq_len);
int fc_decode_attn(const fc_kv_view* k_cache, const fc_kv_view* v_cache, int32_t layer,
                   const void* q, void* out, int32_t num_q_heads, const int32_t* context_lens,
                   float scale, void* workspace, int64_t workspace_bytes, void* stream);

/*
 * fc_decode_attn for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc): the chunk partials go to a buffer built into the library, a
 * file-scope device array of fc_decode_attn_static_capacity() bytes (16 MiB) that every GPU the library runs on
 * holds until the process ends.  No counterpart in the reference.  Same arguments and results as fc_decode_attn
 * minus the workspace; the call allocates nothing and frees nothing.  Shapes whose
 * fc_decode_attn_workspace_bytes() exceed the capacity are rejected with FC_EUNSUPPORTED.  All calls on one GPU
 * share the one buffer: calls that overlap on a GPU (different streams, concurrent graphs) race; calls on one
 * stream are ordered and safe.  Nothing in the buffer has to start at zero, so no clearing is done.
 * With FC_STATIC_GUARD=1 in the environment (read once) the call remembers the stream of the previous call on the
 * device and returns FC_EINVAL when another stream calls while that one still has work pending (it queries the
 * previous stream, so leave the variable unset while streams are being captured).
 */
int64_t fc_decode_attn_static_capacity(void);
int fc_decode_attn_static(const fc_kv_view* k_cache, const fc_kv_view* v_cache, int32_t layer,
                          const void* q, void* out, int32_t num_q_heads, const int32_t* context_lens,
                          float scale, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FASTCACHE_HIP_H */
