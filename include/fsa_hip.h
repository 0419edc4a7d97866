/*
 * fsa_hip.h - C ABI of libfsa_gfx950.so: NSA selected attention (and the
 * kernels around it) as hand-written HIP kernels for gfx950 (MI355X).
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless the name ends in _host;
 *   - the library never allocates, frees or synchronises: outputs and
 *     workspaces are passed in, kernels are enqueued on `stream`
 *     (a hipStream_t passed as void*; NULL = the default stream);
 *   - return value: 0 = ok, < 0 = invalid argument (see fsa_last_error()),
 *     > 0 = a hipError_t from a launch;
 *   - dtype codes: FSA_BF16 / FSA_FP16 for q, k, v, o and gradients;
 *   - strides are in ELEMENTS; the innermost (head_dim) stride is 1; token
 *     and head strides are non-negative, a token stride and the span of one kv
 *     head's group of q heads stay below 2^31 elements, and the dense
 *     (compressed / window) kernels need 64 rows of k or v within 4 GiB -
 *     anything else is an invalid-argument error, nothing is launched;
 *   - block ids inside topk_idx are local to the query's sequence, -1 = padding.
 *
 * The packed varlen layout is the reference's: q[N,Hq,D], k/v[N,Hkv,D],
 * topk_idx[Hkv,N,T] int32, cu_seqlens[B+1] int32, lse[Hq,N] fp32 base 2
 * (fsa/ops/FSA_topk_sparse_attention.py:1887-1932).
 */
#ifndef FSA_HIP_H
#define FSA_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FSA_BF16 0
#define FSA_FP16 1

#define FSA_ERR_INVALID (-1)
#define FSA_ERR_UNSUPPORTED (-2)
#define FSA_ERR_WORKSPACE (-3)

/* Library version (major*10000 + minor*100 + patch).  A caller built against an
 * older header must check it at load: argument lists changed at
 *   200: fsa_decode_topk (scores_to_bf16 added), fsa_decode_selattn (seqlens added);
 *   210: fsa_cmp_topk (score_head_as_written added); fsa_native_head_dim and
 *        fsa_pad_head_dim are new. */
#define FSA_HIP_VERSION 210
int fsa_version(void);
/* Human-readable description of the last error on the calling thread. */
const char* fsa_last_error(void);

/* Head dims other than 64 / 128 / 256.  The kernels are built for those three;
 * the reference pads any head_dim <= 256 to the next power of two inside its
 * kernels (fsa/ops/FSA_topk_sparse_attention.py:692, 760, 904, 1456).  Here the
 * caller runs the kernels on zero-padded copies: q.k and P.V are unchanged by
 * zero columns, the softmax scale must be passed explicitly (1/sqrt of the TRUE
 * head_dim), and the padded columns of outputs and gradients are cut off again.
 *   fsa_native_head_dim(d): the built size to pad to (d itself if built), -1 if d > 256;
 *   fsa_pad_head_dim: dst[r, h, 0..d_dst) = src[r, h, 0..min(d_src, d_dst)) then
 *   zeros, for 16-bit elements - pads (d_dst > d_src) and cuts (d_dst < d_src);
 *   strides in elements, multiples of 4, d_dst a multiple of 4. */
int fsa_native_head_dim(int32_t head_dim);
int fsa_pad_head_dim(const void* src, int64_t src_stride_n, int64_t src_stride_h, int32_t d_src,
                     void* dst, int64_t dst_stride_n, int64_t dst_stride_h, int32_t d_dst,
                     int64_t rows, int32_t heads, void* stream);

/* Per-kernel timing for benchmarks (replaces the CUDA-event timer of
 * utils.py:6-27).  While enabled, every kernel launch of the library is
 * bracketed by HIP events on its stream; fsa_profile_get waits for record i and
 * returns its label and duration in milliseconds.  fsa_profile_enable(0 or 1)
 * also discards the records collected so far. */
int fsa_profile_enable(int on);
int fsa_profile_count(void);
int fsa_profile_get(int i, char* name, int name_cap, float* ms);

/* ------------------------------------------------------------------------
 * Inverted block->query index.
 * Replaces: torch.bincount + build_block_to_token_triton + boolean compaction
 * + cumsum/pad + index_mapping (fsa/ops/FSA_topk_sparse_attention.py:951-955,
 * 59-135, 1016-1026, 621-668) and reorder_topk_idx
 * (nsa_ref/ops/topk_sparse_attention.py:412-476), for all sequences and kv
 * heads in one call.
 *
 * Global block id of block b of sequence s: cu_blocks[s] + b with
 * cu_blocks = cumsum(ceil(len_s / block_size)).  max_blocks is any upper bound
 * of cu_blocks[batch] known on the host, e.g. ceil(N / block_size) + batch.
 *
 *   cu_blocks  [batch+1]               out
 *   counts     [Hkv, max_blocks]       out  entries per block
 *   starts     [Hkv, max_blocks+1]     out  exclusive prefix of counts
 *   sel_tokens [Hkv, N*T]              out  global query rows grouped by block,
 *                                           ascending inside a block; -1 tail
 *   slot_of    [Hkv, N, T]             out  position of (query, slot) in
 *                                           sel_tokens, -1 for padding
 * ---------------------------------------------------------------------- */
size_t fsa_index_workspace_bytes(int64_t total_tokens, int32_t topk, int32_t num_kv_heads,
                                 int64_t max_blocks);

int fsa_build_index(const int32_t* topk_idx, int64_t topk_stride_h, int64_t topk_stride_n,
                    const int32_t* cu_seqlens, int32_t batch, int64_t total_tokens,
                    int32_t num_kv_heads, int32_t topk, int32_t block_size, int64_t max_blocks,
                    int32_t* cu_blocks, int32_t* counts, int32_t* starts, int32_t* sel_tokens,
                    int32_t* slot_of, void* workspace, size_t workspace_bytes, void* stream);

/* Block lists over blocks of `block_size` keys rewritten as lists over blocks
 * of block_size / factor keys: entry (t, j) of the output is
 * topk_idx[t] * factor + j when that sub-block starts at or before the query's
 * position in its sequence, otherwise -1; out is contiguous
 * [Hkv, N, T * factor].  Attention over the selected blocks is attention over
 * the union of their keys, so the result is the same operator at a block size
 * the kernels are built for: this is how block_size 256, which the reference
 * accepts (fsa/ops/FSA_topk_sparse_attention.py:926), runs on the 128-key
 * kernels.  No counterpart in the reference. */
int fsa_split_topk_blocks(const int32_t* topk_idx, int64_t topk_stride_h, int64_t topk_stride_n,
                          const int32_t* cu_seqlens, int32_t batch, int64_t total_tokens,
                          int32_t num_kv_heads, int32_t topk, int32_t block_size, int32_t factor,
                          int32_t* out, void* stream);

/* Work list for the block-major kernels: tile_prefix[h, gb] = number of
 * row tiles of blocks < gb, a row tile being `rows_per_tile` gathered
 * (query, head-in-group) rows of one block.  tile_prefix is [Hkv, max_blocks+1].
 * Replaces the rectangular grids with early exit of
 * fsa/ops/FSA_topk_sparse_attention.py:758-821. */
int fsa_build_tiles(const int32_t* counts, int32_t num_kv_heads, int64_t max_blocks,
                    int32_t group_size, int32_t rows_per_tile, int32_t* tile_prefix, void* stream);

/* Upper bound of the number of row tiles per kv head (host arithmetic only). */
int64_t fsa_max_tiles(int64_t total_tokens, int32_t topk, int32_t group_size, int32_t rows_per_tile,
                      int64_t max_blocks);

/* ------------------------------------------------------------------------
 * Selected attention forward.
 * Replaces _topk_sparse_attention_fwd_opt (online_softmax/qk_kernel,
 * qkv_kernel/forward_kernel_opt, reduce_output/reduce_kernel;
 * fsa/ops/FSA_topk_sparse_attention.py:569-618, 671-907, 910-1116).
 *
 * Stage 1 (block-major): for every kv block, the queries that selected it are
 * gathered into MFMA tiles; a normalised partial O row and its base-2 LSE are
 * written per (query, block, head):
 *     o_part   [Hkv, N*T, g, D]   same dtype as q
 *     lse_part [Hkv, N*T, g]      fp32
 * Stage 2 (query-major): the <= T partials of each (query, head) are merged.
 * The workspace holds o_part, lse_part and the tile list.
 * ---------------------------------------------------------------------- */
size_t fsa_selattn_fwd_workspace_bytes(int64_t total_tokens, int32_t num_q_heads, int32_t num_kv_heads,
                                       int32_t head_dim, int32_t topk, int64_t max_blocks);

int fsa_selattn_fwd(const void* q, const void* k, const void* v, int32_t dtype,
                    int64_t q_stride_n, int64_t q_stride_h, int64_t k_stride_n, int64_t k_stride_h,
                    int64_t v_stride_n, int64_t v_stride_h,
                    const int32_t* cu_seqlens, int32_t batch, int64_t total_tokens,
                    int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim, int32_t topk,
                    int32_t block_size, int64_t max_blocks, float softmax_scale,
                    const int32_t* cu_blocks, const int32_t* counts, const int32_t* starts,
                    const int32_t* sel_tokens, const int32_t* slot_of,
                    void* o, int64_t o_stride_n, int64_t o_stride_h, float* lse /* [Hq, N] */,
                    void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------
 * Selected attention backward.
 * Replaces _topk_sparse_attention_bwd_opt (backward_sum_o_do, backward_dkdv,
 * dq_compute_kernel, dq_reduce_kernel; fsa/ops/FSA_topk_sparse_attention.py:
 * 1715-1884, 1119-1321, 1547-1712; nsa_ref/ops/topk_sparse_attention.py:197-230).
 * dq has q's layout, dk/dv have k's layout (already summed over the g heads
 * of a group).  All outputs are fully overwritten.
 * ---------------------------------------------------------------------- */
size_t fsa_selattn_bwd_workspace_bytes(int64_t total_tokens, int32_t num_q_heads, int32_t num_kv_heads,
                                       int32_t head_dim, int32_t topk, int32_t block_size,
                                       int64_t max_blocks);

int fsa_selattn_bwd(const void* q, const void* k, const void* v, const void* o, const void* d_o,
                    const float* lse, int32_t dtype,
                    int64_t q_stride_n, int64_t q_stride_h, int64_t k_stride_n, int64_t k_stride_h,
                    int64_t v_stride_n, int64_t v_stride_h, int64_t o_stride_n, int64_t o_stride_h,
                    int64_t do_stride_n, int64_t do_stride_h,
                    const int32_t* cu_seqlens, int32_t batch, int64_t total_tokens,
                    int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim, int32_t topk,
                    int32_t block_size, int64_t max_blocks, float softmax_scale,
                    const int32_t* cu_blocks, const int32_t* counts, const int32_t* starts,
                    const int32_t* sel_tokens, const int32_t* slot_of,
                    void* dq, void* dk, void* dv /* contiguous [N,H,D] */,
                    void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------
 * Compressed attention: every query against the compressed keys / values of
 * its sequence; compressed key j is visible to the query at sequence-local
 * position i iff i >= j*kernel_stride + kernel_size - 1.  Queries without a
 * visible key get O = 0, LSE = -inf.
 * Replaces CompressedAttention / _compressed_attention_fwd / _bwd and their
 * kernels (nsa_ref/ops/compressed_attention.py:27-518, 521-829).
 * ck / cv are [total_k, Hkv, D] with cu_seqlens_k [batch+1]; lse is [Hq, total_q]
 * fp32 base 2; dq is contiguous [total_q, Hq, D], dck / dcv contiguous
 * [total_k, Hkv, D].  max_seqlen_q is any upper bound of the longest sequence.
 * ---------------------------------------------------------------------- */
int fsa_cmpattn_fwd(const void* q, const void* ck, const void* cv, int32_t dtype,
                    int64_t q_stride_n, int64_t q_stride_h, int64_t k_stride_n, int64_t k_stride_h,
                    int64_t v_stride_n, int64_t v_stride_h,
                    const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k, int32_t batch,
                    int64_t total_q, int64_t max_seqlen_q, int32_t num_q_heads, int32_t num_kv_heads,
                    int32_t head_dim, int32_t kernel_size, int32_t kernel_stride, float softmax_scale,
                    void* o, int64_t o_stride_n, int64_t o_stride_h, float* lse, void* stream);

size_t fsa_cmpattn_bwd_workspace_bytes(int64_t total_q, int64_t total_k, int64_t max_seqlen_q,
                                       int32_t batch, int32_t num_q_heads, int32_t num_kv_heads,
                                       int32_t head_dim);

int fsa_cmpattn_bwd(const void* q, const void* ck, const void* cv, const void* o, const void* d_o,
                    const float* lse, int32_t dtype,
                    int64_t q_stride_n, int64_t q_stride_h, int64_t k_stride_n, int64_t k_stride_h,
                    int64_t v_stride_n, int64_t v_stride_h, int64_t o_stride_n, int64_t o_stride_h,
                    int64_t do_stride_n, int64_t do_stride_h,
                    const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k, int32_t batch,
                    int64_t total_q, int64_t total_k, int64_t max_seqlen_q,
                    int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                    int32_t kernel_size, int32_t kernel_stride, float softmax_scale,
                    void* dq, void* dck, void* dcv, void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------
 * Top-k block selection from the compressed-attention probabilities.
 * Replaces _get_attention_score / score_kernel, transform_score /
 * _transform_score_kernel and the torch.topk + sort + mask of
 * nsa_ref/ops/compressed_attention.py:832-1003, 1006-1158, 1272-1315
 * (per kv head, probabilities of the FIRST q head of the group; with
 * score_head_as_written != 0 kv head kh is scored with q head kh instead, which
 * is what the reference's parallel_topk_compute=True path does when it hands
 * the unsliced q to score_kernel, compressed_attention.py:870, 898, 906).
 *   topk_idx    [Hkv, total_q, min(topk, nblk)] int32 out, nblk = ceil(max_seqlen_q / block_size)
 *   block_score [Hkv, total_q, nblk] fp32 out, optional (NULL to skip)
 * scores_to_bf16 != 0 rounds the block scores to bf16 before the selection, as
 * the reference's per-head path does.  Equal scores are ordered by lower block id.
 * The workspace holds the fp32 probabilities, max_seqlen_k columns per query and
 * kv head.  With kernel_size == 2 * kernel_stride and block_size == 4 * kernel_stride
 * the block scores are formed where the probabilities are computed and only
 * they are stored: fsa_cmp_topk_workspace_bytes(total_q, num_kv_heads,
 * max_seqlen_k / 4 + 1) is enough then (the size for max_seqlen_k is always accepted).
 * ---------------------------------------------------------------------- */
size_t fsa_cmp_topk_workspace_bytes(int64_t total_q, int32_t num_kv_heads, int64_t max_seqlen_k);

int fsa_cmp_topk(const void* q, const void* ck, const float* lse, int32_t dtype,
                 int64_t q_stride_n, int64_t q_stride_h, int64_t k_stride_n, int64_t k_stride_h,
                 const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k, int32_t batch,
                 int64_t total_q, int64_t max_seqlen_q, int64_t max_seqlen_k,
                 int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                 int32_t kernel_size, int32_t kernel_stride, int32_t block_size, int32_t topk,
                 int32_t init_blocks, int32_t local_blocks, int32_t scores_to_bf16,
                 int32_t score_head_as_written, float softmax_scale,
                 int32_t* topk_idx, float* block_score, void* workspace, size_t workspace_bytes,
                 void* stream);

/* ------------------------------------------------------------------------
 * One-step decode: ONE new query per request, a batch of requests per call
 * (the reference handles a batch of one).  q is [B, Hq, D]; caches are packed
 * [total_rows, Hkv, D] with cu_* [B+1]; o is contiguous [B, Hq, D]; lse [Hq, B].
 *
 * fsa_decode_cmpattn replaces _compressed_attention_fwd_decode /
 * forward_kernel_decode and the score recomputation of score_kernel_decode
 * (fsa_preview/ops/compressed_attention_decode.py:15-97, 361-490, 494-592):
 * compressed key j is visible iff j*stride + ks - 1 <= pos[b].  If raw_score is
 * not NULL the unscaled q.k of the scoring head of every kv head is stored in
 * raw_score[Hkv, B, raw_ld] (raw_ld >= longest visible compressed length,
 * multiple of 4); the scoring head is the first head of the group, or - with
 * score_head_as_written - the q head whose index equals the kv head's (:560,568).
 *
 * fsa_decode_topk replaces transform_score_decode + topk (:284-357, 203-205):
 * ids ordered by descending score (equal scores by lower id), -1 where fewer
 * than topk blocks exist.  as_written = 1 reproduces the reference literally
 * (candidate blocks = ceil(compressed_len / block_size), own block taken as 0);
 * as_written = 0 uses ceil(seqlens[b] / block_size) blocks and own block
 * (seqlens[b]-1) / block_size.  scores_to_bf16 != 0 ranks the block scores after
 * rounding them to bf16, as the prefill selection of the layer does
 * (nsa_ref/ops/compressed_attention.py:1307-1308), so that a decode step picks the
 * blocks the prefill picks for the same token; the reference's decode ranks fp32
 * scores (0).  block_score is optional [Hkv, B, max_blocks] (fp32, unrounded).
 *
 * fsa_decode_selattn replaces _topk_sparse_attention_decode
 * (fsa_preview/ops/selected_attention_decode.py:8-42): the g heads of a group
 * attend every cached key of the selected blocks (ids < 0, past the cache or
 * repeated are ignored).  Request b owns rows [cu_k[b], cu_k[b+1]) of the
 * caches; seqlens (optional, [B] on the device, may be null) gives the number
 * of those rows that hold tokens, for callers that keep every request in a
 * slot of fixed capacity and let it grow (a step recorded into a HIP graph
 * stays valid while the lengths change in device memory).
 *
 * Both attention calls run a grid of single-wave work-groups that stays
 * resident for the whole launch; the key tiles of all (request, kv head) pairs
 * are dealt to the waves in equal contiguous shares, and the fp32 partials of
 * a pair are merged in a fixed order (results are reproducible for a given
 * batch; across different batches a request's output agrees up to fp32
 * rounding of the partial sums).  The caller provides a workspace of
 * fsa_decode_workspace_bytes(...) bytes (max_keys is kept for compatibility
 * and does not change the size).  max_keys of fsa_decode_cmpattn is a host
 * upper bound of the visible compressed cache of one request (keys beyond it
 * are ignored).  One launch serves up to 16 query heads per kv head; larger
 * GQA groups (and groups of 16 when score_head_as_written asks for a score
 * column of its own) are served by several launches inside the call, each of
 * which reads the keys again.
 * ---------------------------------------------------------------------- */
size_t fsa_decode_workspace_bytes(int32_t batch, int32_t num_q_heads, int32_t num_kv_heads,
                                  int32_t head_dim, int64_t max_keys);

int fsa_decode_cmpattn(const void* q, const void* ck, const void* cv, int32_t dtype,
                       int64_t q_stride_b, int64_t q_stride_h, int64_t k_stride_n, int64_t k_stride_h,
                       int64_t v_stride_n, int64_t v_stride_h, const int32_t* cu_ck, const int32_t* pos,
                       int32_t batch, int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                       int32_t kernel_size, int32_t kernel_stride, float softmax_scale,
                       int32_t score_head_as_written, int64_t max_keys, void* o, float* lse,
                       float* raw_score, int64_t raw_ld, void* workspace, size_t workspace_bytes,
                       void* stream);

int fsa_decode_topk(const float* raw_score, int64_t raw_ld, const float* lse, const int32_t* cu_ck,
                    const int32_t* pos, const int32_t* seqlens, int32_t batch, int32_t num_q_heads,
                    int32_t num_kv_heads, int32_t kernel_size, int32_t kernel_stride, int32_t block_size,
                    int32_t topk, int32_t init_blocks, int32_t local_blocks, int32_t as_written,
                    int32_t scores_to_bf16, float softmax_scale, int64_t max_blocks, int32_t* topk_idx,
                    float* block_score, void* stream);

int fsa_decode_selattn(const void* q, const void* k_cache, const void* v_cache, int32_t dtype,
                       int64_t q_stride_b, int64_t q_stride_h, int64_t k_stride_n, int64_t k_stride_h,
                       int64_t v_stride_n, int64_t v_stride_h, const int32_t* cu_k, const int32_t* seqlens,
                       const int32_t* topk_idx, int32_t batch, int32_t num_q_heads, int32_t num_kv_heads,
                       int32_t head_dim, int32_t topk, int32_t block_size, float softmax_scale, void* o,
                       float* lse, void* workspace, size_t workspace_bytes, void* stream);

/* fsa_decode_selattn for callers that cannot allocate (a step recorded into a HIP
 * graph, a serving loop with a fixed memory plan, a harness that forbids
 * allocation): same arguments and results as fsa_decode_selattn, but the partial
 * results live in a buffer of FSA_DECODE_STATIC_SCRATCH_BYTES that is part of the
 * library's code object (each device the library runs on holds its copy until the
 * process ends), and the call allocates nothing.  No counterpart in the
 * reference.  Sizes with fsa_decode_workspace_bytes(...) above the buffer are
 * refused with FSA_ERR_WORKSPACE.  All calls on one device share the buffer.
 * Eager calls are kept apart by the library: a call on another stream than the
 * previous one first waits (hipStreamWaitEvent) for that call's completion event,
 * so consecutive calls never overlap on the buffer whatever their streams; calls
 * issued from several threads at once are serialised only in their set-up, so
 * give each thread's calls an order of your own.  Calls recorded into a graph
 * take no part in that (a capturing stream cannot wait for eager work): replays
 * that overlap other calls on the device race.  The first call on a device looks
 * the buffer up (hipGetSymbolAddress) and creates the event; make it outside a
 * stream capture. */
#define FSA_DECODE_STATIC_SCRATCH_BYTES (16u << 20)
int fsa_decode_selattn_static(const void* q, const void* k_cache, const void* v_cache, int32_t dtype,
                              int64_t q_stride_b, int64_t q_stride_h, int64_t k_stride_n, int64_t k_stride_h,
                              int64_t v_stride_n, int64_t v_stride_h, const int32_t* cu_k,
                              const int32_t* seqlens, const int32_t* topk_idx, int32_t batch, int32_t num_q_heads,
                              int32_t num_kv_heads, int32_t head_dim, int32_t topk, int32_t block_size,
                              float softmax_scale, void* o, float* lse, void* stream);

/* ------------------------------------------------------------------------
 * Sliding-window attention: the query at sequence-local position i attends the
 * keys p with i - window <= p <= i of its own sequence (window + 1 keys).
 * Replaces flash_attn_varlen_func(causal=True, window_size=(window, -1)) in
 * fsa/module/fsa.py:149-159 (a third-party kernel in the reference).  Same
 * layouts as selected attention; dq contiguous [N,Hq,D], dk/dv contiguous
 * [N,Hkv,D]; max_seqlen is an upper bound of the longest sequence.
 * ---------------------------------------------------------------------- */
int fsa_winattn_fwd(const void* q, const void* k, const void* v, int32_t dtype,
                    int64_t q_stride_n, int64_t q_stride_h, int64_t k_stride_n, int64_t k_stride_h,
                    int64_t v_stride_n, int64_t v_stride_h, const int32_t* cu_seqlens, int32_t batch,
                    int64_t total_tokens, int64_t max_seqlen, int32_t num_q_heads, int32_t num_kv_heads,
                    int32_t head_dim, int32_t window, float softmax_scale, void* o, int64_t o_stride_n,
                    int64_t o_stride_h, float* lse, void* stream);

size_t fsa_winattn_bwd_workspace_bytes(int64_t total_tokens, int64_t max_seqlen, int32_t window,
                                       int32_t batch, int32_t num_q_heads, int32_t num_kv_heads,
                                       int32_t head_dim);

int fsa_winattn_bwd(const void* q, const void* k, const void* v, const void* o, const void* d_o,
                    const float* lse, int32_t dtype, int64_t q_stride_n, int64_t q_stride_h,
                    int64_t k_stride_n, int64_t k_stride_h, int64_t v_stride_n, int64_t v_stride_h,
                    int64_t o_stride_n, int64_t o_stride_h, int64_t do_stride_n, int64_t do_stride_h,
                    const int32_t* cu_seqlens, int32_t batch, int64_t total_tokens, int64_t max_seqlen,
                    int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim, int32_t window,
                    float softmax_scale, void* dq, void* dk, void* dv, void* workspace,
                    size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------
 * Rotary embedding on packed sequences (non-interleaved halves): token j of a
 * sequence sits at position start + j*stride; cos/sin are evaluated in fp32 from
 * inv_freq [D/2] (device), scaled by attention_scaling and rounded to the tensor
 * dtype before the fp32 rotation.  inverse != 0 applies the opposite rotation,
 * which is the backward of the forward.  Replaces RotaryEmbedding.forward /
 * flash_attn apply_rotary_emb (nsa_ref/module/rope.py:89-134).
 * ---------------------------------------------------------------------- */
int fsa_rope(const void* x, void* out, int32_t dtype, int64_t x_stride_n, int64_t x_stride_h,
             int64_t o_stride_n, int64_t o_stride_h, const int32_t* cu_seqlens, int32_t batch,
             int64_t total_tokens, int32_t num_heads, int32_t head_dim, const float* inv_freq,
             float attention_scaling, int32_t start, int32_t stride, int32_t inverse, void* stream);

/* ------------------------------------------------------------------------
 * Linear compression of keys / values:
 *   y[n, h, :] = sum_{k < kernel_size} x[n*kernel_stride + k, h, :] @ W[h, k]   (+ pe-bias)
 * with W = w viewed as [H, kernel_size, D, D], y_len = floor((len - ks)/stride) + 1
 * (0 if len < ks), cu_seqlens_y given by the caller.  pe [H, ks, D] is optional;
 * its contribution einsum(pe, W) is rounded to the dtype and added to the rounded
 * y, as in the reference.  Replaces linear_compress / LinearCompress and their
 * kernels (nsa_ref/ops/linear_compress.py:28-131, 135-292, 295-502); the backward
 * uses no atomics.  y / dx / dw / dpe are contiguous; bias_scratch is [H, D] of
 * the dtype, dbias_scratch [H, D] fp32.
 * ---------------------------------------------------------------------- */
int fsa_linear_compress_fwd(const void* x, const void* w, const void* pe, int32_t dtype,
                            int64_t x_stride_n, int64_t x_stride_h, const int32_t* cu_seqlens_x,
                            const int32_t* cu_seqlens_y, int32_t batch, int64_t max_seqlen_y,
                            int32_t num_heads, int32_t head_dim, int32_t kernel_size, int32_t kernel_stride,
                            void* y, void* bias_scratch, void* stream);

int fsa_linear_compress_bwd(const void* x, const void* w, const void* pe, const void* dy, int32_t dtype,
                            int64_t x_stride_n, int64_t x_stride_h, const int32_t* cu_seqlens_x,
                            const int32_t* cu_seqlens_y, int32_t batch, int64_t max_seqlen_x, int64_t total_y,
                            int32_t num_heads, int32_t head_dim, int32_t kernel_size, int32_t kernel_stride,
                            void* dx, void* dw, void* dpe, float* dbias_scratch, void* stream);

/* ------------------------------------------------------------------------
 * Gate-weighted merge of the three branch outputs, one pass:
 *   out[n, :] = gate[n,0] a[n, :] + gate[n,1] b[n, :] + gate[n,2] c[n, :]
 * a, b, c, out contiguous [N, row_elems] (row_elems = Hq*D), gate contiguous
 * [N, 3] (already passed through the sigmoid), all in `dtype`; fp32 sum, one
 * rounding.  Backward: d_a = gate[n,0] d_out (same for b, c), d_gate[n,i] =
 * <d_out[n, :], x_i[n, :]>.  Replaces the broadcast multiply-adds of
 * fsa/module/fsa.py:162-167 (five elementwise passes forward, nine backward).
 * ---------------------------------------------------------------------- */
int fsa_gate_merge_fwd(const void* a, const void* b, const void* c, const void* gate, int32_t dtype,
                       int64_t total_tokens, int32_t row_elems, void* out, void* stream);

int fsa_gate_merge_bwd(const void* d_out, const void* a, const void* b, const void* c, const void* gate,
                       int32_t dtype, int64_t total_tokens, int32_t row_elems, void* d_a, void* d_b,
                       void* d_c, void* d_gate, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FSA_HIP_H */
