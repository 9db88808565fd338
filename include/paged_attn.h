/*
 * paged_attn.h - C ABI of libpaged_attn.so: paged-KV attention for one MI355X
 * (gfx950) behind the attention / KV-cache call surface of the `rollouts`
 * inference engine.
 *
 * Conventions for every entry point
 *   - plain pointers and sizes; device pointers unless the name says host;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream);
 *     work is enqueued asynchronously on it, nothing synchronises;
 *   - the return value is a status: PA_OK, or a negative PA_ERR_* after which
 *     pa_last_error() (thread-local text) says what was wrong.  Arguments are
 *     checked on the host before any HIP call, so a rejected call has touched
 *     neither the GPU nor its buffers;
 *   - the library allocates nothing: the caller owns inputs, outputs and the
 *     decode workspace;
 *   - indices read from device memory (slots, block ids) are range-checked by
 *     the kernels against `total_slots` / `num_blocks`: an out-of-range index
 *     is skipped (append) or reads as zeros (gather, attention), never a fault.
 *
 * Pool layout (fixed by the reference, attention/config.py:43-45, one layer's
 * slice): element [slot][kv_head][d] at ((slot*num_kv_heads)+kv_head)*head_dim+d,
 * slot = block_id*block_size + offset_in_block.
 *
 * Reference citations are relative to rollouts/rollouts/inference/.
 */
#ifndef PAGED_ATTN_H
#define PAGED_ATTN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PA_OK 0
#define PA_ERR_INVALID_ARG (-1) /* NULL pointer, negative size, inconsistent dims */
#define PA_ERR_UNSUPPORTED (-2) /* dtype / head_dim / group size has no kernel */
#define PA_ERR_WORKSPACE (-3)   /* decode workspace missing or too small */
#define PA_ERR_HIP (-4)         /* a HIP launch reported an error */

/* element types of q / out / the KV pool */
#define PA_F32 0
#define PA_BF16 1
#define PA_F16 2
#define PA_FP8_E4M3 3 /* OCP e4m3fn, KV pool only; q/out stay 16- or 32-bit */

/* Library ABI version (bumped when an entry point is added or a signature or contract changes; now 6). */
int pa_version(void);

/* Text of the calling thread's most recent error; "" if none. */
const char *pa_last_error(void);

/* Bytes per element of a PA_* dtype, or 0 for an unknown code. */
int pa_dtype_bytes(int dtype);

/*
 * KV append / scatter.  Replaces FlexAttentionBackend._store_kv
 * (attention/flex_backend.py:116-142):
 *     for i in range(n_tokens): s = slots[i]
 *         if s >= 0: k_cache[s] = k_src[i]; v_cache[s] = v_src[i]
 * A pure byte copy of rows of num_kv_heads*head_dim elements; rows whose slot
 * is negative (the reference's filter, :139-142) or >= total_slots are
 * dropped.  Duplicate slots in one call: which source row wins is unspecified
 * (as for the reference's index_put on a GPU).
 *   k_cache,v_cache : one layer's pool slice, [total_slots][row]
 *   k_src,v_src     : [n_tokens][row], contiguous
 *   slots           : int64[n_tokens]
 *   elem_bytes      : 1, 2 or 4; row bytes must be a multiple of 4
 */
int pa_kv_scatter(void *k_cache, void *v_cache, const void *k_src, const void *v_src,
                  const int64_t *slots, int64_t n_tokens, int64_t total_slots,
                  int num_kv_heads, int head_dim, int elem_bytes, void *stream);

/*
 * Block-table gather.  Replaces FlexAttentionBackend._gather_kv_from_cache
 * (attention/flex_backend.py:233-279):
 *     out[b][pos] = cache[bt[b][pos / bs] * bs + pos % bs]   for pos < seq_lens[b]
 * and zeros for pos >= seq_lens[b], for positions whose block-table entry is
 * missing (the reference's short-table case, :274; here: entry < 0, entry >=
 * num_blocks, or pos / bs >= bt_stride), up to max_len.  Bit-exact copy.
 *   block_tables : int32[batch][bt_stride], row-padded with -1
 *   seq_lens     : int32[batch]
 *   k_out,v_out  : [batch][max_len][row], every byte is written
 */
int pa_kv_gather(const void *k_cache, const void *v_cache, void *k_out, void *v_out,
                 const int32_t *block_tables, int64_t bt_stride, const int32_t *seq_lens,
                 int batch, int64_t max_len, int64_t num_blocks, int block_size,
                 int num_kv_heads, int head_dim, int elem_bytes, void *stream);

/*
 * Workspace of pa_decode in bytes (host arithmetic only, no GPU call); 0 on
 * error.  pa_decode splits the batch's pool blocks evenly over a machine-sized
 * grid of workgroups; a sequence whose blocks fall into several workgroups
 * leaves one partial result per piece in the workspace.  The size depends on
 * the shapes only, never on the sequence lengths, so one allocation serves
 * every step of a model.  Alignment: 256 bytes.  The first
 * PA_DECODE_TICKET_BYTES bytes hold the arrival counters of the merge inside
 * the split pass: zero-fill them once after allocating the workspace (before
 * its first use; outside any stream capture) and leave them to the library
 * afterwards - every call returns them to "nothing arrived", whatever its
 * shapes, so captured graphs replay without clearing anything.  The rest need
 * not be initialised.  Calls that share a workspace must not overlap in time.
 */
#define PA_DECODE_TICKET_BYTES (640u << 10)
size_t pa_decode_workspace_bytes(int batch, int num_q_heads, int num_kv_heads, int head_dim,
                                 int kv_dtype);

/*
 * Kernel launches one pa_decode call of these shapes makes on the current device: 1 when the batch is large
 * enough that the split pass merges a sequence's pieces itself, else 2 (split pass, reduction pass); negative on
 * error.  For callers that time or profile the passes.  (No counterpart in the reference.)
 */
int pa_decode_passes(int batch, int num_q_heads, int num_kv_heads, int head_dim, int kv_dtype);

/*
 * Paged decode attention.  Replaces FlexAttentionBackend._decode_attention
 * (attention/flex_backend.py:187-231) together with the gather and the GQA
 * repeat_interleave it performs: for sequence b and query head h
 *     kvh = h / (num_q_heads / num_kv_heads)
 *     out[b][h] = softmax_j( scale * q[b][h] . K[b][j][kvh] ) . V[b][j][kvh],  j < seq_lens[b]
 * with K/V rows addressed through the block table as in pa_kv_gather; a
 * position whose block-table entry is missing acts as an all-zero key and
 * value (logit 0), as it does in the reference.  Accumulation is fp32.  All
 * integer inputs stay on the device: the host never reads seq_lens.
 *   q, out        : [batch][num_q_heads][head_dim], dtype q_dtype, 16-byte aligned
 *   head_dim      : a multiple of 8 up to 256 (of 16 for an fp8 pool; rows of whole 16-byte vectors); the
 *                   reference takes any head_dim (attention/config.py:22-24)
 *   kv_dtype      : q_dtype, or PA_FP8_E4M3 with k_scale/v_scale =
 *                   float[num_blocks][num_kv_heads] (value = fp8 * scale)
 *   extra_zero_keys: NULL, or int32[batch]: that many additional all-zero
 *                   keys take part in sequence b's softmax.  The reference
 *                   zero-pads ragged batches to the longest sequence without a
 *                   mask (:253-264, :227-229); passing max_len - seq_lens[b]
 *                   reproduces it.
 *   window        : 0, or a sliding window: only the last `window` keys of each sequence are attended
 *                   (j >= seq_lens[b] - window), the rule of the reference's causal_sliding_window_mask
 *                   (attention/mask.py:83-89: q_idx - kv_idx < window_size) for the query at position
 *                   seq_lens[b]-1; blocks wholly before the window are never read.  The reference's own
 *                   decode applies a window only through a caller-built ctx.block_mask
 *                   (flex_backend.py:220-225).  Not combinable with extra_zero_keys.
 *   batch         : any; more than 8192 sequences are taken 8192 at a time, one after the other on the stream
 *   workspace     : pa_decode_workspace_bytes(...) bytes, its first PA_DECODE_TICKET_BYTES zero-filled once
 *   A sequence of length 0 yields zeros.
 */
int pa_decode(const void *q, const void *k_cache, const void *v_cache, void *out,
              const int32_t *block_tables, int64_t bt_stride, const int32_t *seq_lens,
              const int32_t *extra_zero_keys, const float *k_scale, const float *v_scale,
              int batch, int num_q_heads, int num_kv_heads, int head_dim, int block_size,
              int64_t num_blocks, float scale, int window, int q_dtype, int kv_dtype, void *workspace,
              size_t workspace_bytes, void *stream);

/*
 * The two passes of pa_decode as separate calls, same arguments:
 * pa_decode_split followed by pa_decode_reduce on the same stream and
 * workspace give pa_decode's result (to rounding: for large batches pa_decode
 * merges inside its one launch, in another order; see pa_decode_passes).  For
 * callers that time or schedule the passes separately.  (The
 * reference has one fused call site, attention/flex_backend.py:227-229; these
 * have no separate counterpart there.)
 */
int pa_decode_split(const void *q, const void *k_cache, const void *v_cache, void *out,
                    const int32_t *block_tables, int64_t bt_stride, const int32_t *seq_lens,
                    const int32_t *extra_zero_keys, const float *k_scale, const float *v_scale,
                    int batch, int num_q_heads, int num_kv_heads, int head_dim, int block_size,
                    int64_t num_blocks, float scale, int window, int q_dtype, int kv_dtype, void *workspace,
                    size_t workspace_bytes, void *stream);
int pa_decode_reduce(const void *q, const void *k_cache, const void *v_cache, void *out,
                     const int32_t *block_tables, int64_t bt_stride, const int32_t *seq_lens,
                     const int32_t *extra_zero_keys, const float *k_scale, const float *v_scale,
                     int batch, int num_q_heads, int num_kv_heads, int head_dim, int block_size,
                     int64_t num_blocks, float scale, int window, int q_dtype, int kv_dtype, void *workspace,
                     size_t workspace_bytes, void *stream);

/*
 * pa_decode without a workspace argument and without any allocation, for callers that cannot allocate device
 * memory: code under HIP graph capture, serving loops with a fixed memory plan, harnesses that forbid
 * hipMalloc.  (No counterpart in the reference, which allocates freely inside its decode,
 * attention/flex_backend.py:253-264.)  The partial results of the split pass go to a scratch array of
 * PA_DECODE_STATIC_SCRATCH_BYTES that the library's code object holds on every GPU it is loaded on, from load
 * until the process ends.  Arguments and results are those of pa_decode, bit for bit.
 *   - Shapes whose partials do not fit return PA_ERR_WORKSPACE (the message gives the bytes needed); the
 *     need is (workgroups of the split pass + planes * batch) * heads * (head_dim + 2) * 4 bytes, e.g.
 *     8.5 MB for batch 256, 32 query / 8 kv heads of 128 on a 256-CU device.
 *   - Every call on one GPU shares that GPU's array, which keeps the previous call's partials: calls whose
 *     kernels may overlap on one GPU (different streams, different threads) race; order them.
 *   - The first call on a device asks the runtime for the array's address (hipGetSymbolAddress); make that
 *     call outside a stream capture.  No call allocates or frees.
 */
#define PA_DECODE_STATIC_SCRATCH_BYTES (16u << 20)
int pa_decode_static(const void *q, const void *k_cache, const void *v_cache, void *out,
                     const int32_t *block_tables, int64_t bt_stride, const int32_t *seq_lens,
                     const int32_t *extra_zero_keys, const float *k_scale, const float *v_scale, int batch,
                     int num_q_heads, int num_kv_heads, int head_dim, int block_size, int64_t num_blocks,
                     float scale, int window, int q_dtype, int kv_dtype, void *stream);

/*
 * Causal prefill attention over a paged context.  Covers both
 * FlexAttentionBackend._prefill_attention (attention/flex_backend.py:144-185,
 * the is_causal SDPA over the step's own K/V) and chunked prefill over cached
 * prefix blocks (a composition the reference does not have): for sequence b
 * the q_lens[b] query rows are the LAST q_lens[b] positions of a context of
 * ctx_lens[b] keys, and row i attends keys j <= ctx_lens[b] - q_lens[b] + i.
 * The keys are read through the block table, so the step's new K/V must have
 * been appended (pa_kv_scatter) first.  Sequences that list the same block
 * ids share those blocks.
 *   q, out   : [total_q][num_q_heads][head_dim] packed rows, sequence b's rows
 *              start at q_starts[b]; dtype PA_BF16 or PA_F16 (MFMA path) or
 *              PA_F32 (vector path)
 *   head_dim : a multiple of 8 up to 256.  bf16 / fp16 run on the matrix cores: 32, 64, 128 and 256 have
 *              kernels of their own, every other multiple of 8 runs the kernel of the next larger size (rows in
 *              memory keep their length); PA_F32 runs on the vector kernel
 *   ctx_lens, q_lens, q_starts : int32[batch]
 *   max_q_len: upper bound of q_lens (grid sizing)
 *   window   : 0, or the sliding window of CacheConfig.sliding_window (attention/config.py:31): row i at
 *              position p = ctx_lens[b] - q_lens[b] + i attends keys p - window < j <= p
 *              (attention/mask.py:83-89); tiles wholly before the window of a workgroup's rows are not loaded.
 *   row_first_key : NULL, or int32[total_q] indexed like the rows of q: the first key position (in the
 *              row's own sequence) the row attends, on top of the causal bound -- the packed-document mask
 *              of create_document_mask (attention/mask.py:141-191: same document and q_idx >= kv_idx) with
 *              row_first_key = start of the row's document.  Must not decrease along a sequence; values
 *              are clamped to [0, position of the row], so a row always sees itself.  Combines with window
 *              (the later of the two bounds applies).
 */
int pa_prefill_paged(const void *q, const void *k_cache, const void *v_cache, void *out,
                     const int32_t *block_tables, int64_t bt_stride, const int32_t *ctx_lens,
                     const int32_t *q_lens, const int32_t *q_starts, const int32_t *row_first_key,
                     int batch, int max_q_len, int num_q_heads, int num_kv_heads, int head_dim,
                     int block_size, int64_t num_blocks, float scale, int window, int dtype, void *stream);

/*
 * pa_prefill_paged with a workspace, for launches of few query rows.  The reference's SDPA call
 * (attention/flex_backend.py:180-182) spreads one long row's keys over the machine however PyTorch likes; the
 * matrix-core kernels here give a workgroup 256 row-head pairs and all their keys, so one 2048-row chunk behind a
 * long cached context occupies a quarter of the compute units.  Given a workspace, such a launch cuts every
 * workgroup's keys into up to 8 pieces run by workgroups of their own, which leave (maximum, sum, unnormalised
 * output row) per piece in the workspace, and a second kernel merges them - the arithmetic of pa_decode's
 * reduction pass.  Results equal pa_prefill_paged's to fp32 merge-order rounding.
 *   total_q        : rows of q / out (every q_starts[b] + q_lens[b] <= total_q)
 *   workspace      : pa_prefill_workspace_bytes(...) bytes, 256-byte aligned, contents need not be initialised;
 *                    NULL or too small for any split: the call is pa_prefill_paged.  A smaller workspace is used
 *                    for as many pieces as it holds.
 * pa_prefill_workspace_bytes: what the split the library would choose for these shapes on the current device needs
 * (0 when the launch fills the device anyway, or for fp32, which only the unsplit vector kernel takes; a head size
 * between 32 / 64 / 128 / 256 is sized for partial rows of the next larger one); host arithmetic plus one
 * device-attribute query.
 * bt_stride * block_size bounds the context length the split is sized for.
 */
size_t pa_prefill_workspace_bytes(int batch, int max_q_len, int64_t total_q, int64_t bt_stride, int block_size,
                                  int window, int num_q_heads, int num_kv_heads, int head_dim, int dtype);
int pa_prefill_paged_ws(const void *q, const void *k_cache, const void *v_cache, void *out,
                        const int32_t *block_tables, int64_t bt_stride, const int32_t *ctx_lens,
                        const int32_t *q_lens, const int32_t *q_starts, const int32_t *row_first_key,
                        int batch, int max_q_len, int num_q_heads, int num_kv_heads, int head_dim,
                        int block_size, int64_t num_blocks, float scale, int window, int dtype, void *stream,
                        int64_t total_q, void *workspace, size_t workspace_bytes);

/*
 * Attention under an arbitrary mask: what FlexAttentionBackend does with a ctx.block_mask built from any
 * mask_mod(b, h, q_idx, kv_idx) predicate (attention/flex_backend.py:170-178 in prefill, :220-225 in decode;
 * predicates such as attention/mask.py:42, :84, :171).  The caller evaluates the predicate into bits; row r of
 * sequence b (packed row q_starts[b] + r), query head h attends key j < n_keys iff bit j of its mask row is
 * set - nothing else is implied, a causal bound included.  Keys j >= ctx_lens[b] and keys in absent blocks are
 * zero rows (logit 0, zero value), which is what the reference's zero-padded decode gather hands to
 * flex_attention (:253-264); a row with no bit set gives zeros.
 *   q, out  : [total_q][num_q_heads][head_dim], dtype F32 / BF16 / F16
 *   kv_dtype: dtype, or PA_FP8_E4M3 (16-bit q) with k_scale / v_scale float[num_blocks][num_kv_heads] as in pa_decode
 *   mask    : uint32 [total_q][mask_heads][mask_words], bit j of word j/32; mask_heads is 1 (all heads share
 *             the row) or num_q_heads
 * The general path, not a fast one: one workgroup per (head, row), a wave-wide reduction per visible key.  The
 * structured masks (causal, sliding window, packed documents) go through pa_prefill_paged / pa_decode.
 */
int pa_attend_masked(const void *q, const void *k_cache, const void *v_cache, void *out,
                     const int32_t *block_tables, int64_t bt_stride, const int32_t *ctx_lens,
                     const int32_t *q_lens, const int32_t *q_starts, const uint32_t *mask, int mask_heads,
                     int mask_words, int n_keys, int batch, int max_q_len, int num_q_heads, int num_kv_heads,
                     int head_dim, int block_size, int64_t num_blocks, float scale, int dtype, int kv_dtype,
                     const float *k_scale, const float *v_scale, void *stream);

/*
 * pa_prefill_paged evaluated by the vector kernel (one workgroup per query row, the decode inner loop) whatever
 * the element type: the path fp32 and fp8-pool calls take anyway, selectable for the 16-bit shapes too so that
 * the two kernels can be checked against each other.  Same arguments, same results to rounding.
 * (No separate counterpart in the reference: both are attention/flex_backend.py:144-185.)
 */
int pa_prefill_paged_rowwise(const void *q, const void *k_cache, const void *v_cache, void *out,
                             const int32_t *block_tables, int64_t bt_stride, const int32_t *ctx_lens,
                             const int32_t *q_lens, const int32_t *q_starts, const int32_t *row_first_key,
                             int batch, int max_q_len, int num_q_heads, int num_kv_heads, int head_dim,
                             int block_size, int64_t num_blocks, float scale, int window, int dtype, void *stream);

/*
 * fp8-e4m3 pool construction (no counterpart in the reference; its oracle is
 * "dequantise, then attend in fp32").  For every (block, kv head):
 *     s = max|x| / 448  (s = 1 when the block is all zero)
 *     dst = e4m3fn_rne(x / s),  scale[block][kv_head] = s
 *   src   : [num_blocks*block_size][num_kv_heads][head_dim], src_dtype F32/BF16/F16
 *   dst   : same shape, one byte per element
 *   scale : float[num_blocks][num_kv_heads]
 */
int pa_quantize_kv_e4m3(const void *src, void *dst, float *scale, int64_t num_blocks,
                        int block_size, int num_kv_heads, int head_dim, int src_dtype,
                        void *stream);

/*
 * Append rows to an fp8-e4m3 pool (no counterpart in the reference: its _store_kv, flex_backend.py:116-142,
 * copies rows of the pool's own type).  Policy, per (block, kv head) tile: "re-round on growth".
 *   - rows of the tile below the lowest offset this call writes are its content so far; a call that writes
 *     offset 0 starts the tile over (recycled blocks need no clearing);
 *   - a_old = scale * max|stored value| over the content, a_new = max|x| over the rows written by this call;
 *   - a_new <= a_old: scale unchanged; otherwise scale' = a_new/448 (1 if a_new = 0) and every content byte
 *     becomes e4m3fn_rne(float(byte) * (scale / scale'));
 *   - new rows are stored as e4m3fn_rne(x / scale').
 *   slots          : int64[n_tokens], slot = block*block_size + offset; negative or out-of-pool slots are skipped;
 *                    of two tokens with the same slot the later one is stored
 *   touched_blocks : int32[n_touched], the distinct blocks the slots fall in (extra entries are harmless,
 *                    a block must not appear twice)
 *   row_order, block_start : optional index of the rows by touched block (both NULL: every workgroup scans the
 *                    whole slot list, n_touched * n_tokens slot reads per tensor, fine for a decode step and
 *                    quadratic in the length of a prefill chunk).  row_order int32[n_tokens]: token indices
 *                    grouped by touched block; block_start int32[n_touched + 1]: tokens
 *                    row_order[block_start[i]] .. row_order[block_start[i+1] - 1] are those whose slots fall in
 *                    touched_blocks[i].  A token the index leaves out is not stored; entries out of range are
 *                    ignored.
 *   k_src, v_src   : [n_tokens][num_kv_heads][head_dim] in src_dtype (F32/BF16/F16)
 *   k_scale,v_scale: float[num_blocks][num_kv_heads], updated in place
 */
int pa_kv_append_e4m3(void *k_cache, void *v_cache, float *k_scale, float *v_scale, const void *k_src,
                      const void *v_src, const int64_t *slots, int64_t n_tokens,
                      const int32_t *touched_blocks, int n_touched, const int32_t *row_order,
                      const int32_t *block_start, int64_t num_blocks, int block_size, int num_kv_heads,
                      int head_dim, int src_dtype, void *stream);

/*
 * Rotary position embedding fused with the KV append: the step a model runs immediately before this path
 * (rollouts/tools/functional_extractor/llama_functional.py:203 applies apply_rotary_pos_emb, :75-98, right
 * before attention, :210) merged with FlexAttentionBackend._store_kv (attention/flex_backend.py:116-142), so
 * the step's new K rows are read once and written once.  For every token i, with r = positions[i] (or i):
 *     x_embed = (x * cos[r]) + (rotate_half(x) * sin[r]),   rotate_half(x) = cat(-x[D/2:], x[:D/2])
 * for every head of q (written to q_out, which may be q itself) and of k; the rotated k row goes to
 * k_cache[slots[i]] (and to k_out[i] when k_out is given), the v row to v_cache[slots[i]].  Every product and
 * the sum are rounded to `dtype`, as when the statement is evaluated on tensors of that type: results equal
 * that evaluation bit for bit.
 *   q, q_out     : [n_tokens][num_q_heads][head_dim]
 *   k_src, v_src : [n_tokens][num_kv_heads][head_dim];  k_out: same shape or NULL
 *   k_cache, v_cache : [total_slots][num_kv_heads][head_dim] of the same dtype
 *   cos, sin     : [rope_rows][head_dim] of the same dtype (both halves are read, as the statement does)
 *   positions    : int32[n_tokens] rows of cos/sin, clamped to the table; NULL: token i uses row i
 *                  (tables laid out per token, the (batch, seq_len, head_dim) form of llama_functional.py:101-136)
 *   slots        : int64[n_tokens]; negative or out-of-pool slots skip the cache write; NULL: no cache write
 *                  (then k_out is required)
 * head_dim/2 elements must fill whole 16-byte vectors (head_dim % 16 == 0 for 16-bit types).
 */
int pa_rope_kv_append(const void *q, void *q_out, const void *k_src, const void *v_src, void *k_out,
                      void *k_cache, void *v_cache, const void *cos, const void *sin, const int32_t *positions,
                      int64_t rope_rows, const int64_t *slots, int64_t n_tokens, int64_t total_slots,
                      int num_q_heads, int num_kv_heads, int head_dim, int dtype, void *stream);

/*
 * The same for an fp8-e4m3 pool: q is rotated to q_out, the k rows are rotated as pa_rope_kv_append does
 * (rounded to src_dtype) while pa_kv_append_e4m3's append reads them, and the v rows are appended as they are.
 * Arguments as in pa_rope_kv_append and pa_kv_append_e4m3; the result equals pa_rope_kv_append into a dense
 * k_out followed by pa_kv_append_e4m3 of k_out, bit for bit.
 */
int pa_rope_kv_append_e4m3(const void *q, void *q_out, const void *k_src, const void *v_src, void *k_cache,
                           void *v_cache, float *k_scale, float *v_scale, const void *cos, const void *sin,
                           const int32_t *positions, int64_t rope_rows, const int64_t *slots, int64_t n_tokens,
                           const int32_t *touched_blocks, int n_touched, const int32_t *row_order,
                           const int32_t *block_start, int64_t num_blocks, int block_size, int num_q_heads,
                           int num_kv_heads, int head_dim, int src_dtype, void *stream);

/*
 * Dequantise listed blocks of an fp8-e4m3 pool into a compact 16-bit pool (no counterpart in the reference):
 * block j of dst = block block_ids[j] of the pool, every value float(byte) * scale[block][kv_head] rounded to
 * dst_dtype (BF16/F16).  Used to run prefill over an fp8 pool on the matrix cores: dequantise the blocks the
 * step's block tables name (each once, however many sequences share it), renumber the tables to positions in
 * block_ids, and call pa_prefill_paged on dst.  Ids outside [0, num_blocks) give zero blocks.
 *   cache : [num_blocks*block_size][num_kv_heads][head_dim] bytes;  scale: float[num_blocks][num_kv_heads]
 *   dst   : [n_ids*block_size][num_kv_heads][head_dim] of dst_dtype;  head_dim % 16 == 0
 */
int pa_dequantize_blocks_e4m3(const void *cache, const float *scale, const int32_t *block_ids, int n_ids,
                              void *dst, int64_t num_blocks, int block_size, int num_kv_heads, int head_dim,
                              int dst_dtype, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* PAGED_ATTN_H */
