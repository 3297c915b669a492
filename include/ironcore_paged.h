/*
 * ironcore_paged.h -- C ABI of the MI355X (gfx950) paged-attention library.
 *
 * The reference (haanjack/ironcore) has no FFI, no KV cache and no native
 * code: its attention boundary is the Python call
 *     Attention.forward(query, key, value, attention_mask=None)
 *         ironcore/layers/attention.py:208-253
 * made from TransformerLayer.custom_forward
 *         ironcore/models/transformer.py:101-103
 * Each entry point below names the reference code whose work it takes over
 * when that call runs against a block KV cache.
 *
 * Conventions
 *  - Every pointer is a DEVICE pointer borrowed for the duration of the call
 *    (the kernels are enqueued on `stream`; the memory must stay valid until
 *    the stream reaches them).  The library never allocates or frees.
 *  - `stream` is a hipStream_t passed as void* (NULL = the default stream).
 *  - Return value: IC_OK (0) or a negative IC_ERR_* code.  Argument errors
 *    are detected on the host before anything is launched.  The library
 *    never throws and never exits the process.  Calls may come from any
 *    host thread; ordering is the stream's.  What the library remembers
 *    between calls never shows in a result: per device, the CU count and
 *    the address of the static scratch below; per process, the occupancy
 *    the runtime reported for each decode kernel variant and LDS size
 *    class (asked once, see ic_decode_occupancy_queries) and whether a
 *    variant's dynamic-LDS limit has been raised.  All of it is written
 *    once and read with atomics.
 *  - Device memory the library owns: one array of IC_STATIC_SCRATCH_BYTES
 *    (32 MiB), part of the code object, so every process that loads the
 *    library holds it on each GPU it uses, whether or not it ever calls
 *    ic_paged_decode_static (the only entry point that touches it).
 *  - Head dimensions with attention kernels: 32, 64 and 128 (the append
 *    entry points take any head dimension whose rows are a multiple of 16
 *    bytes); others return IC_ERR_UNSUPPORTED.  Block sizes: any multiple
 *    of 16 tokens.
 *  - Element type is selected by `dtype` (IC_DTYPE_*).  Strides are in
 *    ELEMENTS.  The head dimension is always contiguous.
 *
 * Block KV cache layout (defined by this library; the reference has none)
 *  - k_pool, v_pool: num_blocks blocks of `block_size` tokens.  Element
 *    (block, kv_head, token_in_block, d) lives at
 *        block*pool_stride_block + kv_head*pool_stride_head
 *        + token_in_block*pool_stride_token + d.
 *    The native layout is [num_blocks, gn, block_size, hd] contiguous
 *    (pool_stride_block = gn*block_size*hd, pool_stride_head = block_size*hd,
 *    pool_stride_token = hd), which makes one (block, kv_head) tile a single
 *    contiguous run of block_size*hd elements.
 *  - block_tables: int32 [n_seqs, block_table_stride]; entry j of row i is
 *    the pool block that holds tokens [j*block_size, (j+1)*block_size) of
 *    sequence i.  Rows may alias blocks (shared prefixes).
 *  - context_lens: int32 [n_seqs]; number of tokens visible to the query,
 *    including tokens appended for this step.
 *  - slot_mapping: int64 [n_tokens]; block*block_size + token_in_block for
 *    each new K/V row; a negative slot marks a padding row and is skipped.
 *  - GQA: query head h reads KV head h / (hn / gn)
 *    (ironcore/layers/attention.py:95-102).
 */
#ifndef IRONCORE_PAGED_H
#define IRONCORE_PAGED_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define IC_OK                 0
#define IC_ERR_NULL_POINTER  (-1)  /* a required pointer is NULL                 */
#define IC_ERR_BAD_SHAPE     (-2)  /* a size/stride is non-positive or inconsistent */
#define IC_ERR_UNSUPPORTED   (-3)  /* dtype / head_dim / group size / block size not built */
#define IC_ERR_WORKSPACE     (-4)  /* workspace missing or too small             */
#define IC_ERR_LAUNCH        (-5)  /* hipGetLastError() reported a launch failure */
#define IC_ERR_ALIGNMENT     (-6)  /* a pointer or stride breaks the 16-byte rule */
#define IC_ERR_STATIC_LIMIT  (-7)  /* batch too large for ic_paged_decode_static's scratch */

#define IC_DTYPE_BF16 0
#define IC_DTYPE_F16  1
#define IC_DTYPE_F32  2

/* Library ABI version (major*10000 + minor*100 + patch). */
int ic_version(void);

/* Static, NUL-terminated description of an IC_* code. */
const char *ic_error_string(int code);

/*
 * Diagnostic, no counterpart in the reference: launches a loop of `iters` x 16
 * independent v_mfma_f32_32x32x16_bf16 per wave, one wave per SIMD on every
 * CU, operands in registers (no memory, LDS or vector work), and returns the
 * launch's flop count (negative: IC_ERR_*).  Timed over a second or more of
 * back-to-back launches it gives the matrix rate the device sustains once its
 * clock has settled under load, which bench.py reports beside the nominal
 * 2.5 PFLOP/s.  sink: 4 bytes of device memory, never written in practice.
 */
int64_t ic_mfma_probe(int iters, void *sink, void *stream);

/*
 * Diagnostic, no counterpart in the reference: how many times the decode
 * launcher has asked the HIP runtime for a kernel's occupancy in this process.
 * The answers are kept per kernel variant and LDS size class (whole KiB), so
 * the count stops growing once a serving loop has seen its batch-size classes;
 * a launch whose answer is known makes no runtime query, which is what lets a
 * stream capture on any host thread follow a warm-up on another.
 */
int64_t ic_decode_occupancy_queries(void);

/*
 * KV append: copy the K/V rows a transformer layer produced for n_tokens new
 * tokens into their cache slots, bit for bit.  Replaces nothing in the
 * reference (which recomputes K/V for the whole sequence every step,
 * examples/generate_text.py:27); the rows are the `key`/`value` tensors of
 * ironcore/models/transformer.py:88-98.
 *
 *   k_new, v_new   [n_tokens, gn, hd], row stride new_stride_token, heads and
 *                  head_dim contiguous within a row
 *   slot_mapping   int64 [n_tokens]
 * Slots outside [0, num_blocks*block_size) are skipped.
 */
int ic_kv_append(const void *k_new, const void *v_new, int64_t new_stride_token,
                 void *k_pool, void *v_pool,
                 int64_t pool_stride_block, int64_t pool_stride_head,
                 int64_t pool_stride_token,
                 const int64_t *slot_mapping, int64_t n_tokens,
                 int gn, int hd, int block_size, int64_t num_blocks,
                 int dtype, void *stream);

/*
 * KV append with rotary position embedding: in one pass, rotate the query rows
 * in place, rotate the new key rows into their cache slots and copy the new
 * value rows into theirs.  Takes over ironcore/models/transformer.py:95-98
 * (query = rope(query); key = rope(key)) together with the append above.
 * Element pairs (2i, 2i+1) are rotated by the angle of table row
 * positions[t], with the arithmetic of
 * ironcore/layers/positional_embedding/rotary.py:69-83 (fp32, each product and
 * sum rounded separately, result rounded to the element type), so the result
 * is bit-identical to that expression evaluated by torch.
 *
 *   q              [n_tokens, hn, hd], row stride q_stride_token; rotated IN
 *                  PLACE; NULL = no query work
 *   k_new, v_new   as for ic_kv_append; both NULL = rotate q only (then the
 *                  pool arguments and slot_mapping are ignored)
 *   positions      int32 [n_tokens]: table row of each token, clamped to
 *                  [0, table_rows).  The reference indexes its tables by the
 *                  BATCH index of a row (rotary.py:55-64 after the transpose at
 *                  :55); a cached decoder passes the token's position in its
 *                  sequence.  The choice is the caller's.
 *   cos_table, sin_table   fp32 [table_rows, hd/2], 16-byte aligned: the
 *                  cos_emb / sin_emb buffers of rotary.py:36-51
 */
int ic_rope_kv_append(void *q, int64_t q_stride_token, int hn,
                      const void *k_new, const void *v_new, int64_t new_stride_token,
                      void *k_pool, void *v_pool,
                      int64_t pool_stride_block, int64_t pool_stride_head,
                      int64_t pool_stride_token,
                      const int64_t *slot_mapping, const int32_t *positions,
                      const float *cos_table, const float *sin_table, int64_t table_rows,
                      int64_t n_tokens, int gn, int hd, int block_size,
                      int64_t num_blocks, int dtype, void *stream);

/*
 * Workspace the decode entry point needs (block-count prefix sums and
 * split-K partials), in bytes, for a batch of n_seqs sequences with these
 * head counts.  Returns 0 for invalid arguments.
 */
size_t ic_paged_decode_workspace_bytes(int n_seqs, int hn, int gn, int hd);

/*
 * Paged decode: one query token per sequence against the block KV cache.
 * Computes what ironcore/layers/attention.py:68-142 (_attention) returns for
 * sq = 1 on the rows the block table points at:
 *     out[i, h*hd + d] = sum_j softmax_j(q[i,h] . k[i,j,h/G] * scale) * v[i,j,h/G,d]
 *
 *   out           [n_seqs, hn*hd], row stride out_stride_seq (16-byte aligned
 *                 rows for bf16 / fp16)
 *   q             [n_seqs, hn, hd], row stride q_stride_seq
 *   scale         multiplies q.k (the reference divides by sqrt(hd),
 *                 attention.py:65,110; pass 1/sqrt(hd))
 *   max_context_len  upper bound on context_lens; larger entries are clamped
 *                 to it, and block_table_stride must cover it
 *   min_chunk_tokens  the K/V stream of the whole batch is cut into equal
 *                 shares, one per resident wave (split-K); this is the
 *                 smallest share (multiple of 16), 0 = default
 *   block_size    a multiple of 16 (the kernel loads whole 16-token tiles)
 *   workspace     at least ic_paged_decode_workspace_bytes(...) bytes, 256-byte
 *                 aligned; contents need not be initialised
 * Sequences with context_lens[i] <= 0 produce zeros.
 */
int ic_paged_decode(void *out, int64_t out_stride_seq,
                    const void *q, int64_t q_stride_seq,
                    const void *k_pool, const void *v_pool,
                    int64_t pool_stride_block, int64_t pool_stride_head,
                    int64_t pool_stride_token,
                    const int32_t *block_tables, int64_t block_table_stride,
                    const int32_t *context_lens,
                    int n_seqs, int hn, int gn, int hd, int block_size,
                    int64_t num_blocks, int max_context_len, float scale,
                    int min_chunk_tokens, void *workspace, size_t workspace_bytes,
                    int dtype, void *stream);

/*
 * Paged decode for batches whose sequences alias prefix blocks (sampling
 * several continuations of one prompt: the block tables of a group repeat the
 * prompt's blocks, as a fork of the block KV cache leaves them).  Same result
 * as ic_paged_decode on the same arguments; the aliased blocks are streamed
 * from HBM once per cohort instead of once per sequence.  The reference has
 * no counterpart (it has no KV cache; every sample recomputes its prompt,
 * examples/generate_text.py:27); the attention it must reproduce is still
 * ironcore/layers/attention.py:68-142.
 *
 *   cohort_size           S >= 1: sequences i*S .. i*S+S-1 of the batch form
 *                         cohort i (the last one may be short).  1 = no
 *                         sharing, identical to ic_paged_decode.
 *                         bf16 / fp16 only; hn / gn <= 16, and S at most
 *                         8 * (16 / (hn / gn)) (integer division): a wave
 *                         carries the heads of 16 / (hn / gn) members and up
 *                         to 8 waves of a workgroup share a cohort's tiles.
 *   cohort_shared_blocks  int32 [ceil(n_seqs / S)]: for each cohort, how many
 *                         leading block-table entries are the SAME pool block
 *                         in all its members' rows.  May under-state the
 *                         sharing (0 is always valid); must not over-state it.
 *                         Only blocks every member's context covers entirely
 *                         are treated as shared.  Ignored (may be NULL) when
 *                         cohort_size is 1.
 *   workspace             at least ic_paged_decode_shared_workspace_bytes(...)
 * Everything else as for ic_paged_decode.
 */
size_t ic_paged_decode_shared_workspace_bytes(int n_seqs, int hn, int gn, int hd,
                                              int cohort_size);
int ic_paged_decode_shared(void *out, int64_t out_stride_seq,
                           const void *q, int64_t q_stride_seq,
                           const void *k_pool, const void *v_pool,
                           int64_t pool_stride_block, int64_t pool_stride_head,
                           int64_t pool_stride_token,
                           const int32_t *block_tables, int64_t block_table_stride,
                           const int32_t *context_lens,
                           int n_seqs, int hn, int gn, int hd, int block_size,
                           int64_t num_blocks, int max_context_len, float scale,
                           int min_chunk_tokens,
                           int cohort_size, const int32_t *cohort_shared_blocks,
                           void *workspace, size_t workspace_bytes,
                           int dtype, void *stream);

/*
 * Paged decode that allocates nothing and takes no workspace: ic_paged_decode
 * with the workspace (row prefix sums and split-K partials) in a static device
 * array of IC_STATIC_SCRATCH_BYTES inside the library.  It has no counterpart
 * in the reference; it is for callers that cannot allocate device memory and
 * have no workspace to pass: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  Same arguments, same kernels and same
 * result as ic_paged_decode (the grid is capped at 4096 waves, which no current
 * GPU exceeds).
 *
 *  - Limit: ic_paged_decode_static_scratch_bytes(n_seqs, hn, gn, hd) must not
 *    exceed IC_STATIC_SCRATCH_BYTES, else IC_ERR_STATIC_LIMIT and nothing is
 *    launched.  The need is 520 * (4096 + n_seqs * gn * ceil(G / 8)) * min(G, 8)
 *    bytes at hd 128 (G = hn / gn), plus 4 * (n_seqs + 2) rounded up to 256:
 *    21.3 MB for 128 sequences of 64 q / 8 kv heads, 22.4 MB for 512 sequences
 *    of 28 / 4 heads, 3.2 MB for 64 sequences of 32 / 32 heads.
 *  - Each GPU the library is used on holds the array from the first call on
 *    that device until the process ends.  The first call on a device looks the
 *    array's address up (hipGetSymbolAddress) and, like the first launch of any
 *    kernel variant, must not be made under stream capture.
 *  - Every call on a GPU uses that GPU's one array: calls that overlap in time
 *    on one GPU (two streams, two host threads) race on the partials.  Calls
 *    ordered on one stream are safe; nothing in the array has to be cleared
 *    between calls (each call writes every value it later reads).
 */
#define IC_STATIC_SCRATCH_BYTES (32u << 20)
size_t ic_paged_decode_static_scratch_bytes(int n_seqs, int hn, int gn, int hd);
int ic_paged_decode_static(void *out, int64_t out_stride_seq,
                           const void *q, int64_t q_stride_seq,
                           const void *k_pool, const void *v_pool,
                           int64_t pool_stride_block, int64_t pool_stride_head,
                           int64_t pool_stride_token,
                           const int32_t *block_tables, int64_t block_table_stride,
                           const int32_t *context_lens,
                           int n_seqs, int hn, int gn, int hd, int block_size,
                           int64_t num_blocks, int max_context_len, float scale,
                           int min_chunk_tokens, int dtype, void *stream);

/*
 * Chunked prefill against the block KV cache: each sequence brings a chunk of
 * new query tokens whose K/V rows are already appended; query row r of a
 * chunk of length C in a sequence of context length L sees keys
 * j <= (L - C) + r.  Computes what attention.py:68-142 returns for
 * sq = C, sk = L with the causal mask of ironcore/language_model.py:109-114
 * shifted by the cached prefix.  With causal = 0 every query row sees all L
 * keys (the reference's attention_mask=None case).  bf16 / fp16 pools run on
 * the 16-bit matrix-core kernel; fp32 pools on an fp32 kernel that keeps
 * every product, sum and probability in fp32.
 *
 *   out           [n_tokens, hn*hd], row stride out_stride_token
 *   q             [n_tokens, hn, hd], row stride q_stride_token; the chunk of
 *                 sequence i is rows cu_seqlens_q[i] .. cu_seqlens_q[i+1]-1
 *   cu_seqlens_q  int32 [n_seqs + 1]
 *   max_chunk_len upper bound on any chunk length (sizes the grid)
 * The 16-bit kernel addresses inside a pool block with 32 bits: a call whose
 * pool_stride_block, or pool_stride_token times the rows of a block, reaches
 * 2^31 elements (a block of 4 GiB) returns IC_ERR_UNSUPPORTED.
 */
int ic_paged_prefill(void *out, int64_t out_stride_token,
                     const void *q, int64_t q_stride_token,
                     const void *k_pool, const void *v_pool,
                     int64_t pool_stride_block, int64_t pool_stride_head,
                     int64_t pool_stride_token,
                     const int32_t *block_tables, int64_t block_table_stride,
                     const int32_t *context_lens, const int32_t *cu_seqlens_q,
                     int n_seqs, int max_chunk_len,
                     int hn, int gn, int hd, int block_size,
                     int64_t num_blocks, float scale, int causal,
                     int dtype, void *stream);

/*
 * Chunked prefill under a general attention mask: ic_paged_prefill with the
 * causal rule replaced by the caller's mask, for the attention_mask argument
 * of ironcore/layers/attention.py:208-253 when it is neither absent nor the
 * causal pattern (any mask broadcastable to [b, 1, sq, sk], attention.py:115-117;
 * e.g. the per-document masks of ironcore/language_model.py:140-152).
 *
 *   mask    uint8; the byte of (sequence i, query head h, chunk row r, key j) is
 *           mask[i*mask_stride_seq + h*mask_stride_head + r*mask_stride_row + j],
 *           nonzero = visible.  A stride of 0 broadcasts over that index.
 *   mask_keys  keys every mask row covers (its extent along j): a key at or
 *           beyond it is hidden, and no byte past it is read.
 * Hidden keys get the reference's FINITE fill value (attention.py:66): next to a
 * visible key they weigh nothing; a query row with no visible key returns the
 * plain average of V over its context, as the reference does.  A chunk may be
 * longer than its context here (sq > sk).  bf16, fp16 and fp32.
 */
int ic_paged_prefill_masked(void *out, int64_t out_stride_token,
                            const void *q, int64_t q_stride_token,
                            const void *k_pool, const void *v_pool,
                            int64_t pool_stride_block, int64_t pool_stride_head,
                            int64_t pool_stride_token,
                            const int32_t *block_tables, int64_t block_table_stride,
                            const int32_t *context_lens, const int32_t *cu_seqlens_q,
                            int n_seqs, int max_chunk_len,
                            int hn, int gn, int hd, int block_size,
                            int64_t num_blocks, float scale,
                            const uint8_t *mask, int64_t mask_stride_seq,
                            int64_t mask_stride_head, int64_t mask_stride_row,
                            int64_t mask_keys, int dtype, void *stream);

/*
 * Paged decode under a key mask, fp32 only: ic_paged_decode where sequence i's
 * query head h sees key j only if
 * key_mask[i*key_mask_stride_seq + h*key_mask_stride_head + j] is nonzero
 * (key_mask_stride_head 0 = one mask row for all heads; key_mask_stride_seq
 * >= max_context_len).  Same finite-fill semantics as ic_paged_prefill_masked.
 * For single-token steps of an fp32 model under a general mask; chunks, and
 * 16-bit calls of any length, use ic_paged_prefill_masked (16-bit pools get
 * IC_ERR_UNSUPPORTED here).
 */
int ic_paged_decode_masked(void *out, int64_t out_stride_seq,
                           const void *q, int64_t q_stride_seq,
                           const void *k_pool, const void *v_pool,
                           int64_t pool_stride_block, int64_t pool_stride_head,
                           int64_t pool_stride_token,
                           const int32_t *block_tables, int64_t block_table_stride,
                           const int32_t *context_lens,
                           int n_seqs, int hn, int gn, int hd, int block_size,
                           int64_t num_blocks, int max_context_len, float scale,
                           int min_chunk_tokens,
                           const uint8_t *key_mask, int64_t key_mask_stride_seq,
                           int64_t key_mask_stride_head,
                           void *workspace, size_t workspace_bytes,
                           int dtype, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* IRONCORE_PAGED_H */
