/*
 * pace_kv_hip.h -- C ABI of the MI355X (gfx950) KV-cache hot path.
 *
 * Everything that crosses this boundary is a raw device pointer, an explicit
 * size/stride, or a plain-old-data struct.  No torch types, no C++ types.
 * Every entry point enqueues on the HIP stream it is given and returns without
 * synchronising; it returns 0 on success and a negative code on failure, with
 * the text of the failure available from pace_kv_last_error() (thread-local).
 *
 * Reference interfaces these entry points stand behind (reference repository
 * paths, file:line):
 *   - pace::attention torch op          csrc/ops/attention.cpp:18-108
 *   - kernels::attention_kernel         csrc/ops/kernels/attention_kernels.h:26-32
 *   - KVCacheBase.update_cache          pace/llm/cache.py:134-143, 268-326, 370-400
 *   - KVCacheBase.remove_cache          pace/llm/cache.py:224-240, 352-368 (host metadata only)
 *   - update_cache_with_beam_indices    pace/llm/cache.py:161-167
 *   - repeat_kv (folded into the kernels) pace/llm/models/llama.py:50-61
 *   - RotaryEmbedding.apply_rotary_emb   pace/ops/rotary_embedding.py:412-474 (the step before the append)
 *
 * Storage: a block pool.  Block size is 16 tokens.  One (block, KV head) slab
 * holds 16 tokens x head_dim values in an order private to the library (see
 * k_slab_offset / v_slab_offset in the sources: 16-byte granules arranged so
 * that every wavefront-wide load of the attention kernel is contiguous and
 * already in matrix-core operand order); callers only ever move data through
 * append / gather / copy_blocks.  Slabs are addressed as
 *   base + block * block_stride + head * head_stride   (strides in elements),
 * which covers both two separate K / V allocations and one interleaved
 * [block][2][head][16*head_dim] allocation.  Unwritten slots must hold finite
 * bit patterns (allocate the pool zero-filled).
 *
 * A pool may hold fp32 instead (elem_bytes = 4: the reference's caches keep
 * whatever dtype the model runs in, pace/llm/cache.py:255-266, and its
 * attention is registered for float32 and bfloat16, pace/ops/backends/jit.py:31-34).
 * Its slabs are plain rows, [16 tokens][head_dim] floats, head_dim any multiple
 * of 4 up to 256, strides in floats.  Append, append_paged, gather,
 * gather_packed, copy_blocks, compact_blocks and the decode / verify attention
 * take such a pool (new tokens, gathered rows, queries and outputs are then
 * fp32 too; the attention needs no work list, and a workspace only helps it when
 * the batch leaves compute units idle: with room for batch * num_q_heads * q_len
 * * parts * (head_dim + 4) floats it cuts every sequence over up to parts <= 64
 * workgroups); what folds other steps into
 * a launch (pace_rope_append_paged, args->rope, args->k_new) is bf16 only and
 * says so when handed such a pool.
 */
#ifndef PACE_KV_HIP_H
#define PACE_KV_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PACE_KV_BLOCK_TOKENS 16

enum {
  PACE_KV_OK = 0,
  PACE_KV_EINVAL = -1, /* an argument violates the documented contract          */
  PACE_KV_EHIP = -2,   /* a HIP runtime call failed (launch, attribute query...) */
};

enum { PACE_DTYPE_F32 = 0, PACE_DTYPE_BF16 = 1 };

typedef struct pace_kv_pool {
  void* k;                /* bf16, K slabs                                   */
  void* v;                /* bf16, V slabs                                   */
  int64_t k_block_stride; /* elements between consecutive blocks of K        */
  int64_t k_head_stride;  /* elements between consecutive KV heads of K      */
  int64_t v_block_stride;
  int64_t v_head_stride;
  int32_t num_blocks;
  int32_t num_kv_heads;
  int32_t head_dim;       /* bf16: 64, 96, 128 or 256; fp32: 4 .. 256, % 4   */
  int32_t block_size;     /* must be PACE_KV_BLOCK_TOKENS                    */
  int32_t elem_bytes;     /* 0 or 2: bf16 slabs; 4: fp32 rows (see above)    */
  int32_t reserved;       /* 0                                               */
} pace_kv_pool_t;

/* Text of the last failure on the calling thread ("" if none). */
const char* pace_kv_last_error(void);

/* ABI version; bumped on any signature change. */
int32_t pace_kv_abi_version(void);

/*
 * Append: scatter new tokens into the pool by slot id.
 * Stands behind KVCacheBase.update_cache (pace/llm/cache.py:268-326, 370-400):
 * the reference concatenates / narrow-copies [B,H,T,D] onto its contiguous
 * buffer; here token (b,t) goes to slot_mapping[b*T+t] = block*16 + offset.
 * k_new / v_new: bf16 [batch][num_kv_heads][n_tokens][head_dim] addressed with
 * the element strides given (innermost dim contiguous); a GQA-expanded
 * [B,Hq,T,D] input is deduplicated by passing stride_h * n_rep.
 * slot_mapping: device int64 [batch*n_tokens]; negative = skip the token.
 */
int pace_kv_append(const pace_kv_pool_t* pool, const void* k_new, const void* v_new,
                   int64_t stride_b, int64_t stride_h, int64_t stride_t,
                   int32_t batch, int32_t n_tokens, const int64_t* slot_mapping,
                   void* stream);

/*
 * Append by position: the same scatter, with the destination of token (b,t)
 * resolved on the device as position seq_lens[b] + pos_offset + t of sequence
 * b through the block table, so a decode loop needs no per-step slot upload.
 * (Pass the lengths after the append with pos_offset = -n_tokens, or the
 * lengths before it with pos_offset = 0.)  Positions outside the table row or
 * mapped to a block id outside the pool are skipped.
 */
int pace_kv_append_paged(const pace_kv_pool_t* pool, const void* k_new, const void* v_new,
                         int64_t stride_b, int64_t stride_h, int64_t stride_t,
                         int32_t batch, int32_t n_tokens,
                         const int32_t* block_table, int32_t table_stride,
                         const int32_t* seq_lens, int32_t pos_offset, void* stream);

/*
 * pace_kv_append_paged with one more offset that is read on the device: token (b,t) goes to position
 * seq_lens[b] + pos_offset + *pos_offset_dev + t.  For a decode step captured in a HIP graph, whose
 * lengths advance in a device counter (seq_len_bias_ptr of the attention arguments) while seq_lens and
 * the block table stay as they were captured; the fused append of the attention launch (k_new) does
 * the same for bf16 pools in one launch.  pos_offset_dev == NULL: pace_kv_append_paged.
 */
int pace_kv_append_paged_at(const pace_kv_pool_t* pool, const void* k_new, const void* v_new,
                            int64_t stride_b, int64_t stride_h, int64_t stride_t,
                            int32_t batch, int32_t n_tokens,
                            const int32_t* block_table, int32_t table_stride,
                            const int32_t* seq_lens, int32_t pos_offset,
                            const int32_t* pos_offset_dev, void* stream);

/*
 * Gather: block-table walk back into the reference's dense layout.
 * Produces what the reference cache holds (pace/llm/cache.py:391-399 after
 * repeat_kv, pace/llm/models/llama.py:151-158): k_out / v_out are bf16
 * [batch][num_kv_heads*n_rep][out_len][head_dim] with the element strides
 * given (rows contiguous).  Rows >= seq_lens[b] are written as zeros when
 * zero_fill is non-zero (the reference's BMC buffers are zero-padded,
 * pace/llm/cache.py:255-266) and left untouched otherwise -- in a ragged batch
 * the padding is most of the dense tensor.
 * block_table: device int32 [batch][table_stride]; seq_lens: device int32 [batch]
 * (length of sequence b = seq_lens[b] + seq_len_bias).
 */
int pace_kv_gather(const pace_kv_pool_t* pool, const int32_t* block_table, int32_t table_stride,
                   const int32_t* seq_lens, int32_t seq_len_bias, int32_t batch, int32_t n_rep,
                   void* k_out, void* v_out, int64_t out_stride_b, int64_t out_stride_h,
                   int32_t out_len, int32_t zero_fill, void* stream);

/*
 * Gather without padding: the same rows packed back to back, k_out / v_out bf16
 * [sum of lengths][num_kv_heads*n_rep][head_dim] (contiguous), sequence b starting at row
 * cu_seqlens[b] (device int32 [batch+1], exclusive prefix sum of the lengths).  The rows of a
 * sequence are the rows [b, :, :len_b, :] of the dense form, token-major.  total_tokens: rows of
 * k_out / v_out = cu_seqlens[batch], known to the host that allocated them (it sizes the grid -- one
 * workgroup per block and KV head that can exist, none for padding -- and no row at or past it is written).
 * Same block_table / seq_lens contract as above.
 */
int pace_kv_gather_packed(const pace_kv_pool_t* pool, const int32_t* block_table, int32_t table_stride,
                          const int32_t* seq_lens, int32_t seq_len_bias, const int32_t* cu_seqlens,
                          int32_t batch, int32_t n_rep, void* k_out, void* v_out, int32_t total_tokens,
                          void* stream);

/*
 * The dense form of pace_kv_gather without zero fill (rows past each length are left untouched), launched like the
 * packed form: one workgroup per block that exists, found through cu_seqlens (device int32 [batch + 1], the running
 * sum of the lengths, total_tokens = its last entry).  In a ragged batch most of a dense [out_len] row range lies
 * past the lengths; this launch starts no workgroup for it.
 */
int pace_kv_gather_live(const pace_kv_pool_t* pool, const int32_t* block_table, int32_t table_stride,
                        const int32_t* seq_lens, int32_t seq_len_bias, const int32_t* cu_seqlens, int32_t batch,
                        int32_t n_rep, void* k_out, void* v_out, int64_t out_stride_b, int64_t out_stride_h,
                        int32_t out_len, int32_t total_tokens, void* stream);

/*
 * Copy whole blocks (compaction, beam copy-on-write; the reference's only cache
 * copy of this kind is index_select, pace/llm/cache.py:161-167).
 * pairs: device int32 [n_pairs][2] = (src block, dst block).  When src and dst
 * are the same pool the set of src ids and the set of dst ids must be disjoint.
 */
int pace_kv_copy_blocks(const pace_kv_pool_t* src, const pace_kv_pool_t* dst,
                        const int32_t* pairs, int32_t n_pairs, void* stream);

/*
 * Host-side compaction plan (no GPU work; host arrays).  block_table [batch][table_stride] with
 * n_blocks[b] entries in use per row.  Finds the moves that pack the live blocks into ids 0 .. n_live-1 with
 * the fewest copies (every live block at or above n_live goes to a free id below it), writes them to
 * moves [capacity][2] = (src, dst) -- the layout pace_kv_copy_blocks takes -- and, when apply is non-zero,
 * rewrites the table in place and fills refs [num_blocks] with the owners of every block after the moves.
 * Returns the number of moves, or a negative code.  A block owned by several rows moves once.
 */
int32_t pace_kv_plan_compaction(int32_t* block_table, int32_t table_stride, const int64_t* n_blocks,
                                int32_t batch, int32_t num_blocks, int32_t* moves, int32_t capacity,
                                int32_t apply, int32_t* refs);

/* The second half of pace_kv_plan_compaction on its own: rewrite the table for moves [n_moves][2] whose data
 * is being copied, and count the owners of every block into refs [num_blocks].  (Planning, starting the copy
 * and then applying lets the host's table rewrite run while the GPU copies.) */
int pace_kv_apply_moves(int32_t* block_table, int32_t table_stride, const int64_t* n_blocks, int32_t batch,
                        int32_t num_blocks, const int32_t* moves, int32_t n_moves, int32_t* refs);

/*
 * Compaction in one call: pace_kv_plan_compaction (apply = 0; with is_free != NULL: pace_kv_plan_compaction_flags,
 * below) into moves_host [capacity][2], the upload of the
 * moves to moves_dev (device memory for as many pairs) and pace_kv_copy_blocks for each of the n_pools pools that
 * share the table (the layers of a model), all on `stream`.  Returns the number of moves or a negative code.
 * Afterwards the caller rewrites its table with pace_kv_apply_moves(moves_host, returned count) -- on the host,
 * while the copies run.  moves_host should be pinned memory (else the upload waits for the stream) and must stay
 * untouched until the upload has run.  Like compaction as a whole, this has no counterpart in the reference, whose
 * caches are dense tensors (pace/llm/cache.py:161-167 is its only copy between cache rows).
 */
int32_t pace_kv_compact_blocks(const pace_kv_pool_t* const* pools, int32_t n_pools, const int32_t* block_table,
                               int32_t table_stride, const int64_t* n_blocks, int32_t batch, const uint8_t* is_free,
                               int32_t* moves_host, int32_t capacity, int32_t* moves_dev, void* stream);

/*
 * The plan of pace_kv_plan_compaction from the allocator's own record of the pool instead of the table: is_free
 * [num_blocks], one byte per block id, non-zero = free (every id the table names must be marked used).  The same
 * moves in the same order; a pass over num_blocks bytes instead of a walk over every table entry.
 */
int32_t pace_kv_plan_compaction_flags(const uint8_t* is_free, int32_t num_blocks, int32_t* moves, int32_t capacity);

/*
 * pace_kv_apply_moves with the allocator's bookkeeping moved along instead of recounted: refs [num_blocks] (owners
 * per block) and is_free [num_blocks] (1 = free, 0 = used) are updated in place -- a moved block takes its owners
 * with it, its old id becomes free -- and the free list is written afresh into free_stack [num_blocks]: *n_free ids,
 * the lowest id last (the stack's top).  Every move must take a used id to a free one and no id may occur twice
 * (else PACE_KV_EINVAL and nothing is changed).
 */
int pace_kv_apply_moves_tracked(int32_t* block_table, int32_t table_stride, const int64_t* n_blocks, int32_t batch,
                                int32_t num_blocks, const int32_t* moves, int32_t n_moves, int32_t* refs,
                                uint8_t* is_free, int32_t* free_stack, int32_t* n_free);

/*
 * Rotary position embedding, the step the models run on q and k right before the
 * append (pace/llm/models/llama.py:147-158; operator pace/ops/rotary_embedding.py:370-474).
 * cos / sin: device tables [table_rows][rotary_dim/2] as RotaryEmbedding builds them
 * (cos_cache / sin_cache, pace/ops/rotary_embedding.py:366-367), bf16 or fp32; fp32 entries
 * are rounded to bf16 on load, which is what forward()'s `.to(x.dtype)` does (:399-400).
 * Token t of sequence b uses table row positions[b*pos_stride_b + t]; with positions == NULL
 * the row is the token's position in its sequence.  Rows outside the table are clamped.
 * The first rotary_dim dims of every head row are rotated, the rest pass through
 * (:421-430; pace/llm/models/gptj.py:115-131).  Results are bit-identical to the reference's
 * bf16 tensor arithmetic (each product and the sum rounded separately).
 */
typedef struct pace_rope {
  const void* cos;
  const void* sin;
  int32_t table_dtype;   /* PACE_DTYPE_BF16 / PACE_DTYPE_F32                              */
  int32_t table_rows;
  int32_t rotary_dim;    /* multiple of 16, <= head_dim                                   */
  int32_t interleaved;   /* 0: neox style, dim i pairs with i + rotary_dim/2 (is_neox_style=True);
                            1: GPT-J style, dim 2i pairs with 2i+1                         */
  const int32_t* positions; /* optional device int32 [batch][tokens]                      */
  int32_t pos_stride_b;
} pace_rope_t;

/*
 * RotaryEmbedding.apply_rotary_emb on dense tensors (pace/ops/rotary_embedding.py:445-474):
 * q [batch][num_q_heads][n_tokens][head_dim] and k [batch][num_k_heads][n_tokens][head_dim],
 * bf16, element strides given (innermost contiguous), rotated into q_out / k_out (same
 * strides; may alias the inputs).  Either tensor may be NULL.  rope->positions is required.
 */
int pace_rope_apply(const pace_rope_t* rope, const void* q, void* q_out,
                    int64_t q_stride_b, int64_t q_stride_h, int64_t q_stride_t, int32_t num_q_heads,
                    const void* k, void* k_out,
                    int64_t k_stride_b, int64_t k_stride_h, int64_t k_stride_t, int32_t num_k_heads,
                    int32_t batch, int32_t n_tokens, int32_t head_dim, void* stream);

/*
 * The same operator on fp32 tensors (the reference's operator takes any float dtype and casts cos / sin to it,
 * pace/ops/rotary_embedding.py:398-399): q / k / outputs fp32, rope->cos / sin fp32 tables, any even head_dim and
 * rotary_dim.  Each product and the sum are rounded separately, as the tensor operations round them.
 */
int pace_rope_apply_f32(const pace_rope_t* rope, const void* q, void* q_out,
                        int64_t q_stride_b, int64_t q_stride_h, int64_t q_stride_t, int32_t num_q_heads,
                        const void* k, void* k_out,
                        int64_t k_stride_b, int64_t k_stride_h, int64_t k_stride_t, int32_t num_k_heads,
                        int32_t batch, int32_t n_tokens, int32_t head_dim, void* stream);

/*
 * Rotate-and-append in one launch: the rope(q, k) + update_cache(k, v) sequence of
 * pace/llm/models/llama.py:147-158.  q is rotated into q_out (may alias q; NULL q = keys
 * only); k_new is rotated and stored, v_new stored, at positions seq_lens[b] + pos_offset + t
 * through the block table exactly as pace_kv_append_paged does.  With rope->positions == NULL
 * the same position selects the table row.  k_new / v_new are not modified.
 */
int pace_rope_append_paged(const pace_kv_pool_t* pool, const pace_rope_t* rope,
                           const void* q, void* q_out,
                           int64_t q_stride_b, int64_t q_stride_h, int64_t q_stride_t, int32_t num_q_heads,
                           const void* k_new, const void* v_new,
                           int64_t stride_b, int64_t stride_h, int64_t stride_t,
                           int32_t batch, int32_t n_tokens,
                           const int32_t* block_table, int32_t table_stride,
                           const int32_t* seq_lens, int32_t pos_offset, void* stream);

typedef struct pace_paged_attn_args {
  const void* q;          /* bf16 [batch][num_q_heads][q_len][head_dim]               */
  int64_t q_stride_b, q_stride_h, q_stride_s; /* elements; innermost contiguous      */
  void* out;              /* bf16, same logical shape as q                            */
  int64_t o_stride_b, o_stride_h, o_stride_s;
  const int32_t* block_table; /* device int32 [batch][table_stride]                  */
  int32_t table_stride;
  const int32_t* seq_lens;    /* device int32 [batch]; length of sequence b = seq_lens[b] + seq_len_bias:
                                 tokens in cache incl. the q_len new ones                */
  const int32_t* kv_start;    /* optional device int32 [batch]: first readable token (left padding) */
  const void* mask;           /* optional additive mask [batch|1][1][q_len|1][mask_len]  */
  int32_t mask_dtype;         /* PACE_DTYPE_F32 / PACE_DTYPE_BF16                      */
  int32_t mask_len;           /* columns in the mask; tokens >= mask_len are masked    */
  int64_t mask_stride_b, mask_stride_s; /* elements; 0 for a broadcast dim            */
  int32_t batch, num_q_heads, q_len;
  int32_t causal;             /* 1: query row s reads tokens <= seq_len - q_len + s    */
  int32_t max_seq_len;        /* host-side upper bound of seq_lens (sizes the grid)    */
  int32_t partition_tokens;   /* context split size per workgroup, multiple of 32; 0 = auto   */
  float scale;                /* softmax scale (> 0), reference uses 1/sqrt(head_dim)  */
  void* workspace;            /* device scratch, >= pace_paged_attn_workspace_bytes()  */
  size_t workspace_bytes;
  /* Optional fused append (NULL = off).  The last n_new (1..32) tokens of every sequence, i.e.
   * positions seq_len - n_new .. seq_len - 1, are read from k_new / v_new
   * [batch][num_kv_heads][n_new][head_dim] (element strides below, innermost contiguous) instead
   * of from the pool, and this launch also stores them into their pool slots through the block
   * table, so no separate append launch is needed for them.  Same contract as pace_kv_append_paged
   * with pos_offset = -n_new. */
  const void* k_new;
  const void* v_new;
  int64_t new_stride_b, new_stride_h, new_stride_t;
  int32_t n_new;
  /* Optional work list (NULL = a dense partition x sequence grid whose partitions the kernel derives from
   * each length and partition_tokens).  Device int32 [n_work_items][PACE_ATTN_WORK_INTS], one descriptor per
   * (sequence, partition) in the order they should be scheduled, as pace_paged_attn_plan() writes them (layout
   * below).  A descriptor carries the partition's token range and the pool blocks of its first units, so a
   * workgroup's first K / V loads wait for one 64-byte read instead of the length -> block table -> K / V chain;
   * the ranges are fixed by the host, and only the last partition of a sequence (open ended) grows with it.
   * The list stays valid while the lengths only grow and the block-table entries below the planned lengths
   * keep their values (appends qualify; rollback, eviction, compaction and beam forks need a new plan).
   * With a work list, seq_parts (device int32 [batch]: partitions of each sequence) and max_parts (its
   * largest entry) are required, and the workspace is sized by pace_paged_attn_workspace_bytes_for_parts(). */
  const int32_t* work_items;
  int32_t n_work_items;
  const int32_t* seq_parts;
  int32_t max_parts;
  int32_t seq_len_bias;       /* host-side constant added to every seq_lens entry, so that uniform
                                 appends / rollbacks need no device update of the lengths */
  /* Optional rotary embedding folded into the launch (NULL = off; needs rotary_dim == head_dim).
   * q holds the un-rotated queries: each row is rotated as it is loaded.  With the fused append,
   * k_new holds the un-rotated keys: they are rotated before they are attended to and stored
   * (n_new must equal q_len).  Positions: rope->positions [batch][q_len], or NULL for
   * seq_len - q_len + s.  One launch then covers rope + append + attention of
   * pace/llm/models/llama.py:147-165. */
  const pace_rope_t* rope;
  /* Optional device int32 (NULL = off) added to every length like seq_len_bias.  A decode step captured
   * into a HIP graph bakes in every host-side argument; with this the graph itself can advance the
   * lengths between replays (a one-element increment kernel inside the graph).  max_seq_len must then
   * bound the lengths over all replays, and the block table must already hold their blocks. */
  const int32_t* seq_len_bias_ptr;
} pace_paged_attn_args_t;

/* The context split size (tokens per workgroup) the library uses for these sizes when
 * partition_tokens is 0; a sequence of n tokens is cut into ceil(n / split) equal partitions. */
int32_t pace_paged_attn_partition_tokens(int32_t batch, int32_t num_q_heads, int32_t q_len,
                                         int32_t head_dim, int32_t max_seq_len,
                                         int32_t partition_tokens, int32_t num_kv_heads);

/*
 * Work descriptor of one (sequence, partition), PACE_ATTN_WORK_INTS int32:
 *   [0] sequence   [1] partition index   [2] partitions of the sequence
 *   [3] first token (multiple of 32)     [4] one past the last token, -1 = up to the sequence's length
 *   [5] n: how many of the unit entries below are set   [6..7] 0
 *   [8 + 2u], [9 + 2u], u < PACE_ATTN_WORK_FIRST_UNITS: pool block ids of tokens first + 32u .. first + 32u + 31
 *       (set for the leading units that lay wholly below the planned length)
 */
#define PACE_ATTN_WORK_INTS 16
#define PACE_ATTN_WORK_FIRST_UNITS 4

typedef struct pace_attn_plan {
  int32_t n_work_items;     /* descriptors written (or needed, when the capacity was too small)  */
  int32_t max_parts;        /* largest entry of seq_parts                                        */
  int32_t partition_tokens; /* the split size the cut started from (informational)               */
  int32_t reserved;
  size_t workspace_bytes;   /* scratch a launch with this plan needs                             */
} pace_attn_plan_t;

/*
 * Host-side planner for one attention launch; no GPU work, every pointer is host memory.  It stands where the
 * reference has nothing: its attention walks one contiguous [B, H, L, D] tensor per call
 * (csrc/ops/kernels/attention_kernels.cpp:218-257).  seq_lens [batch]: the lengths the launch will see
 * (new tokens included); block_table [batch][table_stride]: the host copy of the table.  Cuts every sequence
 * into equal partitions of whole 32-token units -- at partition_tokens (0: chosen from the sizes; a ragged
 * batch is cut at about its mean length), or, when the whole launch fits the GPU in one round, into the
 * partition counts that make the partitions most equal -- and writes the descriptors to work_items
 * (capacity in descriptors; longest partitions first in a ragged batch) and the counts to seq_parts [batch].
 * masked: the launch will carry an explicit mask (changes the launch shape).  The caller uploads both
 * arrays and passes them, with plan->max_parts and plan->n_work_items, in pace_paged_attn_args_t.
 */
int pace_paged_attn_plan(const int32_t* seq_lens, const int32_t* block_table, int32_t table_stride,
                         int32_t batch, int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                         int32_t q_len, int32_t masked, int32_t partition_tokens,
                         int32_t* work_items, int32_t work_capacity, int32_t* seq_parts,
                         pace_attn_plan_t* plan);

/* Name of the kernel instantiation pace_paged_attn_decode / _verify would launch for these arguments, as a
 * profiler prints it (nothing is launched): lets a measurement be tied to the kernel it was taken on. */
int pace_paged_attn_kernel_name(const pace_kv_pool_t* pool, const pace_paged_attn_args_t* args,
                                char* out, size_t out_bytes);

/* Scratch bytes the two entry points below need for these sizes (0 = none): the partial results
 * of sequences cut into several partitions and, for launches of more than 64 query rows per KV
 * head, two int32 per (sequence, query token) in which a launch with an explicit mask keeps a
 * summary of the mask (the last column each row can use; the first one, if the row's mask line is
 * 0 over one stretch of columns and at the floor elsewhere).  The partials are required; a
 * workspace without room for the summary is accepted: the launch then walks every column (no room
 * for the first int) or reads the mask values of every unit (no room for the second). */
size_t pace_paged_attn_workspace_bytes(int32_t batch, int32_t num_q_heads, int32_t q_len,
                                       int32_t head_dim, int32_t max_seq_len,
                                       int32_t partition_tokens, int32_t num_kv_heads);

size_t pace_paged_attn_workspace_bytes_for_parts(int32_t batch, int32_t num_q_heads, int32_t q_len,
                                                 int32_t head_dim, int32_t max_parts);

/*
 * Decode attention over the paged cache, q_len == 1.
 * Stands behind MultiHeadAttention.forward -> backend.execute
 * (pace/ops/attention.py:29-38, pace/ops/backends/native.py:44-47,
 * pace/ops/backends/jit.py:43-47) for one new token per sequence.
 */
int pace_paged_attn_decode(const pace_kv_pool_t* pool, const pace_paged_attn_args_t* args, void* stream);

/*
 * Multi-token (speculative verify / chunked prefill) attention over the paged
 * cache: q_len >= 1 new tokens per sequence already appended; causal among
 * themselves (the mask pace/llm/models/llama.py:292-299 builds for q_len > 1).
 */
int pace_paged_attn_verify(const pace_kv_pool_t* pool, const pace_paged_attn_args_t* args, void* stream);

/*
 * pace_paged_attn_verify (any q_len >= 1, so decode too) for callers that cannot allocate device memory:
 * code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart
 * in the reference.  args->workspace / workspace_bytes are ignored; the partial results of sequences cut
 * into several partitions (and the per-row mask summary of prefill-sized masked launches) live in an array of
 * PACE_PAGED_ATTN_STATIC_SCRATCH_BYTES that is part of the library's device image -- every GPU the library
 * runs on holds one copy until the process ends.  A launch that needs more (see
 * pace_paged_attn_workspace_bytes*) is refused with PACE_KV_EINVAL and nothing is launched.  The call
 * allocates and frees nothing.  All calls on one GPU share that GPU's array: calls that may overlap there
 * (different streams, different threads) race; order them on one stream.  Nothing in the array needs
 * clearing between calls: every partial a launch reads, it has written.
 * Under graph capture: the array's address is looked up once per device, on the first attention call of any
 * entry point there (pace_paged_attn_decode / _verify / _verify_static).  Run one attention step eagerly on the
 * device before capturing -- the warm-up step every capture needs anyway -- so that the look-up is not recorded.
 */
#define PACE_PAGED_ATTN_STATIC_SCRATCH_BYTES (32u << 20)
int pace_paged_attn_verify_static(const pace_kv_pool_t* pool, const pace_paged_attn_args_t* args, void* stream);

/*
 * Dense attention: body of the torch op
 *   pace::attention(Tensor input_Q, Tensor input_K, Tensor input_V,
 *                   Tensor? input_mask, Scalar? use_KQ) -> Tensor
 * (csrc/ops/attention.cpp:18-108; kernel csrc/ops/kernels/attention_kernels.cpp:162-257).
 * q [B][N][S][H], k/v [B][N][L][H] and out [B][N][S][H] are dense row-major as
 * the reference requires (csrc/pace_tensor/pace_aten_interface.cpp:151-179);
 * mask is an additive [mB][mN][mS][L] tensor, each of mB/mN/mS either 1 or the
 * full extent.  qkv_dtype / mask_dtype: PACE_DTYPE_*.  out has qkv_dtype.
 */
int pace_attn_dense(const void* q, const void* k, const void* v, void* out,
                    int32_t qkv_dtype, int32_t B, int32_t N, int32_t S, int32_t L, int32_t H,
                    const void* mask, int32_t mask_dtype, int32_t mB, int32_t mN, int32_t mS,
                    void* stream);

/*
 * The same op (csrc/ops/attention.cpp:18-108) with scratch memory of the caller's: `workspace` (4-byte
 * aligned, pace_attn_dense_workspace_bytes() of these sizes, device memory) lets a prefill-sized bf16 launch
 * with a mask look over the mask once before the attention kernel -- where its lines are 0 over one stretch
 * of columns and at the floor elsewhere (a causal mask, padded or not) the rows are then walked by that
 * stretch and the mask is not read again.  Results are the same up to rounding (the weights of such rows
 * are formed as exp2((qk - max) * scale * log2 e) instead of exp2((qk * scale + 0 - max) * log2 e)).
 * A NULL or short workspace is accepted: the call is then pace_attn_dense.
 */
size_t pace_attn_dense_workspace_bytes(int32_t qkv_dtype, int32_t S, int32_t H, int32_t has_mask,
                                       int32_t mB, int32_t mN, int32_t mS);
int pace_attn_dense_ws(const void* q, const void* k, const void* v, void* out,
                       int32_t qkv_dtype, int32_t B, int32_t N, int32_t S, int32_t L, int32_t H,
                       const void* mask, int32_t mask_dtype, int32_t mB, int32_t mN, int32_t mS,
                       void* workspace, size_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* PACE_KV_HIP_H */
