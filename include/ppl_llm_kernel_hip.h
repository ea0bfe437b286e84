/*
 * C ABI of the MI355X (gfx950) kernel library behind the llm_hip engine's dynamic-batching attention path.
 *
 * It takes the place of the un-vendored C++ library `ppl.llm.kernel.cuda` that the reference engine calls from
 *   src/ppl/nn/engines/llm_cuda/kernels/opmx/dynamic_batching/multi_head_cache_attention_kernel.cc:170-230
 *   (`dynamic_batching_multi_head_cache_attention::heuristic_prepare` + `forward`), and from
 *   src/ppl/nn/engines/llm_cuda/kernels/opmx/dynamic_batching/key_value_cache_kernel.cc:23-114 (a stub there).
 *
 * Conventions: plain pointers and sizes only; every pointer named `d_*` or documented "device" is a device
 * address valid on the current HIP device; `stream` is a `hipStream_t` passed as `void*` (NULL = default stream);
 * every function returns a `pplhip_retcode` and enqueues work asynchronously on `stream` unless it says otherwise.
 * Nothing here allocates device memory: the caller owns the KV slab, the tables, the outputs and the workspace.
 */
#ifndef PPL_LLM_KERNEL_HIP_H_
#define PPL_LLM_KERNEL_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Same meaning (and order) as the ppl::common::RetCode values the reference wrappers return
 * (src/ppl/nn/engines/llm_cuda/kernels/opmx/dynamic_batching/multi_head_cache_attention_kernel.cc:90-166). */
typedef enum pplhip_retcode {
    PPLHIP_RC_SUCCESS = 0,
    PPLHIP_RC_OTHER_ERROR = 1,
    PPLHIP_RC_UNSUPPORTED = 2,
    PPLHIP_RC_OUT_OF_MEMORY = 3,
    PPLHIP_RC_INVALID_VALUE = 4,
    PPLHIP_RC_EXISTS = 5,
    PPLHIP_RC_NOT_FOUND = 6,
    PPLHIP_RC_PERMISSION_DENIED = 7,
    PPLHIP_RC_HOST_MEMORY_ERROR = 8,
    PPLHIP_RC_DEVICE_MEMORY_ERROR = 9,
    PPLHIP_RC_DEVICE_RUNTIME_ERROR = 10,
    PPLHIP_RC_OUT_OF_RANGE = 11,
    PPLHIP_RC_INTERNAL_ERROR = 12
} pplhip_retcode;

/* Human-readable text of the last error raised on the calling thread ("" if none). Never NULL. */
const char* pplhip_last_error(void);

/* Library/ABI version: major*10000 + minor*100 + patch. */
int32_t pplhip_version(void);

/* Optional, once per process with the GPU current (the reference engine's counterpart is the device set-up in
 * src/ppl/nn/engines/llm_cuda/llm_cuda_device.cc:60-100): reads the current device's compute-unit count, which sizes
 * the decode plan. Without it pplhip_mhca_prepare plans for the 256 compute units of MI355X. Touches the device. */
pplhip_retcode pplhip_init(void);

/*
 * Argument block of MultiHeadCacheAttention: one field per argument the reference passes to `heuristic_prepare`
 * (multi_head_cache_attention_kernel.cc:170-212), in the same order and with the same meaning.
 *
 * Tensors (fp16 = IEEE binary16, NDARRAY, contiguous):
 *   query         fp16 [S, num_heads, head_dim]       S = seqstarts[batch] packed new tokens
 *   current_key   fp16 [S, num_kv_heads, head_dim]
 *   current_value fp16 [S, num_kv_heads, head_dim]
 *   seqstarts     i64  [batch+1]   prefix sums of new-token counts, seqstarts[0] = 0
 *   kvstarts      i64  [batch+1]   prefix sums of kv lengths (start_pos + seqlen), kvstarts[0] = 0
 *   cachestarts   i64  [batch]     first slab token of each sequence (cache_mode 0), or
 *                      [batch, cachestart_stride_b] first slab token of every PAGE of each sequence (cache_mode 1):
 *                      token j of sequence b lives at slab token cachestarts[b][j / page_size] + j % page_size
 *                      (page table laid out as in tools/benchmark_llama/generation_state.cc:111-117);
 *                      page_size must be a power of two >= 64
 *   start_pos     i64  [batch]     tokens already cached before this call
 *   cache         i8   element (tok, layer, kv, head, d) at
 *                      tok*cache_stride_s + layer*cache_stride_l + kv*cache_stride_kv + head*cache_stride_h + d
 *   scale         fp16 one per group of 8 channels; element strides are the cache strides divided by 8
 *   output        fp16 [S, num_heads, head_dim]
 * Sequences [0, decoding_batches) are decode steps (exactly one new token each) and attend over the int8 cache,
 * the just-written token included; sequences [decoding_batches, batch) are prefill and attend over the fp16
 * current_key/current_value (or over the cache when cache_prefill != 0, which also allows start_pos > 0).
 * Without cache_prefill a prefill sequence's keys are exactly its seqlen new tokens on every kernel path: cached
 * history (start_pos > 0) is not attended to, although its new tokens are still written behind it in the slab and
 * kvstarts still places the sequence's columns in an attn_mask.
 */
typedef struct pplhip_mhca_args {
    const void* d_query;
    const void* d_current_key;
    const void* d_current_value;
    const void* d_attn_mask; /* optional additive fp16 mask (NULL: none), see attn_mask_stride_* below */
    const int64_t* d_seqstarts;
    const int64_t* d_kvstarts;
    const int64_t* d_cachestarts;
    const int64_t* d_start_pos;
    const void* d_alibi_slopes; /* must be NULL: the reference rejects is_alibi (…_kernel.cc:95-98) */
    int32_t is_causal;
    int64_t batch;
    int64_t decoding_batches;
    int64_t max_seqlen;
    int64_t max_kvlen;
    int32_t layer_idx;
    int32_t num_layer;
    int32_t num_heads;
    int32_t num_kv_heads;
    int32_t head_dim;
    int32_t cache_mode; /* 0 = contiguous region per sequence; 1 = paged (see cachestarts above) */
    int32_t page_size;
    int64_t cache_stride_s;
    int64_t cache_stride_l;
    int64_t cache_stride_h;
    int64_t cache_stride_kv;
    int64_t cachestart_stride_b;
    /* engine knobs, same values as EngineConfig (src/ppl/nn/engines/llm_cuda/engine_config.h:25-36) */
    int32_t enable_cache_prefill;
    int32_t enable_decoding_sharemem_mhca; /* accepted, ignored: one decode algorithm serves every shape */
    int32_t enable_decoding_infinity_mhca; /* accepted, ignored */
    int32_t enable_decoding_infinity_gqca; /* accepted, ignored */
    int32_t specify_decoding_attn_split_k; /* 0 coarsest split (1 range per workgroup slot), 1 heuristic, 2 finest */
    int32_t specify_decoding_attn_tpb; /* 0 heuristic, 256, 512 */
    void* d_cache;
    void* d_scale;
    void* d_output;
    int64_t total_new_tokens; /* S = query dim 0 (the reference passes the query TensorShape) */
    /* attn_mask (the reference passes its TensorShape, …_kernel.cc:105-110,178-179): the value added to the scaled score
     * of query token t (of sequence b, head h) and key j of that sequence is
     *     mask[h * attn_mask_stride_h + (seqstarts[b] + t) * attn_mask_stride_q + kvstarts[b] + j]
     * i.e. a [S, >= kvstarts[batch]] matrix over packed query tokens x packed keys (stride_q = its last extent, which
     * exporters pad to a multiple of 8), one per head or, with attn_mask_stride_h == 0, one for all heads. It is
     * applied in addition to is_causal. -inf entries mask a key out; a row with every key masked yields zeros.
     * The layout is this library's definition: the reference's CUDA kernel, which would fix it, is not in its tree. */
    int64_t attn_mask_stride_h;
    int64_t attn_mask_stride_q;
} pplhip_mhca_args;

/* What `heuristic_prepare` stores in the reference kernel object's `.cfg` (…_kernel.cc:218-228 reads
 * `cfg.workspace_size` and sets `cfg.workspace`). Filled by pplhip_mhca_prepare, consumed by pplhip_mhca_forward. */
typedef struct pplhip_mhca_plan {
    uint64_t workspace_bytes; /* device scratch the caller must pass to forward (may be 0) */
    int32_t decode_num_ranges; /* S: the cached tokens of all decode sequences, laid end to end, are cut into S equal
                                  ranges on the device (split-k granularity); one workgroup per range and head group */
    int32_t decode_heads_per_block; /* kv heads served by one decode workgroup (1, 2 or 4) */
    int32_t decode_waves_per_block;
    int32_t prefill_q_tile; /* query rows per prefill workgroup */
    int32_t prefill_num_q_tiles; /* ceil(max_seqlen / prefill_q_tile) */
    int32_t prefill_staging; /* cache-prefill only: 1 = the prompts' cached K/V are first dequantised into fp16 staging
                                rows in the workspace (one streaming pass) and attention runs over those; 0 = the
                                attention kernel dequantises the int8 slab itself (small chunks, or staging too large).
                                The caller may clear it before forward to stay on the second route. */
    int32_t prefill_staging_offset_256; /* where the staging rows start in the workspace, in units of 256 bytes */
    int32_t general_kernel; /* 1 = the call runs the general attention kernel (head_dim other than 128, more than 16
                               query heads per kv head, or an attn_mask): write kernel + one attention launch. With
                               decode_num_ranges > 0 (head_dim 64 / 32 whose kv heads are neighbours in the slab and
                               pair up / go in fours, no mask) the decode sequences of such a call run the decode
                               kernel over those groups of kv heads and the general kernel takes the prompts. */
    int32_t general_decode_splits; /* general kernel only: pieces the longest decode sequence's keys (max_kvlen) are
                                      cut into, shorter sequences into as many pieces of that length as they fill
                                      (partial results go through the workspace and a merge launch); 0 or 1 = none.
                                      The caller may lower it before forward. */
} pplhip_mhca_plan;

/* Host-only: validates `args` exactly like the reference wrapper + kernel library would
 * (unsupported attrs -> PPLHIP_RC_UNSUPPORTED, inconsistent sizes -> PPLHIP_RC_INVALID_VALUE),
 * picks the split-k decomposition (how many equal token ranges) and reports the workspace size. Replaces `heuristic_prepare`
 * (multi_head_cache_attention_kernel.cc:170). Makes no HIP call and reads no environment: the plan depends on `args`
 * and on the compute-unit count recorded by pplhip_init() (256 before it) only. */
pplhip_retcode pplhip_mhca_prepare(const pplhip_mhca_args* args, pplhip_mhca_plan* plan);

/* Enqueues: quantize-on-write of the new K/V tokens, decode attention (+ split-k merge) for the first
 * `decoding_batches` sequences and causal prefill attention for the rest. Replaces `forward(stream)`
 * (multi_head_cache_attention_kernel.cc:230). `d_workspace` must hold plan->workspace_bytes (256-byte aligned).
 * As in the reference, the decode sequences come first and bring exactly one new token each (their packed token
 * index is their sequence index); which kernel quantises which new token into the cache is an implementation detail. */
pplhip_retcode pplhip_mhca_forward(const pplhip_mhca_args* args, const pplhip_mhca_plan* plan, void* d_workspace,
                                   void* stream);

/*
 * pplhip_mhca_forward for callers that cannot allocate device memory or bring a workspace (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc). It has no counterpart in the reference. The split-k
 * partial results go to an array that is part of the library's device image (16 MiB on every GPU the library runs on,
 * held until the process ends); the call allocates nothing and frees nothing. Limits: plan->workspace_bytes must not
 * exceed 16 MiB (PPLHIP_RC_OUT_OF_RANGE otherwise; every configuration named in this header's examples needs under
 * 7 MiB) and plan->prefill_staging must be 0 (PPLHIP_RC_UNSUPPORTED: staging rows need a caller-owned workspace).
 * All calls on one GPU share that GPU's array: calls that overlap in time on one GPU (two streams, two threads) race
 * on it and must be serialised by the caller; calls on different GPUs are independent.
 */
pplhip_retcode pplhip_mhca_forward_noalloc(const pplhip_mhca_args* args, const pplhip_mhca_plan* plan, void* stream);

/*
 * Quantize-on-write alone: new token t of sequence b goes to slab token cachestarts[b] + start_pos[b] + t.
 * Per (token, K|V, kv head, group of 8 channels): scale = max(fp16(absmax / 127), fp16(1e-5)),
 * q = int8(rint(fp16(x / scale))). This is the first step of the reference's fused `forward`.
 */
typedef struct pplhip_kv_write_args {
    const void* d_current_key; /* fp16 [S, num_kv_heads, head_dim] */
    const void* d_current_value;
    const int64_t* d_seqstarts; /* [batch+1] */
    const int64_t* d_cachestarts; /* [batch] */
    const int64_t* d_start_pos; /* [batch] */
    int64_t batch;
    int64_t total_new_tokens; /* S */
    int32_t layer_idx;
    int32_t num_layer;
    int32_t num_kv_heads;
    int32_t head_dim;
    int64_t cache_stride_s;
    int64_t cache_stride_l;
    int64_t cache_stride_h;
    int64_t cache_stride_kv;
    void* d_cache;
    void* d_scale;
    int32_t cache_mode; /* as in pplhip_mhca_args */
    int32_t page_size;
    int64_t cachestart_stride_b;
} pplhip_kv_write_args;

pplhip_retcode pplhip_kv_quantize_write(const pplhip_kv_write_args* args, void* stream);

/*
 * opmx.dynamic_batching::KeyValueCache (inputs/outputs of
 * src/ppl/nn/engines/llm_cuda/kernels/opmx/dynamic_batching/key_value_cache_kernel.cc:26-39, which is a stub that
 * returns RC_UNSUPPORTED in the reference): quantize-on-write as above, then key/value outputs
 * fp16 [kvstarts[batch], num_kv_heads, head_dim] = the dequantised cache rows of every sequence in batch order.
 * `total_kv_tokens` = kvstarts[batch] (the reference reads it back for shape inference,
 * src/ppl/nn/oputils/opmx/reshape_dynamic_batching_key_value_cache.cc:43-53).
 */
typedef struct pplhip_kv_cache_args {
    pplhip_kv_write_args write;
    const int64_t* d_kvstarts; /* [batch+1] */
    int64_t total_kv_tokens;
    int64_t max_kvlen;
    int32_t num_repeat; /* only 1 (key_value_cache_kernel.cc:93-96) */
    int32_t cache_mode; /* only 0 */
    int32_t cache_layout; /* only 0 */
    int32_t reserved;
    void* d_key_out;
    void* d_value_out;
} pplhip_kv_cache_args;

pplhip_retcode pplhip_kv_cache_forward(const pplhip_kv_cache_args* args, void* stream);

/*
 * opmx.dynamic_batching::MultiHeadAttention (no cache): the argument list of
 * `ppl::kernel::llm::cuda::pmx::dynamic_batching_multi_head_attention` as called from
 * src/ppl/nn/engines/llm_cuda/kernels/opmx/dynamic_batching/multi_head_attention_kernel.cc:105-127.
 *   query  fp16 [seqstarts[batch], num_heads, head_dim]
 *   key    fp16 [kvstarts[batch], num_kv_heads, head_dim]   all keys of every sequence, packed in batch order
 *   value  fp16 [kvstarts[batch], num_kv_heads, head_dim]
 *   output fp16 [seqstarts[batch], num_heads, head_dim]
 * The queries of a sequence are its LAST seqlen keys: with is_causal, query i of sequence b attends to keys
 * 0 .. (kvlen_b - seqlen_b) + i; without, to all kvlen_b keys. kvlen_b >= seqlen_b >= 1 is required.
 * MultiHeadCacheAttention == MultiHeadAttention applied to the outputs of KeyValueCache.
 * head_dim: a multiple of 16 up to 256 (128 with at most 16 query heads per kv head and no mask runs the tuned kernel,
 * everything else the general one); no alibi.
 */
typedef struct pplhip_mha_args {
    const void* d_query;
    const void* d_key;
    const void* d_value;
    const void* d_attn_mask; /* optional additive fp16 mask, laid out as for pplhip_mhca_args */
    const int64_t* d_seqstarts; /* [batch+1] */
    const int64_t* d_kvstarts; /* [batch+1] */
    int32_t is_causal;
    int32_t is_alibi; /* must be 0: RC_UNSUPPORTED otherwise (multi_head_attention_kernel.cc:71-74) */
    int64_t batch;
    int64_t decoding_batches; /* accepted for interface parity; every sequence takes the same path */
    int64_t max_seqlen;
    int64_t max_kvlen;
    int32_t num_heads;
    int32_t num_kv_heads;
    int32_t head_dim;
    int32_t reserved;
    void* d_output;
    int64_t attn_mask_stride_h;
    int64_t attn_mask_stride_q;
} pplhip_mha_args;

pplhip_retcode pplhip_mha_forward(const pplhip_mha_args* args, void* stream);

/*
 * opmx.dynamic_batching::RotaryPositionEmbedding: the argument list of
 * `ppl::kernel::llm::cuda::pmx::dynamic_batching_rotary_position_embedding` as called from
 * src/ppl/nn/engines/llm_cuda/kernels/opmx/dynamic_batching/rotary_position_embedding_kernel.cc:110-132.
 *   query / rotated_query  fp16 [total_tokens, num_heads, head_dim]
 *   key   / rotated_key    fp16 [total_tokens, num_key_heads, head_dim]     (outputs may alias the inputs)
 * Token t of sequence b has position start_pos[b] + (t - seqstarts[b]); pair i (0 <= i < rotary_dim / 2) of a head row
 * is rotated by the angle position * theta^(-2i / rotary_dim):
 *     y[lo] = x[lo] cos - x[hi] sin,   y[hi] = x[hi] cos + x[lo] sin.
 * Which two channels form pair i is `pair_layout` (the reference's CUDA kernel is not in its tree, so neither
 * convention can be pinned against it; an integrator picks the one the model was exported for):
 *     PPLHIP_ROPE_PAIRS_INTERLEAVED  (lo, hi) = (2i, 2i + 1)               -- complex-number layout of the original
 *                                                                              LLaMA weights
 *     PPLHIP_ROPE_PAIRS_HALF_SPLIT   (lo, hi) = (i, i + rotary_dim / 2)    -- "rotate_half" layout of weights whose
 *                                                                              q/k projections were permuted for it
 * channels >= rotary_dim are copied; `bypass_key` copies the key unrotated. rotary_dim 0 means head_dim.
 * scaling_type: the values of RotaryPositionEmbeddingParam (src/ppl/nn/params/opmx/rotary_position_embedding_param.h:
 * 12-16). LINEAR divides the position by scaling_factor. DYNAMIC, for a sequence whose total length
 * T = start_pos + seqlen exceeds max_position_embeddings, replaces theta by
 * theta * (scaling_factor * T / max_position_embeddings - (scaling_factor - 1)) ^ (rotary_dim / (rotary_dim - 2)).
 * (The reference wrapper maps the three values through an inverted `!=` chain at
 * rotary_position_embedding_kernel.cc:99-108, which sends NONE to LINEAR and everything else to NONE; this library
 * takes the value at its name.)
 * head_dim and rotary_dim must be multiples of 8, head_dim <= 2048; the half-split layout needs rotary_dim to be a
 * multiple of 16. rotated_query / rotated_key may alias query / key (in-place rotation) in both layouts.
 */
enum {
    PPLHIP_ROPE_PAIRS_INTERLEAVED = 0,
    PPLHIP_ROPE_PAIRS_HALF_SPLIT = 1
};

enum {
    PPLHIP_ROPE_SCALING_NONE = 0,
    PPLHIP_ROPE_SCALING_LINEAR = 1,
    PPLHIP_ROPE_SCALING_DYNAMIC = 2
};

typedef struct pplhip_rope_args {
    const void* d_query;
    const void* d_key;
    const int64_t* d_start_pos; /* [batch] */
    const int64_t* d_seqstarts; /* [batch+1] */
    float theta;
    int32_t bypass_key;
    int32_t rotary_dim;
    int32_t pair_layout; /* PPLHIP_ROPE_PAIRS_* */
    int64_t batch;
    int64_t total_tokens; /* = seqstarts[batch] = dim 0 of query and key */
    int32_t num_heads;
    int32_t num_key_heads;
    int32_t head_dim;
    int32_t max_position_embeddings;
    int64_t max_seqlen;
    int32_t scaling_type;
    float scaling_factor;
    void* d_rotated_query;
    void* d_rotated_key;
} pplhip_rope_args;

pplhip_retcode pplhip_rope_forward(const pplhip_rope_args* args, void* stream);

/*
 * RotaryPositionEmbedding and the quantize-on-write of the same new tokens in ONE launch: what pplhip_rope_forward
 * followed by pplhip_kv_quantize_write (with `write->d_current_key` = `rope->d_rotated_key`) leaves behind, bit for
 * bit -- rotated_query, rotated_key, and the int8 bytes + fp16 scales of the rotated keys and of
 * `write->d_current_value` at the new tokens' slab positions. The reference runs the two steps as separate operators
 * (rotary_position_embedding_kernel.cc:110-132, then the cache write inside multi_head_cache_attention_kernel.cc:230);
 * here the 8 channels a lane rotates are one quantisation group, so the key rows are quantised from the registers
 * they are stored from and K and V are read once. `write->d_current_key` is not read. Both argument blocks must
 * describe the same tokens: same batch, token count, key heads, head_dim and the same seqstarts / start_pos pointers
 * (PPLHIP_RC_INVALID_VALUE otherwise). A MultiHeadCacheAttention call that follows may write the same tokens again
 * (its kernels quantise the new tokens themselves): the bytes are the same.
 */
pplhip_retcode pplhip_rope_kv_write_forward(const pplhip_rope_args* rope, const pplhip_kv_write_args* write, void* stream);

/*
 * opmx.dynamic_batching::PositionIndex (`dynamic_batching_position_index` as called from
 * src/ppl/nn/engines/llm_cuda/kernels/opmx/dynamic_batching/position_index_kernel.cc:60-67):
 * position_idx[t] = start_pos[b] + (t - seqstarts[b]) for every packed token t of sequence b; i64 [total_tokens].
 */
pplhip_retcode pplhip_position_index(const int64_t* d_start_pos, const int64_t* d_seqstarts, int64_t batch,
                                     int64_t total_tokens, int64_t max_seqlen, int64_t* d_position_idx, void* stream);

/*
 * On-device rebuild of the ragged-batch tables, replacing the host loops of
 * tools/benchmark_llama/generation_state.cc:60-125 (FirstStep) and :127-192 (NextStep) plus the eight per-step
 * uploads of tools/benchmark_llama/text_generator.cc:233-291.
 *
 * Slot state (device, one entry per slot, `num_slots` <= 1024):
 *   slot_kvlen[i]   tokens cached for the slot's sequence BEFORE this step (0 for a fresh prompt)
 *   slot_newlen[i]  new tokens this step: 0 = slot idle/retired, 1 with kvlen > 0 = decode step, otherwise prefill
 *   slot_cachestart[i] first slab token of the slot's region
 * Outputs (device): active sequences are compacted stably, decode sequences first, then prefill sequences;
 *   seqstarts/kvstarts [num_slots+1] (entries past the batch repeat the total), cachestarts/start_pos/batch_slots
 *   [num_slots] (batch_slots[b] = slot index of packed sequence b, -1 past the batch), and
 *   header[0..5] = {batch, decoding_batches, max_seqlen, max_kvlen, total_new_tokens, total_kv_tokens}.
 */
typedef struct pplhip_pack_args {
    const int64_t* d_slot_kvlen;
    const int64_t* d_slot_newlen;
    const int64_t* d_slot_cachestart;
    int32_t num_slots;
    int32_t advance_slots; /* 0: the slot state is only read. 1: once the tables are built the same launch also does what
                              pplhip_advance_slots does, slot_kvlen[i] += slot_newlen[i] for every active slot (the
                              attention call that follows reads the packed tables, not the slot state, so the state can
                              move on right away and a step needs one launch less); d_slot_kvlen is then written */
    int64_t* d_seqstarts;
    int64_t* d_kvstarts;
    int64_t* d_cachestarts;
    int64_t* d_start_pos;
    int64_t* d_batch_slots;
    int64_t* d_header; /* 6 x i64; may be pinned host memory mapped on the device */
} pplhip_pack_args;

pplhip_retcode pplhip_pack_tables(const pplhip_pack_args* args, void* stream);

/* After a step: slot_kvlen += slot_newlen for every active slot (so the next pack sees the grown sequences). A launch
 * of its own; pplhip_pack_args.advance_slots does the same inside the pack launch. */
pplhip_retcode pplhip_advance_slots(int64_t* d_slot_kvlen, const int64_t* d_slot_newlen, int32_t num_slots,
                                    void* stream);

/*
 * Consistency check of the tables of one MultiHeadCacheAttention call, for debugging a scheduler (the attention
 * kernels trust the tables: one bad entry is an out-of-range slab access, i.e. a GPU fault rather than a wrong
 * number). The reference has no device-side counterpart; its host harness builds the tables it trusts itself
 * (tools/benchmark_llama/generation_state.cc:60-192), and its debug builds synchronise after every op
 * (src/ppl/nn/engines/llm_cuda/kernel.cc:169-177) so that a fault names the op. One small launch reads `args`'
 * seqstarts / kvstarts / cachestarts / start_pos (never the slab, never the activations) and writes to `d_flag`
 * (device, 2 x int32): d_flag[0] = one of PPLHIP_TABLES_* (0 = consistent), d_flag[1] = the first offending sequence
 * (-1 if none). Checked per sequence b: seqlen >= 1; kvlen >= seqlen; start_pos >= 0 and kvlen == start_pos + seqlen;
 * a decode sequence (b < decoding_batches) has exactly one new token at packed index b; seqlen <= max_seqlen and
 * kvlen <= max_kvlen; every slab token the sequence owns lies in [0, max_slab_tokens) -- cachestarts[b] + kvlen in the
 * contiguous mode, every used page of its page-table row (and enough entries in that row) in the paged mode; and
 * seqstarts[0] == kvstarts[0] == 0, seqstarts[batch] == total_new_tokens. `max_slab_tokens` is the slab's token extent
 * (MaxT of the cache tensor). Only the table pointers, sizes, cache_mode / page_size / cachestart_stride_b of `args` are
 * read.
 */
enum {
    PPLHIP_TABLES_OK = 0,
    PPLHIP_TABLES_BAD_SEQSTARTS = 1,        /* not starting at 0, not increasing, or total != total_new_tokens */
    PPLHIP_TABLES_BAD_KVSTARTS = 2,         /* not starting at 0, or a kv length below the sequence's new tokens */
    PPLHIP_TABLES_KVLEN_MISMATCH = 3,       /* kvlen != start_pos + seqlen, or start_pos < 0 */
    PPLHIP_TABLES_BAD_DECODE_ORDER = 4,     /* a decode sequence without exactly one new token at packed index b */
    PPLHIP_TABLES_MAX_EXCEEDED = 5,         /* seqlen > max_seqlen or kvlen > max_kvlen */
    PPLHIP_TABLES_SLAB_RANGE = 6,           /* a slab token outside [0, max_slab_tokens) */
    PPLHIP_TABLES_PAGE_TABLE_TOO_SHORT = 7  /* paged mode: the sequence needs more pages than its table row holds */
};
pplhip_retcode pplhip_check_tables(const pplhip_mhca_args* args, int64_t max_slab_tokens, int32_t* d_flag, void* stream);
/* The same rules, same codes and same choice of the reported finding (the lowest sequence, then the lowest code)
 * for a scheduler that builds its tables in host memory, as the reference's harness does before it uploads them
 * (tools/benchmark_llama/text_generator.cc:233-291): the four table pointers of `args` are HOST pointers here, `flag`
 * is 2 x int32 in host memory, and no device is touched. */
pplhip_retcode pplhip_check_tables_host(const pplhip_mhca_args* args, int64_t max_slab_tokens, int32_t* flag);

#ifdef __cplusplus
}
#endif

#endif /* PPL_LLM_KERNEL_HIP_H_ */
