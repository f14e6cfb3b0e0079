/*
 * C ABI of the MI355X (gfx950) NAtS sparse-attention inference path.
 *
 * Every entry point takes raw device pointers (as produced by hipMalloc or tensor.data_ptr()), plain
 * integer sizes / strides counted in ELEMENTS, and a HIP stream handle passed as void* (NULL = the
 * default stream).  All work is enqueued on that stream; nothing synchronises with the host, nothing
 * allocates or frees device memory and no pointer is kept after the call returns.
 *
 * Return value: 0 on success, a negative nats_status otherwise; nats_last_error() then returns a
 * thread-local, human readable description.
 *
 * Citations name the reference interface each entry point stands in for (paths relative to the
 * reference checkout, src/nats/...).
 */
#ifndef NATS_HIP_H
#define NATS_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define NATS_ABI_VERSION 8

typedef enum {
  NATS_OK = 0,
  NATS_ERR_NULL_POINTER = -1,
  NATS_ERR_BAD_SHAPE = -2,
  NATS_ERR_BAD_DTYPE = -3,
  NATS_ERR_UNSUPPORTED = -4,
  NATS_ERR_WORKSPACE = -5,
  NATS_ERR_LAUNCH = -6
} nats_status;

typedef enum { NATS_DTYPE_BF16 = 0, NATS_DTYPE_F32 = 1 } nats_dtype;

/* role codes, the option order of token_states_info (components/cache/nats_chunk_layer_cache.py:188-190) */
enum { NATS_ROLE_GLOBAL = 0, NATS_ROLE_LOCAL = 1, NATS_ROLE_SW = 2 };

int nats_abi_version(void);
const char* nats_last_error(void);

/* ------------------------------------------------------------------------------------------------
 * Role assignment.  Replaces BaseNAtSAttentionLayer._sample_for_token_info_values_inference
 * (models/transformer/attention/nats_attention.py:96-109) and the open-chunk rule of
 * models/transformer/attention/nats_chunk_attention.py:92-94.
 *   logits  [B, S, H_kv, 3] contiguous, dtype bf16 or f32
 *   roles   [B, H_kv, S] uint8 out (0 global, 1 local, 2 sliding window)
 *   one_hot [B, H_kv, S, 3] out, same dtype as logits, may be NULL
 * global_bias is added to option 0 in the logits' dtype (0.1 in the reference module, 0 in the HF
 * twins); the first maximal option wins; slot 0 / the last slot are forced global on request.
 */
int nats_roles_from_logits(const void* logits, int dtype, int64_t B, int64_t S, int64_t H_kv, float global_bias,
                           int force_first_global, int force_last_global, uint8_t* roles, void* one_hot,
                           void* stream);

/* ------------------------------------------------------------------------------------------------
 * Fused role step: chunk pooling of the hidden states, role projection, bias, argmax with forced globals and
 * the next-global scan in one call.  Replaces NAtSCache.update_nats_cached_x_across_chunk / _in_chunk
 * (components/cache/dyn_cache.py:117-171) with the pooling of chunk_utils.py:13-62, followed by proj_layer and
 * _sample_for_token_info_values_inference (models/transformer/attention/nats_chunk_attention.py:64-95,
 * nats_attention.py:96-109) and the index scan of components/masks/utils.py:85-87.
 *   x         [B, L, dim] hidden states of the new tokens, strides (stride_b, stride_l), last dimension contiguous
 *   carry_in  [B, dim] running statistic of the open chunk (sum of x / C, or max); required when pre_fill > 0
 *   weight    [H_kv * 3, dim] contiguous, the role projection (bias free)
 *   pre_fill  tokens already in the open chunk (chunk_fill_size before this call), 0 <= pre_fill < C
 *   merge_max 0 = mean pooling, 1 = max pooling
 * With total = pre_fill + L:  total < C  -> no chunk completes, only carry_out = statistic so far is written;
 * otherwise S = ceil(total / C) role slots are produced, the open last one (total % C != 0) forced global and
 * its statistic written to carry_out.
 *   roles     [B, H_kv, S] uint8 out; roles_head_stride = 0: contiguous, else the entries between the roles of two
 *             consecutive (b, kv head) streams (>= S): the roles land in a slice of a wider [B, H_kv, U] buffer, as
 *             the per-token cache keeps the roles of its pending tokens (nats_layer_cache.py:196-200); no index scan then
 *   one_hot   [B, H_kv, S, 3] out, dtype of x, may be NULL
 *   logits    [B, S, H_kv, 3] out (before the bias), dtype of x, may be NULL
 *   end_idx / vis_lim  [B, H_kv, S] as nats_role_scan, may be NULL
 * The pooled statistic and the logits are rounded to the dtype of x where the torch ops round them; logits
 * are accumulated in fp32 in an order of their own, so they agree with a library GEMM to rounding only.
 * C must be a power of two here (NATS_ERR_UNSUPPORTED otherwise): the chunk mean is sum * (1 / C), which is torch's
 * mean bit for bit only then.  The other entry points take any chunk size that divides the window.
 */
int nats_role_step(const void* x, const void* carry_in, const void* weight, int dtype, int64_t B, int64_t L, int64_t dim,
                   int64_t H_kv, int64_t C, int64_t W, int64_t pre_fill, int merge_max, float global_bias,
                   int force_first_global, const int64_t* x_strides, uint8_t* roles, int64_t roles_head_stride,
                   void* one_hot, void* logits, void* carry_out, int64_t* end_idx, int32_t* vis_lim, void* stream);

/* next-global index and the per-slot visibility limit derived from it.
 * Replaces the first half of generate_hard_seq_masks (components/masks/utils.py:85-87).
 *   roles    [B, H_kv, S] uint8
 *   end_idx  [B, H_kv, S] int64 out, may be NULL: first global slot >= n, the last slot counting as global
 *   vis_lim  [B, H_kv, S] int32 out, may be NULL: the last query slot that still sees key slot n
 *            (global: INT32_MAX, local: end_idx[n], sliding window: n + W / C)
 */
int nats_role_scan(const uint8_t* roles, int64_t B, int64_t H_kv, int64_t S, int64_t W, int64_t C, int64_t* end_idx,
                   int32_t* vis_lim, void* stream);

/* ------------------------------------------------------------------------------------------------
 * debug / parity output: the token-level bool mask of a prefill from an empty cache, as
 * NAtSChunkLayerCache.generate_mask builds it (components/cache/nats_chunk_layer_cache.py:589-620),
 * evaluated with the same per-key limits the prefill kernels use.
 *   roles     [B, H_kv, S] uint8, S = ceil(L / C)
 *   mask      [B, H_kv, L, L] uint8 out (1 = attend)
 *   workspace nats_prefill_workspace_bytes(B, *, H_kv, L, *, C) bytes
 */
int nats_prefill_mask(const uint8_t* roles, int64_t B, int64_t H_kv, int64_t L, int64_t C, int64_t W, uint8_t* mask,
                      void* workspace, size_t workspace_bytes, void* stream);

/* debug / parity output: the block-sparse tile-skip map the prefill kernel walks.
 *   tiles  [B, H_kv, T, T] uint8 out, T = ceil(L / 64): 1 = the 64x64 tile (query tile, key tile) is loaded
 */
int nats_prefill_tile_map(const uint8_t* roles, int64_t B, int64_t H_kv, int64_t L, int64_t C, int64_t W,
                          uint8_t* tiles, void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------------------------------
 * role-masked chunked flash-attention prefill from an empty cache.
 * Replaces nats_prefill(...) with global_kv_size=None (models/transformer/triton/nats_flashattn_fwd.py:617-692)
 * and the generate_mask + SDPA branch of multi_head_attention
 * (models/transformer/attention/nats_chunk_attention.py:130-149).
 *   q [B, H_q, L, D], k / v [B, H_kv, L, D], o [B, H_q, L, D]; the last dimension is contiguous, the other
 *   three strides are given in elements (stride_b, stride_h, stride_l)
 *   roles [B, H_kv, S] uint8, S = ceil(L / C)
 *   workspace: nats_prefill_workspace_bytes(...) bytes of device memory (contents need not be kept).  It belongs to
 *   the call until its kernels have run: besides the per-key limits it holds the counter from which a large launch
 *   deals its lightest query groups and, for chunks shorter than 16 tokens, the lists of the rows that stay visible
 *   for more than a window (those rows are gathered row by row instead of walked in 16-row granules), so two calls
 *   that may overlap on the device need a workspace each.
 * D in {16, 32, 64, 128, 256} (the head dims of nats_flashattn_fwd.py:634); C > 0; W % C == 0;
 * H_q % H_kv == 0.
 * dtype bf16 with D 32, 64, 128 or 256 runs QK^T and PV on bf16 MFMA with fp32 softmax state (D 256: a kernel of its
 * own, four wavefronts with the whole register file; rows that are not 16-byte aligned go to the plain kernel);
 * dtype f32, and bf16 at D 16, run an fp32 FMA kernel.
 */
size_t nats_prefill_workspace_bytes(int64_t B, int64_t H_q, int64_t H_kv, int64_t L, int64_t D, int64_t C);

/* Extra workspace bytes (behind the ones above; already included in nats_prefill_workspace_bytes) for one optional
 * form of the bf16 launch.  Few query tiles over many key rows (a short segment over a long cache): several
 * workgroups share the key tiles of one query tile and a second kernel merges their partial results, so that the
 * launch still fills the device (NATS_PREFILL_SPLIT=0 in the environment switches this off).
 * A call whose workspace is smaller runs one workgroup per query tile; results are the same to rounding.  0 for
 * shapes that do not use it.  n_queries: new tokens of the call, n_rows: key rows (L for a prefill from an empty cache,
 * n_ctx_data + x_len over a filled one).
 */
size_t nats_prefill_sched_workspace_bytes(int64_t B, int64_t H_q, int64_t H_kv, int64_t n_queries, int64_t n_rows);

int nats_prefill_fwd(const void* q, const void* k, const void* v, const uint8_t* roles, void* o, int64_t B,
                     int64_t H_q, int64_t H_kv, int64_t L, int64_t D, int64_t C, int64_t W, const int64_t* q_strides,
                     const int64_t* k_strides, const int64_t* v_strides, const int64_t* o_strides, float sm_scale,
                     int dtype, void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------------------------------
 * A multi-token segment over a cache that earlier segments have filled and evicted.
 * Replaces NAtSChunkLayerCache._generate_mask for x_len > 1 over a non-empty cache
 * (components/cache/nats_chunk_layer_cache.py:462-511, with _fit_sliding_queue_masks :658-713) followed by
 * SDPA over cache_k / cache_v[:, :, :n_ctx_data + x_len]
 * (models/transformer/attention/nats_chunk_attention.py:130-149).  Call it after the cache update that
 * appended the segment's keys / values and before the eviction of that segment.
 *
 * nats_past_state holds the cache scalars as they stand before the segment is evicted:
 */
typedef struct {
  int64_t n_ctx_data; /* live rows before the segment was appended (the segment sits at rows
                         [n_ctx_data, n_ctx_data + x_len)) */
  int64_t old_fill;   /* tokens of the open chunk cached before the segment: chunk_fill_size - x_len */
  int64_t gmin;       /* _n_global_min */
  int64_t tail;       /* sliding_queue_tail */
  int64_t seen;       /* _seen_tokens (not yet counting the segment) */
  int64_t fill_last;  /* chunk_fill_size_last */
  int64_t update_chunk; /* 0: the chunked cache (NAtSChunkLayerCache).  U > 0: the per-token cache (NAtSLayerCache,
                           components/cache/nats_layer_cache.py:469-517, 603-649) with update chunk size U; C must be 1,
                           old_fill < U counts the pending tokens and `tail` is the ring slot written last */
} nats_past_state;

/*   q [B, H_q, x_len, D], o like q; cache_k / cache_v [B, H_kv, >= n_ctx_data + x_len, D]
 *   valid [B, H_kv, >= n_ctx_data] uint8 (valid_tokens), strides (stride_b, stride_h)
 *   size_global / size_local [B, H_kv] int64 contiguous
 *   roles [B, H_kv, S] uint8, S = ceil((old_fill + x_len) / C): one slot per chunk of the open-chunk region
 *   workspace: nats_prefill_past_workspace_bytes(B, H_kv, n_ctx_data + x_len, S) bytes, optionally followed by
 *              nats_prefill_sched_workspace_bytes(B, H_q, H_kv, x_len, n_ctx_data + x_len) more
 * Query i is token old_fill + i of the region that starts at row n_ctx_data - old_fill.
 */
size_t nats_prefill_past_workspace_bytes(int64_t B, int64_t H_kv, int64_t n_rows, int64_t S);

int nats_prefill_past_fwd(const void* q, const void* cache_k, const void* cache_v, const uint8_t* valid,
                          const int64_t* size_global, const int64_t* size_local, const uint8_t* roles, void* o,
                          int64_t B, int64_t H_q, int64_t H_kv, int64_t x_len, int64_t D, int64_t C, int64_t W,
                          const nats_past_state* state, const int64_t* q_strides, const int64_t* k_strides,
                          const int64_t* v_strides, const int64_t* valid_strides, const int64_t* o_strides,
                          float sm_scale, int dtype, void* workspace, size_t workspace_bytes, void* stream);

/* debug / parity output: the mask of that segment, [B, H_kv, x_len, n_ctx_data + x_len] uint8 */
int nats_prefill_past_mask(const uint8_t* valid, const int64_t* size_global, const int64_t* size_local,
                           const uint8_t* roles, int64_t B, int64_t H_kv, int64_t x_len, int64_t C, int64_t W,
                           const nats_past_state* state, const int64_t* valid_strides, uint8_t* mask, void* workspace,
                           size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------------------------------
 * one-token decode attention over the evicted, ragged cache.
 * Replaces _generate_mask_one_step + SDPA (components/cache/nats_chunk_layer_cache.py:622-632,
 * models/transformer/attention/nats_chunk_attention.py:131-142) and the flattened varlen call of
 * models/transformer/hf/llama.py:274-295.
 *   q [B, H_q, D] contiguous (one query token), o [B, H_q, D] contiguous
 *   cache_k / cache_v [B, H_kv, >= n_rows, D], last dimension contiguous, strides (stride_b, stride_h, stride_row)
 *   valid [B, H_kv, >= n_rows] uint8 (the cache's valid_tokens), strides (stride_b, stride_h), rows contiguous
 *   n_rows = n_ctx_data + 1: rows [0, n_rows) with valid != 0 take part; rows with valid == 0 are never loaded
 *   row_end [B, H_kv] int64, optional (NULL = no hint): per head, rows [row_end, tail_start) are known to
 *           hold nothing valid (the cache's size_global_kv + size_local_kv and the start of the open chunk,
 *           components/cache/nats_chunk_layer_cache.py:644-656) and are skipped without reading valid
 *   workspace: nats_decode_workspace_bytes(...) bytes
 * D in {16, 32, 64, 128, 256}; H_q % H_kv == 0 (any group size); dtype bf16 (MFMA for D 32, 64, 128 and 256) or f32
 * (fp32 FMA kernel, which also takes bf16 at D 16 and ignores the hint).
 * bf16: a batch of more than 1024 (b, kv head) streams is taken in groups of whole sequences, launched one after
 * the other on `stream`.
 */
size_t nats_decode_workspace_bytes(int64_t B, int64_t H_q, int64_t H_kv, int64_t D, int64_t n_rows);

int nats_decode_fwd(const void* q, const void* cache_k, const void* cache_v, const uint8_t* valid,
                    const int64_t* row_end, int64_t tail_start, void* o, int64_t B, int64_t H_q, int64_t H_kv, int64_t D,
                    int64_t n_rows, const int64_t* kv_strides, const int64_t* valid_strides, float sm_scale, int dtype,
                    void* workspace, size_t workspace_bytes, void* stream);

/* nats_decode_fwd for callers that cannot allocate device memory or bring a workspace: code under HIP graph
 * capture, tight serving loops, harnesses that forbid the allocator.  It has no counterpart in the reference.
 * Same arguments, same kernels and bit-identical results; the partial results of the split kernels live in a
 * static device array of NATS_DECODE_STATIC_SCRATCH_BYTES that every GPU the library runs on holds until the
 * process ends.  The call allocates and frees nothing.  A shape whose nats_decode_workspace_bytes(...) exceeds
 * that size is rejected with NATS_ERR_WORKSPACE (take nats_decode_fwd then).  All calls on one GPU share the
 * array: calls that overlap in time on one GPU (two streams, two threads) race on it; order them on one stream.
 */
#define NATS_DECODE_STATIC_SCRATCH_BYTES (8u << 20)

size_t nats_decode_static_scratch_bytes(void);

int nats_decode_fwd_static(const void* q, const void* cache_k, const void* cache_v, const uint8_t* valid,
                           const int64_t* row_end, int64_t tail_start, void* o, int64_t B, int64_t H_q, int64_t H_kv,
                           int64_t D, int64_t n_rows, const int64_t* kv_strides, const int64_t* valid_strides,
                           float sm_scale, int dtype, void* stream);

/* ------------------------------------------------------------------------------------------------
 * KV eviction + compaction: NAtSChunkLayerCache._post_update from its ring insert to its
 * valid_tokens rewrite (components/cache/nats_chunk_layer_cache.py:270-371, 391-437, 634-656, 715-868)
 * with merge_local_to_global_caches (components/cache/cache_update.py:25-76).
 *
 * Host-side facts travel in nats_evict_params, device-side results come back in nats_evict_result
 * (device memory, 64 bytes, written by the call; copy it to the host when the numbers are needed).
 */
typedef struct {
  int64_t B, H_kv, D;
  int64_t C, W;
  int64_t S;           /* role slots handed to the last update (one per chunk touched, open chunk included) */
  int64_t x_len;       /* tokens appended by the last update */
  int64_t fill;        /* chunk_fill_size after that update (old open-chunk tokens + x_len), >= C */
  int64_t n_ctx_data;  /* before this call */
  int64_t gmin;        /* _n_global_min before this call */
  int64_t tail;        /* sliding_queue_tail before this call */
  int64_t first;       /* 1 if these are the first tokens the layer has seen (_seen_tokens == x_len) */
  int64_t n_alloc;     /* rows allocated in cache_k / cache_v / valid (in place) or in the new cache (out of place) */
  int64_t seq;         /* any number the caller chooses; it comes back in nats_evict_result.seq and, its low 32 bits, in
                          the nats_evict_brief a host may poll (which gives every call a new one) */
  int64_t update_chunk; /* 0: the chunked cache.  U > 0: the per-token cache NAtSLayerCache._post_update
                           (components/cache/nats_layer_cache.py:292-418, 424-458, 556-574, 651-770) once U tokens
                           are pending: C = 1, S = fill = the pending block with one role per token, n_ctx_data = the
                           first row of that block, tail = the ring slot written last, first = 1 if the block holds
                           every token seen so far.  Ring rows are copied whatever the role (valid only if
                           sliding-window), rows at and beyond the new n_ctx_data keep their contents, and a block of
                           sliding-window tokens only leaves n_ctx_data where it is.  U = 1 (nothing is deferred, W >= 2):
                           a one-token step is the class's one-step branch (:328-367): the token's row goes to row
                           size_global (a global token) or size_global + size_local (any other) of every head and to ring
                           slot tail + 2 (slot 1 for the first token ever), unless it is sliding-window on every head. */
} nats_evict_params;

typedef struct {
  int64_t n_ctx_data;  /* after the call */
  int64_t gmin;        /* min over (b, h) of size_global after the call */
  int64_t all_sw;      /* 1: every slot was sliding-window, only n_ctx_data and the ring changed */
  int64_t all_local;   /* 1: every slot was local, nothing was moved */
  int64_t max_keep;    /* largest number of kept chunks over (b, h) */
  int64_t max_end;     /* largest (kept + destination base) over (b, h), in chunks */
  int64_t moved_rows;  /* rows copied by the compaction (both tensors counted once), for bandwidth accounting */
  int64_t seq;         /* params->seq of the call that wrote this result */
} nats_evict_result;

/* What a host that does not want to synchronise with the stream polls for: 16 bytes that the plan step writes with
 * one store, meant for pinned host memory.  Whoever reads its own params->seq (its low 32 bits) in `seq` has the rest. */
typedef struct {
  int32_t seq;         /* low 32 bits of params->seq of the call that wrote this */
  int32_t flags;       /* bit 0: all_sw, bit 1: all_local */
  int32_t n_ctx_data;  /* after the call */
  int32_t gmin;        /* after the call */
} nats_evict_brief;

size_t nats_evict_workspace_bytes(int64_t B, int64_t H_kv, int64_t S);

/* Step 1, always: roles -> per-head plan in `workspace`, new sizes and the scalars in `result`.
 *   size_global / size_local [B, H_kv] int64, read here, rewritten by the apply step
 *   workspace: nats_evict_workspace_bytes(...) bytes.  Its first 256 bytes must be zero before the first call that
 *              uses it and every call leaves them zero (a counter lives there); the rest need not be kept between
 *              calls.  Calls that share a workspace must not overlap (calls on one stream do not).
 *   With params->first the sizes are not read: a cache that has seen nothing holds the empty ring (size_global = W,
 *   size_local = 0) whatever the tensors contain; the apply step writes them.
 *   result_mirror: NULL, or 16 bytes (16-byte aligned) that receive the short form of the result in one store, meant
 *              for pinned host memory: a host that sees its own params->seq there has n_ctx_data, gmin and the two
 *              flags without synchronising with the stream
 */
int nats_evict_plan(const uint8_t* roles, const int64_t* size_global, const int64_t* size_local,
                    const nats_evict_params* params, void* workspace, size_t workspace_bytes, nats_evict_result* result,
                    nats_evict_brief* result_mirror, void* stream);

/* Step 2a, in place: ring insert, ordered chunk moves (all sources of a batch are read before any of its
 * destinations is written, which equals the reference's gather-clone-then-scatter), zero fill of rows
 * >= n_ctx_data, valid_tokens rewrite, size update.
 *   cache_k / cache_v [B, H_kv, n_alloc, D] same dtype (element size elem_bytes in {2, 4}), strides (b, h, row)
 *   valid [B, H_kv, n_alloc] uint8 contiguous rows, strides (b, h)
 *   pos   [B, H_kv, n_alloc] int32 optional shadow carrying the stream position of every row (-1 = none);
 *         moved exactly like the rows, it is the surviving-token index map.  May be NULL.
 */
int nats_evict_apply_inplace(void* cache_k, void* cache_v, uint8_t* valid, int32_t* pos, const uint8_t* roles,
                             int64_t* size_global, int64_t* size_local, const nats_evict_params* params,
                             const int64_t* kv_strides, const int64_t* valid_strides, int elem_bytes,
                             const void* workspace, const nats_evict_result* result, void* stream);

/* Step 2b, first prefill, out of place: gathers straight from the raw K / V of the prefill
 * ([B, H_kv, x_len, D], strides (b, h, row)) into a fresh cache of n_alloc rows, producing the same
 * bytes the in-place sequence would leave in rows [0, n_alloc) of [W zeros | K | pad].
 * Requires params->first == 1 and the cache to have been empty; n_alloc = ceil(result.n_ctx_data / C) * C
 * reproduces the reference's truncation (components/cache/nats_chunk_layer_cache.py:373-380).  A caller that does
 * not know result.n_ctx_data yet may pass a larger n_alloc (a cache allocated on an estimate): rows from
 * ceil(result.n_ctx_data / C) * C on are spare capacity and are not written at all, in none of the tensors; the
 * caller zeroes them (valid 0, pos -1) when it extends the cache into them.  With a smaller n_alloc the call has
 * to be made again into a large enough cache.
 */
int nats_evict_apply_first(const void* src_k, const void* src_v, void* cache_k, void* cache_v, uint8_t* valid,
                           int32_t* pos, const uint8_t* roles, int64_t* size_global, int64_t* size_local,
                           const nats_evict_params* params, const int64_t* src_strides, const int64_t* kv_strides,
                           const int64_t* valid_strides, int elem_bytes, const void* workspace,
                           const nats_evict_result* result, void* stream);

/* The row write of the cache update for a cache that already holds rows (NAtSChunkLayerCache.update,
 * components/cache/nats_chunk_layer_cache.py:243-256; NAtSLayerCache.update, nats_layer_cache.py:279-284) in one launch:
 *   cache_k / cache_v[b, h, row0 + l] = k / v[b, h, l],  valid[b, h, row0 + l] = 1,  pos[b, h, row0 + l] = pos0 + l
 *   k / v [B, H_kv, x_len, D]: strides (b, h, l);  cache_k / cache_v [B, H_kv, n_alloc, D]: strides (b, h, row)
 *   valid / pos [B, H_kv, n_alloc]: strides (b, h);  pos may be NULL;  rows and strides multiples of 16 bytes
 */
int nats_cache_append(const void* k, const void* v, void* cache_k, void* cache_v, uint8_t* valid, int32_t* pos, int64_t B,
                      int64_t H_kv, int64_t x_len, int64_t D, int64_t row0, int64_t n_alloc, int64_t pos0,
                      const int64_t* k_strides, const int64_t* v_strides, const int64_t* cache_strides,
                      const int64_t* valid_strides, int elem_bytes, void* stream);

/* nats_cache_append and, in the same launch, nats_evict_plan for the eviction that follows this update (the roles of
 * the chunks the update completes are known when the rows arrive, NAtSChunkLayerCache.update / _post_update,
 * components/cache/nats_chunk_layer_cache.py:171-256, 270-371): a stream that appends a chunk and evicts, step after
 * step, then costs two launches per step, this one and nats_evict_apply_inplace.  `params` describe the coming
 * post_update as they would for nats_evict_plan (n_alloc, n_ctx_data, gmin, tail as they stand before it; x_len = the
 * rows appended here).  For params->S <= 32 and B * H_kv <= 4096; otherwise NATS_ERR_UNSUPPORTED (call the two
 * entry points).
 */
int nats_cache_append_plan(const void* k, const void* v, void* cache_k, void* cache_v, uint8_t* valid, int32_t* pos,
                           int64_t B, int64_t H_kv, int64_t x_len, int64_t D, int64_t row0, int64_t n_alloc, int64_t pos0,
                           const int64_t* k_strides, const int64_t* v_strides, const int64_t* cache_strides,
                           const int64_t* valid_strides, int elem_bytes, const uint8_t* roles, const int64_t* size_global,
                           const int64_t* size_local, const nats_evict_params* params, void* workspace,
                           size_t workspace_bytes, nats_evict_result* result, nats_evict_brief* result_mirror, void* stream);

/* ------------------------------------------------------------------------------------------------
 * Decode-step glue of the HF-shaped caller (models/transformer/hf/llama_nats_chunk.py:171-292 inside a Llama
 * decoder layer): the elementwise work around the attention, fused so that a layer costs a dozen launches.
 * Each entry point keeps the rounding points of the torch ops it replaces.
 */

/* x += delta (optional); out = RMSNorm(x) * weight, normalised in fp32, cast to the dtype, then multiplied
 * (models/transformer/components.py:14-26, the HF LlamaRMSNorm form).  Optionally also the running chunk
 * statistic of the role step for an open chunk (NAtSCache.merge_new_x_values_in_chunk,
 * components/cache/dyn_cache.py:98-124, called from hf/llama_nats_chunk.py:198) from the normalised row:
 *   carry_mode 0 none; 1 carry = out / chunk_size; 2 carry += out / chunk_size; 3 carry = out; 4 carry = max(carry, out)
 *   x [rows, dim] in / out, delta [rows, dim] or NULL, weight [dim], out [rows, dim], carry [rows, dim] or NULL;
 *   all contiguous, dim <= 8192
 */
int nats_add_rms_norm(void* x, const void* delta, const void* weight, void* out, void* carry, int64_t rows,
                      int64_t dim, float eps, int carry_mode, int64_t chunk_size, int dtype, void* stream);

/* out[r, c] = silu(gate_up[r, c]) * gate_up[r, inter + c]: act_fn(gate_proj(x)) * up_proj(x) of the Llama MLP
 * with the two projections stored as one matrix.  gate_up [rows, 2 * inter], out [rows, inter], contiguous.
 */
int nats_silu_mul(const void* gate_up, void* out, int64_t rows, int64_t inter, int dtype, void* stream);

/* y[r, n] = sum_k x[r, k] * w[n, k]: the nn.Linear projections (no bias) of a one-token step
 * (hf/llama_nats_chunk.py:185-187 q / k / v, :290 o_proj, the gate / up / down projections of the HF Llama MLP
 * the reference keeps, lm_head) for 1..4 rows of x.  fp32 accumulation, one rounding to the dtype.
 *   w [n_out, k] (gate != 0: [2 * n_out, k], gate rows first, then up rows), x [x_rows, k], y [x_rows, n_out];
 *   strides in elements, k contiguous; k and the strides of w and x multiples of 16 bytes, w and x 16-byte aligned
 *   gate != 0: y[r, n] = silu(x[r] . w[n]) * (x[r] . w[n_out + n]) with the roundings of the separate ops
 *   (nats_silu_mul after one projection over the stacked matrix)
 */
int nats_matvec(const void* w, const void* x, void* y, int64_t x_rows, int64_t n_out, int64_t k, int64_t w_stride,
                int64_t x_stride, int64_t y_stride, int gate, int dtype, void* stream);

/* Rotary embedding of q and k of a multi-token segment (transformers' apply_rotary_pos_emb as called at
 * hf/llama_nats_chunk.py:227: q * cos + rotate_half(q) * sin, every product and the sum rounded to the dtype):
 *   q_out [B, H_q, x_len, D] and k_out [B, H_kv, x_len, D] contiguous
 *   q [B, H_q, x_len, D], k [B, H_kv, x_len, D]: strides (b, h, l), last dimension contiguous (the transposed views of
 *   a [B, x_len, heads, D] projection are taken as they are); cos / sin [B, x_len, D]: strides (b, l)
 *   D a multiple of 32 bytes, every row 16-byte aligned
 */
int nats_rope_qk(const void* q, const void* k, const void* cos, const void* sin, void* q_out, void* k_out, int64_t B,
                 int64_t H_q, int64_t H_kv, int64_t x_len, int64_t D, const int64_t* q_strides, const int64_t* k_strides,
                 const int64_t* cos_strides, int dtype, void* stream);

/* Rotary embedding of q and k (transformers' apply_rotary_pos_emb, hf/llama_nats_chunk.py:227) and the row
 * write of NAtSChunkLayerCache.update (components/cache/nats_chunk_layer_cache.py:243-256) in one launch:
 *   q_out[b, h, l]            = rope(q[b, h, l])            [B, H_q, x_len, D] contiguous
 *   cache_k[b, h, row0 + l]   = rope(k[b, h, l]),  cache_v[b, h, row0 + l] = v[b, h, l]
 *   valid[b, h, row0 + l] = 1, pos[b, h, row0 + l] = pos0 + l (pos may be NULL)
 *   clear_row >= 0: also valid[b, h, clear_row] = 0 for every (b, h), a row below row0: the ring slot that the
 *   per-token cache switches off after a step whose eviction is deferred (NAtSLayerCache._post_update,
 *   components/cache/nats_layer_cache.py:300-310), written with the next step's rows.  -1: none.
 *   q [B, H_q, x_len, D], k / v [B, H_kv, x_len, D]: strides (b, h, l), last dimension contiguous
 *   cos / sin [B, x_len, D]: strides (b, l);  cache_k / cache_v [B, H_kv, n_alloc, D]: strides (b, h, row)
 *   valid / pos [B, H_kv, n_alloc]: strides (b, h)
 */
int nats_rope_append(const void* q, const void* k, const void* v, const void* cos, const void* sin, void* q_out,
                     void* cache_k, void* cache_v, uint8_t* valid, int32_t* pos, int64_t B, int64_t H_q, int64_t H_kv,
                     int64_t x_len, int64_t D, int64_t row0, int64_t n_alloc, int64_t pos0, int64_t clear_row,
                     const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                     const int64_t* cos_strides, const int64_t* cache_strides, const int64_t* valid_strides, int dtype,
                     void* stream);

#ifdef __cplusplus
}
#endif
#endif /* NATS_HIP_H */
