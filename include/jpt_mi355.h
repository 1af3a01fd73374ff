/*
 * jpt_mi355.h - C ABI of libjpt_mi355.so: the decode-time KV-cache path of
 * jetstream-pytorch for AMD MI355X (gfx950).
 *
 * The reference has no foreign-function interface on this path: it is a
 * Python API (jetstream_pt/cache_manager.py, page_attention_manager.py,
 * attention_kernel.py).  Each entry point below names the reference function
 * whose work it does; the Python package jetstream_pt_amd binds them with
 * ctypes and keeps the reference's class and function signatures.
 *
 * Conventions
 *   - every function returns an int32 status: JPT_OK or a negative JPT_E_*;
 *     jpt_last_error() returns a thread-local message for the last failure;
 *   - device pointers are plain `void*` into HBM owned by the caller; nothing
 *     here allocates device memory; kernels write in place;
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream);
 *     calls only enqueue work, they never synchronise;
 *   - all tensors are contiguous, row-major, with the shapes stated;
 *   - dtype codes are JPT_BF16 / JPT_F32 / JPT_I8.
 */
#ifndef JPT_MI355_H_
#define JPT_MI355_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define JPT_OK 0
#define JPT_E_BADARG (-1)        /* -> ValueError  */
#define JPT_E_NOPAGES (-2)       /* -> queue.Empty (free list exhausted) */
#define JPT_E_PAGE_OVERFLOW (-3) /* -> IndexError  (max_pages_per_sequence) */
#define JPT_E_HIP (-4)           /* -> RuntimeError */

#define JPT_BF16 0
#define JPT_F32 1
#define JPT_I8 2

#define JPT_ROUND_TRUNC 0 /* Int8KVCacheGenerate.quantize, cache_manager.py:532-537 */
#define JPT_ROUND_RNE 1   /* quantize_tensor symmetric int8, quantize.py:58-75 */

int32_t jpt_version(void);
const char* jpt_last_error(void);

/* ------------------------------------------------------------------------
 * KV line scatter: dst[l, b, h, pos[b], :] = src[l, b, h, 0, :]
 *
 * Replaces KVCacheGenerate.update eager branches (cache_manager.py:250-293),
 * KVCacheGenerate.finalize / update_single_cache_line (:154-225) and
 * Int8KVCacheGenerate.finalize / update_single_cache_line (:422-503,
 * :584-657), which issue one scatter or one dynamic_update_slice per slot
 * (and per layer) per tensor.  One launch writes up to JPT_MAX_LINE_TENSORS
 * tensors (K, V and, for int8 caches, both scalers) for all layers.
 *
 * dst is (n_layers, batch, heads, seq, row_bytes) bytes, src is
 * (n_layers, batch, heads, 1, row_bytes).  `pos` is an int32 device array of
 * `pos_count` entries: batch (one position per slot) or 1 (ring buffer: one
 * shared position).  A position outside [0, seq) writes nothing.
 * ---------------------------------------------------------------------- */
#define JPT_MAX_LINE_TENSORS 4
typedef struct {
  void* dst;
  const void* src;
  int32_t heads;
  int32_t row_bytes;
} jpt_line_tensor;

int32_t jpt_kv_scatter_lines(const jpt_line_tensor* tensors, int32_t n_tensors,
                             const int32_t* pos, int32_t pos_count,
                             int32_t n_layers, int32_t batch, int32_t seq,
                             void* stream);

/* ------------------------------------------------------------------------
 * Fused per-token absmax int8 quantisation + append.
 *
 * Replaces Int8KVCacheGenerate.quantize + .update (cache_manager.py:532-582):
 * per token, absmax over (heads, dim) [or over dim when scale_heads == heads],
 * scale and codes computed op by op in `scale_dtype` with the rounding rule
 * `rounding`, codes written to out_* (the k_quant / kscale the reference
 * returns, or its lazy stash new_ks[layer]) and, when cache_* is not NULL,
 * scattered to cache[b, :, pos[b], :] and scale[b, :, pos[b]].
 *
 * new_k/new_v (batch, heads, 1, dim) in in_dtype (bf16 or f32);
 * cache_k/cache_v (batch, heads, seq, dim) int8; k_scale/v_scale
 * (batch, scale_heads, seq) scale_dtype; out_k/out_v (batch, heads, 1, dim)
 * int8; out_k_scale/out_v_scale (batch, scale_heads) scale_dtype.  out_* may
 * be NULL.  scale_dtype is in_dtype or JPT_F32.  An all-zero token yields
 * scale 0 and codes 0 under JPT_ROUND_TRUNC.
 * ---------------------------------------------------------------------- */
typedef struct {
  const void* new_k;
  const void* new_v;
  void* cache_k;
  void* cache_v;
  void* k_scale;
  void* v_scale;
  void* out_k;
  void* out_v;
  void* out_k_scale;
  void* out_v_scale;
  const int32_t* pos;
  int32_t pos_count;
  int32_t batch, heads, seq, dim;
  int32_t in_dtype, scale_dtype, scale_heads, rounding;
  /* NULL, or rotary factors (batch, dim / 2, 2) float32 = (cos, sin) per slot
   * and pair, i.e. view_as_real(freqs_cis) of the step: new_k is then taken
   * UNROTATED and apply_rotary_emb (layers.py:368-379) is applied to it first:
   * pairs (2i, 2i + 1), re = a*cos - b*sin, im = a*sin + b*cos in float32 with one
   * rounding per op, result rounded to in_dtype.  new_v is never rotated. */
  const float* rope;
} jpt_quant_append_args;

int32_t jpt_kv_append_quant_i8(const jpt_quant_append_args* args, void* stream);

/* apply_rotary_emb (layers.py:368-379) on one tensor: x and out (rows, heads,
 * dim) in dtype (bf16 or f32), out may equal x; freqs (rows, dim / 2, 2) float32.
 * The query side of the step (and the key side where no fused append takes it). */
int32_t jpt_rope(void* out, const void* x, const float* freqs, int32_t rows,
                 int32_t heads, int32_t dim, int32_t dtype, void* stream);

/* ------------------------------------------------------------------------
 * Paged KV cache.  Pages are (heads, total_pages, page_size, row_bytes).
 *
 * jpt_paged_insert   - PageAttentionManager.insert_prefill_cache
 *   (page_attention_manager.py:83-142): src (heads, seq_len, row_bytes) is
 *   split into pages; pages[h, page_ids[p], t, :] = src[h, p*ps + t, :], the
 *   tail of the last page is zero-filled.  Two tensors (K, V) per launch.
 * jpt_paged_append   - PageKVCacheGenerate.update (cache_manager.py:681-706):
 *   for column j of `indices` (3, n_active) = (page, j*ps + tok, slot):
 *   pages[h, page_j, tok_j, :] = src[slot_j, h, 0, :]; src is
 *   (batch, heads, 1, row_bytes).
 * jpt_paged_gather   - PageAttentionManager._compress_cache (:195-200):
 *   dst[h, t, :] = pages[h, page_row[t / ps], t % ps, :] for t < length;
 *   page_row holds max_pages ids, and length <= max_pages * ps is required.
 * `page_ids`, `indices`, `page_row` are int32 device arrays.
 * ---------------------------------------------------------------------- */
int32_t jpt_paged_insert(void* pages_k, void* pages_v, const void* src_k,
                         const void* src_v, const int32_t* page_ids,
                         int32_t n_pages, int32_t seq_len, int32_t heads,
                         int32_t total_pages, int32_t page_size,
                         int32_t row_bytes, void* stream);

int32_t jpt_paged_append(void* pages_k, void* pages_v, const void* src_k,
                         const void* src_v, const int32_t* indices,
                         int32_t n_active, int32_t batch, int32_t heads,
                         int32_t total_pages, int32_t page_size,
                         int32_t row_bytes, void* stream);

/* jpt_paged_append with the column count in device memory: `indices` is
 * (3, indices_stride), of which the first *n_active_dev columns are valid
 * (what jpt_dpam_decode_step leaves behind); no host copy of the count. */
int32_t jpt_paged_append_dev(void* pages_k, void* pages_v, const void* src_k,
                             const void* src_v, const int32_t* indices,
                             int32_t indices_stride, const int32_t* n_active_dev,
                             int32_t batch, int32_t heads, int32_t total_pages,
                             int32_t page_size, int32_t row_bytes, void* stream);

int32_t jpt_paged_gather(void* dst, const void* pages, const int32_t* page_row,
                         int32_t max_pages, int32_t length, int32_t heads,
                         int32_t total_pages, int32_t page_size,
                         int32_t row_bytes, void* stream);

/* int8 pages (no reference counterpart: the reference's paged cache is
 * bf16/f32 only, cache_manager.py:717-724).  Same row scatter as
 * jpt_paged_append with the quantiser of jpt_kv_append_quant_i8 in front:
 * codes to pages (heads, total_pages, page_size, dim) int8, scales to
 * (scale_heads, total_pages, page_size) scale_dtype. */
typedef struct {
  const void* new_k;
  const void* new_v;
  void* pages_k;
  void* pages_v;
  void* k_scale_pages;
  void* v_scale_pages;
  const int32_t* indices; /* (3, n_active) */
  int32_t n_active;
  int32_t batch, heads, total_pages, page_size, dim;
  int32_t in_dtype, scale_dtype, scale_heads, rounding;
  /* NULL, or the column count in device memory: then n_active is ignored and
   * `indices` is (3, indices_stride) with the first *n_active_dev columns valid */
  const int32_t* n_active_dev;
  int32_t indices_stride;
  const float* rope; /* as in jpt_quant_append_args, indexed by slot */
} jpt_paged_quant_append_args;

int32_t jpt_paged_append_quant_i8(const jpt_paged_quant_append_args* args,
                                  void* stream);

/* ------------------------------------------------------------------------
 * Prefill -> decode insert of one prompt into one slot, one layer.
 *
 * Replaces the cache part of Engine._insert_no_wrap (engine.py:371-488: a
 * dynamic_update_slice of the prompt's K/V at position `start`, after
 * quantize_tensor over (heads, dim) per token when the cache is int8) and of
 * Engine._insert_wrap (:491-581: rows scattered to (start + t) mod seq).  With
 * page_ids set it is the int8 counterpart of jpt_paged_insert for int8 pages
 * (no reference counterpart): token t goes to page_ids[t / page_size], row
 * t % page_size, and the rows of the last page past `tokens` are zero-filled.
 *
 * src_k/src_v (heads, tokens, dim) in in_dtype.  Dense: dst (batch, heads,
 * seq, dim), scales (batch, scale_heads, seq).  Paged: dst (heads,
 * total_pages, page_size, dim), scales (scale_heads, total_pages, page_size).
 * dst_dtype == in_dtype copies; dst_dtype == JPT_I8 quantises with `rounding`
 * (the reference inserts with JPT_ROUND_RNE, quantize.py:58-75), scales and
 * intermediate results in scale_dtype as in jpt_kv_append_quant_i8.
 * ---------------------------------------------------------------------- */
typedef struct {
  const void* src_k;
  const void* src_v;
  void* dst_k;
  void* dst_v;
  void* k_scale;
  void* v_scale;
  const int32_t* page_ids; /* device array of n_pages ids, or NULL (dense) */
  int32_t n_pages;
  int32_t tokens, heads, dim;
  int32_t slot, batch, seq, start; /* dense */
  int32_t total_pages, page_size;  /* paged */
  int32_t in_dtype, dst_dtype, scale_dtype, scale_heads, rounding;
  /* Several layers in one launch: layer l reads src + l * src_layer_stride and
   * writes dst + l * dst_layer_stride, scales + l * scale_layer_stride (strides
   * in elements; stacked tensors).  n_layers 0 or 1 = one layer. */
  int32_t n_layers;
  int64_t src_layer_stride, dst_layer_stride, scale_layer_stride;
  /* Elements between the heads of src; 0 = tokens * dim (contiguous).  Larger
   * when src is the first `tokens` rows of a longer (heads, T, dim) buffer. */
  int64_t src_head_stride;
} jpt_prefill_insert_args;

int32_t jpt_prefill_insert(const jpt_prefill_insert_args* args, void* stream);

/* The same insert for layers that are tensors of their own (the reference's
 * unstacked DecodeState: a list of per-layer caches, engine.py:371-488 loops
 * over them inside one jitted program): one launch for up to 64 layers, the
 * pointers travelling in the kernel arguments.  `args` gives everything but
 * the six tensor pointers and the layer strides, which are ignored; `layers`
 * is a HOST array of n_layers entries (k_scale/v_scale NULL for a copy). */
typedef struct {
  const void* src_k;
  const void* src_v;
  void* dst_k;
  void* dst_v;
  void* k_scale;
  void* v_scale;
} jpt_insert_layer;

int32_t jpt_prefill_insert_layers(const jpt_prefill_insert_args* args,
                                  const jpt_insert_layer* layers,
                                  int32_t n_layers, void* stream);

/* Several prompts into the pages of one pool in one launch (the engine's
 * insert, engine.py:583-626, for every request whose prefill has finished).
 * `args` gives the destination (dst_k/dst_v/k_scale/v_scale, stacked layers by
 * n_layers and the dst/scale layer strides), geometry, dtypes and rounding; its
 * source, page_ids, tokens and n_pages fields are ignored.  `prompts` is a HOST
 * array: per prompt the source (heads, tokens, dim) tensors, their strides in
 * elements (src_head_stride 0 = tokens * dim), the DEVICE array of its n_pages
 * page ids and its token count.  Equivalent to one jpt_prefill_insert a prompt
 * (and done that way for shapes the one-launch kernel does not take: it
 * needs bf16 prompts, int8 pages, heads * dim == 1024). */
typedef struct {
  const void* src_k;
  const void* src_v;
  const int32_t* page_ids;
  int64_t src_head_stride, src_layer_stride;
  int32_t tokens, n_pages;
} jpt_insert_prompt;

int32_t jpt_prefill_insert_prompts(const jpt_prefill_insert_args* args,
                                   const jpt_insert_prompt* prompts,
                                   int32_t n_prompts, void* stream);

/* ------------------------------------------------------------------------
 * Decode attention.
 *
 * One argument block serves the three reference entry points:
 *   jpt_attn_ragged - ragged_mha / ragged_mqa_reference
 *     (attention_kernel.py:255-580): keys (batch, kv_heads, seq, dim),
 *     positions < lengths[b] attended, returns o plus the running max and
 *     softmax denominator.
 *   jpt_attn_dense  - dense_attention / flash_attention (:605-710): all `seq`
 *     positions (or < lengths[b] when given) plus an optional additive mask.
 *   jpt_attn_paged  - call_paged_attention (:789-808): keys are pages
 *     (kv_heads, total_pages, page_size, dim) addressed through page_table
 *     (batch, max_pages); lengths required.
 *
 * q, out: (batch, q_heads, q_rows, dim) in q_dtype (bf16 or f32).  k, v in
 * kv_dtype (bf16, f32 or int8).  k_scale/v_scale: NULL, or
 * (batch, scale_heads, seq) [paged: (scale_heads, total_pages, page_size)]
 * in scale_dtype; scores are multiplied by k_scale and probabilities by
 * v_scale after the row sum, as the reference does (:303-315, :660-679).
 * out_max/out_denom: NULL or float32 (batch, q_heads, q_rows): row max of
 * the scaled scores (natural-log units) and the sum of exp(score - max).
 * A row that attends nothing gives out = 0, max = -inf, denom = 0.
 *
 * mask: NULL or additive mask in mask_dtype, element
 * (b, h, t, s) at mask + b*mask_stride_b + h*mask_stride_h + t*mask_stride_t + s
 * (strides in elements; 0 broadcasts).
 *
 * new_k/new_v: NULL, or the step's new token (batch, kv_heads, 1, dim) in
 * kv_dtype with new_k_scale/new_v_scale (batch, scale_heads) when
 * quantised; it is attended as one more position and merged by
 * log-sum-exp, which is what AttentionKernel / Int8KVAttentionKernel do in
 * lazy-update mode with a second flash_attention call and seven elementwise
 * ops (layers.py:534-550, :702-718).
 *
 * new_k_raw/new_v_raw: NULL, or the new token before quantisation,
 * (batch, kv_heads, 1, dim) bf16, for an int8 cache.  The call then also does
 * the work of jpt_kv_append_quant_i8 for that token (Int8KVCacheGenerate.update's
 * quantize, cache_manager.py:532-537, 606-633): new_k/new_v and
 * new_k_scale/new_v_scale become OUTPUTS that receive its codes and scales
 * (bit-identical to jpt_kv_append_quant_i8 with `new_rounding`), and the token is
 * attended with them.  One launch less per layer; the reference has the
 * quantiser and the attention as separate XLA ops.
 *
 * new_to_pages (jpt_attn_paged only): the call also does the work of
 * jpt_paged_append / jpt_paged_append_quant_i8 for the new token
 * (PageKVCacheGenerate.update, cache_manager.py:663-724): `lengths` are the
 * slots' lengths BEFORE the step; the token of slot b is attended and written
 * to position lengths[b] of the slot - page page_table[b][lengths[b] /
 * page_size], whose id the allocator has already put there - codes (or bf16
 * rows) into k/v, scales into k_scale/v_scale, which become outputs for those
 * rows.  A slot of length 0 is inactive, as in the reference's token indices
 * (page_attention_manager.py:145-177): nothing is written or attended for it.
 * Needs the streaming kernel's shapes (dim 128, bf16 query, page_size a
 * multiple of 32); other shapes are refused.
 *
 * workspace: device scratch of at least jpt_attn_workspace_bytes(args)
 * bytes, 256-byte aligned.  Its first JPT_ATTN_WS_STATE_BYTES (the state
 * block) must be zero before the first call; calls sharing one workspace
 * must not overlap in time.
 *
 * Errors.  Shape and state errors are refused before anything is enqueued
 * (JPT_E_BADARG; the reference raises on them, attention_kernel.py:525-526,
 * :547-550).  Every wait inside the streaming kernel is bounded; a wave whose
 * wait runs out gives up, the launch ends, and word 0 of the state block is
 * set and stays set: what the launch wrote - and what every later launch on
 * that workspace writes until jpt_attn_status has been called - is then not to
 * be used.  The launch itself cannot report this (the call only enqueues);
 * jpt_attn_status does, and puts the workspace's counters back to what a
 * fresh plan holds, so the plan stays usable afterwards.
 *
 * The device must be the launch's own.  The streaming kernel is one
 * persistent workgroup per compute unit (all of a unit's LDS), and a slot
 * that is cut into three or more chunks is folded by a wave that waits -
 * for some 60 ms at most - for chunks that belong to OTHER workgroups of
 * the same launch.  If part of the grid cannot be resident while the rest
 * runs (compute units masked off, or held for that long by a kernel of another
 * stream or process), that wait runs out and the launch gives up.  Kernels of
 * other streams that merely share the device delay it, they do not break it.
 * ---------------------------------------------------------------------- */
#define JPT_ATTN_WS_STATE_BYTES 65536
#define JPT_ATTN_STATUS_GAVE_UP 1
#define JPT_ATTN_STATUS_SLOT_FULL 2
#define JPT_ATTN_STATUS_PLAN_OVERFLOW 4

typedef struct {
  const void* q;
  /* k, v and their scales are read-only, except with new_to_pages, which writes
   * the new token's row and scales into them; new_k/new_v and their scales are
   * inputs, except with new_k_raw, which makes them outputs: hence no const */
  void* k;
  void* v;
  void* k_scale;
  void* v_scale;
  const int32_t* lengths;
  const int32_t* page_table;
  const void* mask;
  void* new_k;
  void* new_v;
  void* new_k_scale;
  void* new_v_scale;
  void* out;
  float* out_max;
  float* out_denom;
  void* workspace;
  int64_t workspace_bytes;
  int64_t mask_stride_b, mask_stride_h, mask_stride_t;
  int32_t batch, q_heads, kv_heads, q_rows, dim;
  int32_t seq;         /* dense/ragged: cache length; paged: ignored */
  int32_t total_pages; /* paged only */
  int32_t page_size;   /* paged only */
  int32_t max_pages;   /* paged only: row length of page_table */
  int32_t q_dtype, kv_dtype, scale_dtype, scale_heads, mask_dtype;
  float sm_scale;      /* multiplies q.k; 1/sqrt(dim) for ragged/dense/flash */
  int32_t force_generic; /* 1 = use the shape-generic kernel (testing aid) */
  int32_t reuse_plan;    /* 1 = the workspace already holds the split plan for
                            these lengths (same batch, heads and lengths as the
                            previous call on this workspace): skip planning.
                            A decode step plans once and reuses it per layer. */
  const void* new_k_raw; /* see above; both or neither */
  const void* new_v_raw;
  int32_t new_rounding;  /* JPT_ROUND_* of the fused quantiser */
  const float* new_k_rope; /* NULL, or rotary factors (batch, dim / 2, 2) as in
                              jpt_quant_append_args: new_k_raw is unrotated and is
                              rotated before it is quantised (needs new_k_raw) */
  int32_t new_to_pages;    /* see above */
} jpt_attn_args;

int64_t jpt_attn_workspace_bytes(const jpt_attn_args* args);
/* Plans the split of every slot's positions into workgroup-sized chunks and
 * stores the plan in args->workspace without running attention; later calls
 * on that workspace with reuse_plan = 1 skip planning.  Only lengths,
 * batch, q_heads, kv_heads, q_rows, seq (or max_pages and page_size when
 * `paged` is non-zero) and the workspace fields are read.  The reference
 * computes its per-step block tables the same way, once per decode step for
 * all layers (precompute_ragged_block_indices, engine.py:674-729). */
int32_t jpt_attn_plan(const jpt_attn_args* args, int32_t paged, void* stream);
int32_t jpt_attn_ragged(const jpt_attn_args* args, void* stream);
int32_t jpt_attn_dense(const jpt_attn_args* args, void* stream);
int32_t jpt_attn_paged(const jpt_attn_args* args, void* stream);
/* jpt_attn_ragged with the workspace inside the library: a device array of
 * JPT_ATTN_STATIC_SCRATCH_BYTES that every GPU the library runs on holds from
 * the moment its code is loaded there until the process ends.  No counterpart
 * in the reference; it is for callers that cannot allocate device memory -
 * code under HIP graph capture, tight serving loops, harnesses that forbid it.
 * The call allocates nothing (no hipMalloc, no hipFree, no allocating
 * library routine): it plans (unless reuse_plan), attends and merges like
 * jpt_attn_ragged, with identical results.  args->workspace and
 * workspace_bytes are ignored.  Shapes whose workspace
 * (jpt_attn_workspace_bytes) exceeds the array are refused with JPT_E_BADARG.
 * All calls on one GPU share that GPU's array, which keeps the last call's
 * plan (so reuse_plan works across calls with the same lengths): calls that
 * overlap in time on one GPU race, whatever their streams.
 * jpt_attn_status(NULL, ...) reads its status word on the current device. */
#define JPT_ATTN_STATIC_SCRATCH_BYTES (8 << 20)
int32_t jpt_attn_ragged_static(const jpt_attn_args* args, void* stream);

/* Waits for `stream`, then stores the workspace's status word into *status
 * and clears it.  Bits, sticky since the last call:
 *   JPT_ATTN_STATUS_GAVE_UP    a launch gave up (see Errors above);
 *   JPT_ATTN_STATUS_SLOT_FULL  a plan saw a slot whose length had reached the
 *     cache capacity (seq, or max_pages * page_size), whether or not the step
 *     carries a token: the slot is attended up to the capacity, and a token
 *     appended to it in that step is attended but NOT stored (every append on
 *     this path skips positions outside the cache; the reference's
 *     dynamic_update_slice would clamp the position and overwrite the last
 *     row, cache_manager.py:154-173);
 *   JPT_ATTN_STATUS_PLAN_OVERFLOW  a plan had more entries than its array
 *     holds (a fault of the library's own accounting): positions were left
 *     out, the results of launches on that plan are not to be used.
 * After JPT_ATTN_STATUS_GAVE_UP the call also clears the plan's arrival and
 * hand-out counters, which the launch that gave up may have left half counted.
 *  Synchronises: call it where the caller synchronises anyway (the
 * reference raises from inside its jitted step; a kernel cannot).  Not to be
 * called during stream capture.  workspace NULL: the library's own workspace
 * (jpt_attn_ragged_static) on the current device. */
int32_t jpt_attn_status(void* workspace, void* stream, int32_t* status);

/* Log-sum-exp merge of two partial attention results (layers.py:539-548):
 * out = (l1*a*o1 + b*o2*l2) / (a*l1 + b*l2), a = exp(m1-g), b = exp(m2-g),
 * g = max(m1, m2).  o*: (rows, dim) in dtype; m*, l*: float32 (rows). */
int32_t jpt_lse_merge(void* out, const void* o1, const float* m1,
                      const float* l1, const void* o2, const float* m2,
                      const float* l2, int64_t rows, int32_t dim,
                      int32_t dtype, void* stream);

/* ------------------------------------------------------------------------
 * Host page allocator: PageAttentionManager (page_attention_manager.py:21-64,
 * :145-177, :214-222).  FIFO free list, page table (batch, max_pages) int32
 * initialised to the sentinel total_pages-1, lengths (batch) int32.  The
 * tables live in host memory owned by the handle; jpt_pam_tables exposes
 * them (valid until jpt_pam_destroy).  `free_order` is NULL (pages are
 * handed out 0, 1, 2, ... as in the reference) or total_pages page ids.
 * All methods take one internal mutex.
 * ---------------------------------------------------------------------- */
typedef struct jpt_pam jpt_pam;

int32_t jpt_pam_create(int32_t batch, int32_t total_pages, int32_t page_size,
                       int32_t max_pages, const int32_t* free_order,
                       jpt_pam** out);
void jpt_pam_destroy(jpt_pam* pam);
int32_t jpt_pam_tables(jpt_pam* pam, int32_t** page_indices, int32_t** lengths);
/* reserve_pages_insert: sets lengths[slot], pops ceil(seq_len/ps) pages into
 * the row; *num_pages receives the count. */
int32_t jpt_pam_reserve_insert(jpt_pam* pam, int32_t slot, int32_t seq_len,
                               int32_t* num_pages);
/* reserve_pages_decode: pops one page when seq_len > 0 sits on a boundary. */
int32_t jpt_pam_reserve_decode(jpt_pam* pam, int32_t slot, int32_t seq_len);
/* fill_new_pages: reserve_pages_decode for every slot in ascending order. */
int32_t jpt_pam_fill_new_pages(jpt_pam* pam, const int32_t* lens);
/* get_page_token_indices: writes (3, n_active) row-major into out (capacity
 * 3*batch), sets *n_active, and lengths = lens == 0 ? 0 : lens + 1. */
int32_t jpt_pam_page_token_indices(jpt_pam* pam, const int32_t* lens,
                                   int32_t* out, int32_t* n_active);
/* free_pages_resource: returns the slot's pages to the tail of the free
 * list in row order, resets the row to the sentinel and the length to 0. */
int32_t jpt_pam_free(jpt_pam* pam, int32_t slot);
/* number of pages on the free list; with out != NULL (capacity total_pages)
 * also copies the list in FIFO order. */
int32_t jpt_pam_free_count(jpt_pam* pam, int32_t* out);

/* ------------------------------------------------------------------------
 * Device-resident page allocator: PageAttentionManager with its free list,
 * page table and lengths in HBM and every method a one-workgroup kernel, so a
 * paged decode step needs no host round trip (the reference pulls input_pos
 * to the host every step, engine.py:739-745) and can be captured in a HIP
 * graph.  Same FIFO order and tables as jpt_pam_* / the reference
 * (page_attention_manager.py:21-64, :145-177, :214-222), bit for bit.
 *
 * The caller owns the device arrays.  Kernels cannot raise: a failed request
 * is skipped and its bit is set in state[2] (JPT_DPAM_*), where it stays until
 * jpt_dpam_init; every access stays inside the arrays whatever the inputs.
 *   state[0] ring head, state[1] free pages, state[2] status bits,
 *   state[3] n_active of the last jpt_dpam_decode_step.
 * ---------------------------------------------------------------------- */
#define JPT_DPAM_NOPAGES 1  /* free list ran out (the reference raises queue.Empty) */
#define JPT_DPAM_OVERFLOW 2 /* a slot needs more than max_pages pages (IndexError) */
#define JPT_DPAM_BADARG 4   /* slot out of range or negative length */

typedef struct {
  int32_t* state;          /* (4) */
  int32_t* ring;           /* (total_pages) free list, FIFO */
  int32_t* page_indices;   /* (batch, max_pages); unused entries hold total_pages - 1 */
  int32_t* lengths;        /* (batch) positions the next paged attention attends */
  int32_t* n_alloc;        /* (batch) pages each slot was handed */
  int32_t* update_indices; /* (3, batch): rows page, j * page_size + token, slot of
                              the active slots; first state[3] columns valid */
  int32_t batch, total_pages, page_size, max_pages;
} jpt_dpam;

/* Free list = free_order (device, a permutation of the page ids) or 0, 1, 2...;
 * tables at their initial values (page_attention_manager.py:29-39). */
int32_t jpt_dpam_init(const jpt_dpam* pam, const int32_t* free_order, void* stream);
/* reserve_pages_insert for n_req requests, in order.  slots/seq_lens: device
 * arrays of n_req entries, or NULL to take the single request (slot, seq_len). */
int32_t jpt_dpam_reserve_insert(const jpt_dpam* pam, const int32_t* slots,
                                const int32_t* seq_lens, int32_t n_req,
                                int32_t slot, int32_t seq_len, void* stream);
/* free_pages_resource for n_req slots, in order (device array, or NULL and `slot`). */
int32_t jpt_dpam_free(const jpt_dpam* pam, const int32_t* slots, int32_t n_req,
                      int32_t slot, void* stream);
/* fill_new_pages(lens) then get_page_token_indices(lens): lens (batch) device. */
int32_t jpt_dpam_decode_step(const jpt_dpam* pam, const int32_t* lens, void* stream);

/* ------------------------------------------------------------------------
 * Decode-state bookkeeping of one generate step on the device
 * (engine.py:774-817).  update_mask: mask[b, input_pos[b]] = 0, or
 * mask[:, current_position] = 0 with a ring buffer.  advance: input_pos and
 * lens become x == 0 ? 0 : x + 1 (ring buffer: x + 1).  The mask update reads
 * input_pos before it advances.  mask (batch, seq) f32 or bf16, rows
 * mask_stride elements apart, may be NULL; input_pos, lens (batch) int32, lens
 * may be NULL.
 * ---------------------------------------------------------------------- */
int32_t jpt_decode_advance(void* mask, int32_t mask_dtype, int64_t mask_stride,
                           int32_t* input_pos, int32_t* lens, int32_t batch,
                           int32_t seq, int32_t ring_buffer,
                           int32_t current_position, int32_t update_mask,
                           int32_t advance, void* stream);

/* ------------------------------------------------------------------------
 * Engine.precompute_ragged_block_indices (engine.py:674-729): for every grid
 * cell (slot b, block i) of the reference's ring-aware ragged kernel, the
 * (slot, block) it works on.  start, input_pos (batch) int32 on the device,
 * end = (start + input_pos) % cache_len; b_next, i_next (batch, cache_len /
 * block_size) int32.  The attention entry points above do not read these
 * tables (nor does the reference's live kernel, attention_kernel.py:561-579);
 * provided for callers that carry them in their decode state.
 * ---------------------------------------------------------------------- */
int32_t jpt_ragged_block_indices(const int32_t* start, const int32_t* input_pos,
                                 int32_t batch, int32_t cache_len,
                                 int32_t block_size, int32_t* b_next,
                                 int32_t* i_next, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* JPT_MI355_H_ */
