/*
 * kitty_hip.h - C ABI of the MI355X (gfx950) implementation of Kitty's quantized-KV hot path.
 *
 * Every entry point is asynchronous and ordered on the HIP stream passed in (NULL = the default
 * stream), allocates nothing and frees nothing.  State kept between calls: a thread-local error
 * string, the thread-local events of kitty_profile_next_split, the device's SIMD count (asked once)
 * and, for kitty_decode_attn_static, the address of its array on each device.  All data pointers
 * are device pointers owned by the caller.  Return value: 0 on
 * success, a negative KITTY_E_* code when an argument is rejected on the host before anything is
 * launched, a positive hipError_t when a launch fails.  kitty_last_error() describes the last
 * failure on the calling thread.
 *
 * Each function names the reference interface it replaces (paths relative to the reference
 * checkout, src/kitty/kvcache/...).
 *
 * Head dimensions: D = 128 runs on the tuned kernels; D = 64 and D = 256 are served by plain kernels
 * with the same arithmetic and storage format (the reference's kernels take D as a parameter,
 * kernels/kitty_quant_pack.py:42-45, kernels/kitty_attention.py:59-62); any other D is KITTY_E_SHAPE.
 * PAGE_SIZE is 128.
 */
#ifndef KITTY_HIP_H
#define KITTY_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define KITTY_ABI_VERSION 2

enum {
  KITTY_OK = 0,
  KITTY_E_NULL = -1,        /* a required pointer is NULL */
  KITTY_E_SHAPE = -2,       /* unsupported head_dim / page_size / boost count / group size */
  KITTY_E_RANGE = -3,       /* a count or offset is out of range for the buffers described */
  KITTY_E_ALIGN = -4,       /* a pointer or stride breaks the alignment the kernels rely on */
  KITTY_E_WORKSPACE = -5    /* workspace too small */
};

/*
 * One layer's storage, field for field the tensors of the reference's KVCache_Layer
 * (utils_kv_per_layer.py:12-95).  Strides are in bytes, except the page-table row strides, which
 * count int64 entries.  fp16 windows are [MAX_BS, H_KV, rows, D]
 * with D contiguous; *_stride_b / *_stride_h give their batch and head strides.
 *
 * Occupancy is given either by the scalar counters (the reference: host ints shared by the whole
 * batch, utils_kv_per_layer.py:53-54,65,71-72,79-80) or, when seq_counts is not NULL, per
 * sequence: int32 [B][KITTY_SEQ_COUNT_FIELDS] on the device in the order of the enum below.
 */
enum {
  KITTY_CNT_SINK = 0,       /* Sink_Count            (0..S)                                   */
  KITTY_CNT_PAGES_K = 1,    /* PageCount_K                                                    */
  KITTY_CNT_QBUF_K = 2,     /* Q_Buffer_Count_K      (0..PAGE_SIZE)                           */
  KITTY_CNT_PAGES_V = 3,    /* PageCount_V                                                    */
  KITTY_CNT_QBUF_V = 4,     /* Q_Buffer_Count_V      (0..PAGE_SIZE)                           */
  KITTY_CNT_LOCAL_V = 5,    /* Local_Count_V         (0..PAGE_SIZE)                           */
  KITTY_CNT_LOCAL_OFF = 6,  /* Write_Offset_Local_V  (ring head = oldest row)                 */
  KITTY_CNT_FLAGS = 7,      /* KITTY_SEQ_* bits                                               */
  KITTY_SEQ_COUNT_FIELDS = 8
};
/* Flag bits of a sequence's counter row.  INACTIVE: the slot holds no sequence (or a paused one):
 * the append and flush entry points leave it alone; attention still sees what its counters
 * describe, nothing when they are zero. */
enum { KITTY_SEQ_INACTIVE = 1 };

/*
 * Device-side status, one row of int32 per sequence (kitty_kv_layer.status, optional).  The
 * reference stops with a Python assert before a buffer overflows (kitty.py:109,113,118) or a page
 * is missing; kernels that take their occupancy from device memory cannot, so they skip the work
 * that would go out of bounds, exit normally and leave a record here.  The words are sticky: the
 * kernels only ever raise them, the host reads and clears them when it wants to know.
 */
enum {
  KITTY_STATUS_TOKENS_DROPPED = 0,   /* count: tokens not appended because a Q-buffer was still full
                                        (or, for a chunk, because it did not fit)                    */
  KITTY_STATUS_FLUSH_SKIPPED = 1,    /* count: full Q-buffers left unflushed (no page assigned, or
                                        the sequence is at MAX_PAGE)                                 */
  KITTY_STATUS_BAD_PAGE_WRITE = 2,   /* flag: a quantize / flush kernel met a page id outside
                                        [0, cache_pages) other than -1 and wrote nothing             */
  KITTY_STATUS_BAD_PAGE_READ = 3,    /* flag: an attention kernel met a page id outside
                                        [0, cache_pages); it read page 0 instead, the output of that
                                        sequence is meaningless                                      */
  KITTY_STATUS_FIELDS = 4
};

typedef struct kitty_kv_layer {
  int32_t H_KV, D, D_BOOSTED, PAGE_SIZE, S, MAX_PAGE;
  int32_t counts[KITTY_SEQ_COUNT_FIELDS];       /* used when seq_counts == NULL */
  const int32_t* seq_counts;                    /* optional, device, [B][8]; the two append
                                                   entry points below write it */

  int32_t* status;                              /* optional, device, [B][KITTY_STATUS_FIELDS]  */
  int64_t cache_pages_k, cache_pages_v;         /* pages the K / V arrays below hold: every page id
                                                   read from a page table is checked against them */

  const uint8_t* key_cache;    int64_t key_cache_stride_page;     /* KeyCache            */
  const void*    key_meta;     int64_t key_meta_stride_page;      /* KeyCache_metadata   */
  const uint8_t* value_cache;  int64_t value_cache_stride_page;   /* ValueCache          */
  const void*    value_meta;   int64_t value_meta_stride_page;    /* ValueCache_metadata */
  const int64_t* page_table_k; int64_t page_table_k_stride_b;     /* PageTable_K, stride in entries */
  const int64_t* page_table_v; int64_t page_table_v_stride_b;     /* PageTable_V, stride in entries */

  const void* sink_k;  const void* sink_v;      /* Sink_Buffer_K/V  [MAX_BS,H_KV,S,D]         */
  int64_t sink_stride_b, sink_stride_h;
  const void* qbuf_k;  const void* qbuf_v;      /* Q_Buffer_K/V     [MAX_BS,H_KV,PAGE_SIZE,D] */
  const void* local_v;                          /* Local_Buffer_V   [MAX_BS,H_KV,PAGE_SIZE,D] */
  int64_t win_stride_b, win_stride_h;           /* shared by the three PAGE_SIZE-row windows  */
} kitty_kv_layer;

int kitty_abi_version(void);
const char* kitty_last_error(void);

/*
 * Channel-boost selection.  Replaces the torch ops of quantize_pack_k
 * (kernels/kitty_quant_pack.py:275-288): score = mean over the page's tokens of |K| rounded to
 * fp16, top-d_boost channels, slot_map[ch] = rank or d_boost.  Tie rule: higher score first, then
 * lower channel index.  key is fp16 [B,H,T,D] with D contiguous and byte strides as given; pages
 * are the `pages` consecutive PAGE_SIZE-token groups starting at token t_offset.
 * slot_map: uint8 [B,H,pages,D] contiguous.
 */
int kitty_select_boost_k(const void* key, int64_t stride_b, int64_t stride_h, int64_t stride_t,
                         int B, int H, int T, int D, int t_offset, int pages, int page_size, int d_boost,
                         uint8_t* slot_map, void* stream);

/*
 * Replaces quantize_pack_k_kernel and its launch (kernels/kitty_quant_pack.py:13-152, 291-312).
 * Quantizes `pages` pages of every (b,h) into cache pages page_table[b][page_offset + p].
 * slot_map NULL: the selection above is fused into the same kernel (one pass over K).
 * slot_map given: uint8 [B,H,pages,D], consumed exactly like the reference kernel consumes
 * dense_sparse_idx.  meta is fp16 [pages_total,H,D,2] (scale, zero).  page_table_stride_b counts
 * int64 entries; every other stride is in bytes.  A page id outside [0, cache_pages) is never
 * written to; status (optional, device, [B][KITTY_STATUS_FIELDS]) records it.
 */
int kitty_quant_pack_k(const void* key, int64_t stride_b, int64_t stride_h, int64_t stride_t,
                       int B, int H, int T, int D, int t_offset, int pages, int page_size, int d_boost,
                       const uint8_t* slot_map,
                       const int64_t* page_table, int64_t page_table_stride_b, int page_offset,
                       uint8_t* cache, int64_t cache_stride_page,
                       void* meta, int64_t meta_stride_page,
                       int64_t cache_pages, int32_t* status, void* stream);

/*
 * Replaces quantize_pack_v_kernel and its launch (kernels/kitty_quant_pack.py:155-249, 339-356).
 * meta is fp16 [pages_total,H,PAGE_SIZE,2] (scale, zero) per token.
 */
int kitty_quant_pack_v(const void* value, int64_t stride_b, int64_t stride_h, int64_t stride_t,
                       int B, int H, int T, int D, int t_offset, int pages, int page_size,
                       const int64_t* page_table, int64_t page_table_stride_b, int page_offset,
                       uint8_t* cache, int64_t cache_stride_page,
                       void* meta, int64_t meta_stride_page,
                       int64_t cache_pages, int32_t* status, void* stream);

/*
 * Decode attention over the packed cache.  Replaces qk_kernel + torch softmax + sv_kernel as
 * orchestrated by kitty_attention_forward (kernels/kitty_attention.py:403-526): one fused
 * split-K pass (QK^T, online softmax, PV per split of the sequence) and a merge pass.
 * q: fp16 [B,H_Q,1,D] contiguous.  out: fp16 [B,1,H_Q,D] contiguous.
 * workspace: at least kitty_decode_attn_workspace_bytes(B,H_Q,D,num_splits) bytes, 256-aligned.
 * num_splits <= 0 picks kitty_decode_attn_default_splits() (max_tiles = 1 + the 128-token tiles
 * after the sink of the longest sequence; per_sequence_counts = layer->seq_counts is set).
 * variant: 0 = default kernel, 1 = the plain reference-order kernel (fp16 dequantization, no
 * matrix cores).  For D = 64 / 256 both values run the same plain kernel.
 */
size_t kitty_decode_attn_workspace_bytes(int B, int H_Q, int D, int num_splits);
int kitty_decode_attn_default_splits(int B, int H_KV, int max_tiles, int per_sequence_counts);
int kitty_decode_attn(const kitty_kv_layer* layer, const void* q, int B, int H_Q, float scaling,
                      void* out, void* workspace, size_t workspace_bytes, int num_splits,
                      int variant, void* stream);

/*
 * The two passes of kitty_decode_attn on their own.  The split pass leaves, per (b, hq, split),
 * the running maximum of the logits in log2 units, the running sum and the un-normalised output
 * in the workspace; the merge pass combines `num_splits` such partials per (b, hq).  A caller that
 * shards one long sequence over several devices runs the split pass on each shard, gathers the
 * partials into one workspace (splits of all shards side by side) and runs the merge pass once.
 * (The last kitty_decode_attn_workspace_bytes() - partials bytes of a workspace belong to the split
 * pass alone: when it has more workgroups than the device holds at once and the batch is larger than
 * 256 sequences (or a kv head serves more than 8 query heads), a small kernel ahead of it leaves the
 * list of the splits that have work there.  The merge pass does not read them.)
 * No counterpart in the reference, whose grid is (B, H_KV) with no split over the sequence
 * (kernels/kitty_attention.py:433,484).
 */
int kitty_decode_attn_split(const kitty_kv_layer* layer, const void* q, int B, int H_Q, float scaling,
                            void* workspace, size_t workspace_bytes, int num_splits, int variant,
                            void* stream);
int kitty_decode_attn_merge(const void* workspace, size_t workspace_bytes, int B, int H_Q, int D,
                            int num_splits, void* out, void* stream);

/*
 * Measurement aid, no counterpart in the reference (which times whole generate() calls,
 * latency_benchmarking/benchmark_kitty.py:129-183): the next split pass that the calling thread
 * launches (kitty_decode_attn_split, or inside kitty_decode_attn) attaches the two hipEvent_t to its
 * kernel's own dispatch, so that hipEventElapsedTime between them is the kernel's duration on the
 * device - the figure a kernel trace reports - without the host's enqueue gaps that an event pair
 * recorded around the call includes.  The events must have timing enabled and outlive the launch.
 * (NULL, NULL) cancels.  The plain variant records the events around its launch instead.  The pair
 * belongs to the next kitty_decode_attn_split call of the thread whether that call launches or is
 * rejected: a rejected call disarms it too.  Measurement plumbing only: a caller that never calls
 * this can ignore it.
 */
int kitty_profile_next_split(void* start_event, void* stop_event);

/*
 * kitty_decode_attn without a workspace argument and without any allocation: the split-K partials
 * go to an array of KITTY_STATIC_WORKSPACE_BYTES that is part of the library's device image (one copy
 * per device, held until the process ends).  No counterpart in the reference; it is for callers that
 * cannot allocate: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
 * Same kernels, same results as kitty_decode_attn with the same num_splits.  num_splits <= 0 picks
 * kitty_decode_attn's default, cut back to what the array holds; an explicit num_splits whose
 * partials ((2 + D) floats per batch row, query head and split) exceed the array is rejected with
 * KITTY_E_WORKSPACE.  The device that owns the tensors must be the current device.  All calls on one
 * device share the array: calls that overlap there (different streams or threads) race; calls
 * ordered on one stream do not, and nothing in the array needs clearing between them.
 * The first call on a device looks the array's address up in the runtime (hipGetSymbolAddress, under
 * a mutex): make it before capturing a stream, not inside the capture - a first call on a capturing
 * stream is rejected with KITTY_E_RANGE.  Later calls only read the cached address.
 */
#define KITTY_STATIC_WORKSPACE_BYTES (16u << 20)
int kitty_decode_attn_static(const kitty_kv_layer* layer, const void* q, int B, int H_Q, float scaling,
                             void* out, int num_splits, int variant, void* stream);

/*
 * Chunked-prefill attention: T_q new tokens attend to everything the layer already holds (sink
 * rows, packed pages, fp16 windows, in the token order of decode) and, causally, to the keys and
 * values of the chunk itself, which are still fp16 and not yet appended.  An extension: the
 * reference asserts t_query == 1 (kernels/kitty_attention.py:411) and prefills an empty cache
 * with dense attention (benchmark_kitty.py:302); the arithmetic per cached token is that of
 * qk_kernel / sv_kernel (kitty_attention.py:162-165, 317-320).  With an empty layer this is plain
 * causal attention.
 * q: fp16 [B,H_Q,T_q,D], k_new / v_new: fp16 [B,H_KV,T_q,D] (one set of strides for both), D
 * contiguous, byte strides as given.  out: fp16 [B,T_q,H_Q,D] contiguous.  No workspace.
 */
int kitty_prefill_attn(const kitty_kv_layer* layer,
                       const void* q, int64_t q_stride_b, int64_t q_stride_h, int64_t q_stride_t,
                       const void* k_new, const void* v_new,
                       int64_t new_stride_b, int64_t new_stride_h, int64_t new_stride_t,
                       int B, int H_Q, int T_q, float scaling, void* out, void* stream);

/*
 * Decode-time bookkeeping with per-sequence counters kept on the device (layer->seq_counts must be
 * set; it is read AND written; layer->status, when set, is written).  The reference keeps one set of host ints for the whole batch and
 * drives slice copies from them (KittyCache.update, kitty.py:97-123; quantize_decode,
 * kitty.py:194-236); these calls run the same state machine per sequence, with no host
 * round trip, so that sequences of different lengths decode in one batch and the launch sequence
 * of a decode step never changes (a captured graph can replay it).  Call order per step, as in
 * modeling_qwen3.py:225-251: kitty_append_token, kitty_decode_attn, kitty_flush_full.
 *
 * kitty_append_token: one token per sequence.  k_new / v_new: fp16 [B,H_KV,1,D], D contiguous, byte
 * strides.  Per sequence: sink not full -> the sink row; else K -> Q_Buffer_K[Q_Buffer_Count_K],
 * V -> the local ring (a full ring first moves its oldest row to Q_Buffer_V).  A sequence whose
 * Q-buffer is full (a skipped kitty_flush_full) is left unchanged, the token dropped and counted in
 * status[KITTY_STATUS_TOKENS_DROPPED].
 * rope_cos / rope_sin (optional, both or neither): fp16 [B,D] rows with byte stride rope_stride_b,
 * the rotary embedding of each sequence's position.  When given, k_new holds the keys BEFORE the
 * rotation and the kernel stores k * cos + rotate_half(k) * sin, each product and the sum rounded
 * to fp16, which is what the caller's own fp16 tensor expression computes
 * (modeling_qwen3.py:215-220 feeding kitty.py:102-123): one launch less and no rotated copy of K.
 *
 * These three entry points are built for D = 128 (KITTY_E_SHAPE otherwise).
 *
 * kitty_flush_full: every sequence whose K (V) Q-buffer holds PAGE_SIZE rows gets it quantized,
 * with channel selection, into page page_table[b][PageCount] and its counters advanced; the
 * arithmetic is that of kitty_quant_pack_k / _v.  A sequence already at MAX_PAGE pages, or whose
 * page id is outside [0, layer->cache_pages_k / _v) (a page table entry of -1: no page assigned),
 * is left as it is, Q-buffer full, counted in status[KITTY_STATUS_FLUSH_SKIPPED], and drops the
 * tokens appended until a later call finds a page there.
 *
 * kitty_append_chunk: T >= 1 tokens per sequence in one call, k_new / v_new fp16 [B,H_KV,T,D].  The
 * state afterwards is the one T rounds of kitty_append_token + kitty_flush_full leave: same
 * counters, same packed pages bit for bit, same fp16 rows in the same slots of the sink, the
 * Q-buffers and the ring (rows of a Q-buffer beyond its fill count are not part of the state).
 * Pages that fill up inside the chunk are quantized straight from their sources (buffered rows
 * and chunk rows) without a trip through the Q-buffer.  A sequence the chunk does not fit (it
 * would pass MAX_PAGE, or needs a page whose table entry is not a valid page id) is left
 * unchanged and its T tokens counted as dropped.  No counterpart in the reference, whose update()
 * asserts one token per call once the cache holds anything (kitty.py:97-98).
 */
int kitty_append_token(const kitty_kv_layer* layer, const void* k_new, const void* v_new,
                       int64_t stride_b, int64_t stride_h,
                       const void* rope_cos, const void* rope_sin, int64_t rope_stride_b,
                       int B, void* stream);
int kitty_flush_full(const kitty_kv_layer* layer, int B, void* stream);
int kitty_append_chunk(const kitty_kv_layer* layer, const void* k_new, const void* v_new,
                       int64_t stride_b, int64_t stride_h, int64_t stride_t, int B, int T, void* stream);

/*
 * Fake quantization of dense fp16 keys or values in place: replaces fake_quant_groupwise_lastdim of
 * the reference's accuracy simulator (src/kitty_sim/utils_quant.py:64-114) on the slices its cache
 * hands it (src/kitty_sim/kitty_simulate.py:196-252).  Arithmetic as that function evaluates on a GPU
 * for fp16 tensors: every operator rounds its result to fp16, the range is floored at 1e-4, the code
 * is clamped to [0, 2^bit - 1] and then rounded half to even.
 * data: fp16 [B,H,T,D], D contiguous, byte strides; tokens [t_offset, t_offset + n_tokens) are
 * rewritten.  axis 0: groups of group_size consecutive tokens per channel (keys; n_tokens must be a
 * multiple of group_size; groups are counted from t_offset); promote_mask (optional, uint8 / bool,
 * nonzero = promote_bit instead of bit) is indexed [b][h][tile][channel] through its byte strides,
 * tile = 128-token block from t_offset (mask_stride_tile 0: one mask for all tokens, as the reference's
 * [B,nh,D] mask).  axis 1: groups of group_size consecutive channels per token (values), no mask.
 * group_size 32, 64 or 128; bit widths 1..8.
 */
int kitty_fake_quant(void* data, int64_t stride_b, int64_t stride_h, int64_t stride_t, int B, int H, int T, int D,
                     int t_offset, int n_tokens, int axis, int group_size, int bit,
                     const uint8_t* promote_mask, int64_t mask_stride_b, int64_t mask_stride_h,
                     int64_t mask_stride_tile, int promote_bit, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* KITTY_HIP_H */
