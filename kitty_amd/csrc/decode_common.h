// Pieces shared by the decode-attention kernels: per-sequence occupancy, the tiling of a
// sequence into 128-token tiles, the split-K workspace layout and the merge kernel.
//
// Token order (kitty_attention.py:89-207 for K, :270-386 for V) is chronological on both sides:
//   K: [ sink rows | packed pages | Q_Buffer_K rows ]
//   V: [ sink rows | packed pages | Q_Buffer_V rows | Local_Buffer_V rows from the ring head ]
// Both sides start their pages right after the sink, so "body tile" i (tokens 128*i .. 128*i+127
// after the sink) is K page i when i < PageCount_K, else the K Q-buffer; on the V side it is V
// page i when i < PageCount_V, else rows of the fp16 region [Q_Buffer_V | Local ring].
// Tile 0 is the sink; body tile i is tile i+1.
#pragma once
#include "kitty_common.h"

namespace kitty {

__host__ __device__ inline int c_div_up(int a, int b) { return (a + b - 1) / b; }

struct SeqCounts {
  int sink, pk, rk, pv, rv, lv, off;
  int nbody;    // tokens after the sink
  int ntiles;   // 1 (sink) + ceil(nbody / 128)
};

__device__ inline SeqCounts load_counts(const kitty_kv_layer& L, int b) {
  int c[KITTY_SEQ_COUNT_FIELDS];
#pragma unroll
  for (int i = 0; i < KITTY_SEQ_COUNT_FIELDS; ++i)
    c[i] = L.seq_counts ? L.seq_counts[b * KITTY_SEQ_COUNT_FIELDS + i] : L.counts[i];
  SeqCounts s;
  // clamp to what the buffers hold: device-side counts cannot be validated on the host
  s.sink = min(max(c[KITTY_CNT_SINK], 0), L.S);
  s.pk = min(max(c[KITTY_CNT_PAGES_K], 0), L.MAX_PAGE);
  s.rk = min(max(c[KITTY_CNT_QBUF_K], 0), kPage);
  s.pv = min(max(c[KITTY_CNT_PAGES_V], 0), L.MAX_PAGE);
  s.rv = min(max(c[KITTY_CNT_QBUF_V], 0), kPage);
  s.lv = min(max(c[KITTY_CNT_LOCAL_V], 0), kPage);
  s.off = c[KITTY_CNT_LOCAL_OFF] & (kPage - 1);
  if (L.cache_pages_k <= 0) s.pk = 0;   // no page to read, whatever the counters say
  if (L.cache_pages_v <= 0) s.pv = 0;
  s.nbody = min(s.pk * kPage + s.rk, s.pv * kPage + s.rv + s.lv);
  s.ntiles = 1 + (s.nbody + kPage - 1) / kPage;
  return s;
}

// One entry of a page table.  The tables are not written while an attention kernel runs, and the
// compiler cannot know that (the global -> LDS loads are memory writes to it, so every later table
// read counts as possibly changed): read through the constant address space, the entry of a
// wave-uniform index is a scalar load, which neither occupies the vector memory queue nor makes
// the wave wait for the tile loads in flight.
__device__ __forceinline__ int64_t page_id(const int64_t* table, int64_t index) {
  typedef const int64_t __attribute__((address_space(4)))* const_ptr;
  return *(const_ptr)(uintptr_t)(table + index);
}
// A page id as read from a page table, made safe to dereference.  The counters and tables of a
// layer may be written by the caller on the device, so the host cannot vouch for them: an id outside
// [0, cache_pages) (an entry of -1 = no page assigned, or garbage) reads page 0 instead and is noted
// in `bad`; the output of that sequence is then meaningless, but nothing outside the page arrays is
// touched.  The note reaches the sequence's status row once, when the kernel is done
// (report_bad_page): a store next to the table reads would make the compiler treat every later
// table read as possibly changed by it, and turn the scalar loads of the streaming loops into
// vector loads with full waits.
__device__ __forceinline__ int64_t checked_page(int64_t pg, int64_t cache_pages, int& bad) {
  const bool ok = pg >= 0 && pg < cache_pages;
  bad |= ok ? 0 : 1;
  return ok ? pg : 0;
}
__device__ __forceinline__ void report_bad_page(const kitty_kv_layer& L, int b, int bad) {
  if (bad && L.status) L.status[b * KITTY_STATUS_FIELDS + KITTY_STATUS_BAD_PAGE_READ] = 1;
}

// fp16 row of V for token u of the region that follows the V pages
__device__ inline const __half* v_tail_row(const kitty_kv_layer& L, const SeqCounts& c, int b, int h, int u,
                                          int head_dim = kD) {
  const int64_t base = (int64_t)b * L.win_stride_b + (int64_t)h * L.win_stride_h;
  if (u < c.rv) return (const __half*)((const uint8_t*)L.qbuf_v + base) + (int64_t)u * head_dim;
  const int r = (c.off + (u - c.rv)) & (kPage - 1);
  return (const __half*)((const uint8_t*)L.local_v + base) + (int64_t)r * head_dim;
}

// Split-K workspace: [B*H_Q*splits][2] floats (running max of the logits in log2 units, i.e.
// logit * log2(e); running sum of 2^(logit2 - max)), then 256-aligned, [B*H_Q*splits][D] floats
// of un-normalised output.
__host__ __device__ inline size_t ws_ml_bytes(int B, int H_Q, int splits) {
  size_t n = (size_t)B * H_Q * splits * 2 * sizeof(float);
  return (n + 255) & ~(size_t)255;
}
__host__ __device__ inline size_t ws_acc_bytes(int B, int H_Q, int splits, int head_dim = kD) {
  return (size_t)B * H_Q * splits * head_dim * sizeof(float);   // a multiple of 256
}
// After the partials: the work list of a launch that runs in several rounds (decode_plan_kernel) -
// kPlanHeader words, of which the first is the number of items, then one word per item
// (batch row << 16 | split), at most B * splits of them.
constexpr int kPlanHeader = 4;
__host__ __device__ inline size_t ws_plan_bytes(int B, int splits) {
  size_t n = ((size_t)B * splits + kPlanHeader) * sizeof(uint32_t);
  return (n + 255) & ~(size_t)255;
}
__host__ __device__ inline size_t ws_total_bytes(int B, int H_Q, int splits, int head_dim = kD) {
  return ws_ml_bytes(B, H_Q, splits) + ws_acc_bytes(B, H_Q, splits, head_dim) + ws_plan_bytes(B, splits);
}

}  // namespace kitty
