// C ABI entry points of decode attention: argument checks on the host, then the fused split-K
// pass and the merge pass on the caller's stream.
#include "decode_common.h"

namespace kitty {
void launch_decode_plain(const kitty_kv_layer& L, const void* q, int B, int H_Q, float scaling, float* ws_ml,
                         float* ws_acc, int num_splits, hipStream_t stream);
void launch_decode_merge(const float* ws_ml, const float* ws_acc, void* out, int B, int H_Q, int num_splits,
                         hipStream_t stream);
bool decode_mfma_supported(const kitty_kv_layer& L, int H_Q);
void launch_decode_mfma(const kitty_kv_layer& L, const void* q, int B, int H_Q, float scaling, float* ws_ml,
                        float* ws_acc, uint32_t* ws_plan, int num_splits, int n_simds, hipStream_t stream,
                        hipEvent_t ev_start, hipEvent_t ev_stop);
void launch_prefill_attn(const kitty_kv_layer& L, const void* q, int64_t q_stride_b, int64_t q_stride_h,
                         int64_t q_stride_t, const void* k_new, const void* v_new, int64_t new_stride_b,
                         int64_t new_stride_h, int64_t new_stride_t, int B, int H_Q, int Tq, float scaling,
                         void* out, hipStream_t stream);
// head dimensions other than 128 (any_dim.hip)
void launch_decode_any(const kitty_kv_layer& L, const void* q, int B, int H_Q, float scaling, float* ws_ml,
                       float* ws_acc, int num_splits, hipStream_t stream);
void launch_merge_any(int D, const float* ws_ml, const float* ws_acc, void* out, int B, int H_Q, int num_splits,
                      hipStream_t stream);
void launch_prefill_any(const kitty_kv_layer& L, const void* q, int64_t q_stride_b, int64_t q_stride_h,
                        int64_t q_stride_t, const void* k_new, const void* v_new, int64_t new_stride_b,
                        int64_t new_stride_h, int64_t new_stride_t, int B, int H_Q, int Tq, float scaling, void* out,
                        hipStream_t stream);
}  // namespace kitty

using namespace kitty;

extern "C" size_t kitty_decode_attn_workspace_bytes(int B, int H_Q, int D, int num_splits) {
  if (B <= 0 || H_Q <= 0 || !head_dim_supported(D) || num_splits <= 0) return 0;
  return ws_total_bytes(B, H_Q, num_splits, D);
}

namespace kitty {
// SIMDs of the current device (4 per compute unit), asked once per process; 1024 (a whole MI355X)
// when there is no device to ask, so that the split rule can be evaluated without one.
int device_simds() {
  static const int n = [] {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) {
      (void)hipGetLastError();
      cus = 256;
    }
    return 4 * cus;
  }();
  return n;
}
}  // namespace kitty

// Enough single-wave workgroups to put two on every SIMD of the device.  When the splits are short
// (under 8 tiles) the waves with the fp16 rows are the critical path, and a launch that fills the
// machine exactly puts two of them on the same SIMD (workgroup i shares a SIMD with i + SIMDs):
// 15/16 of the machine is faster then (B=1, 128k tokens: 32 us with 240 splits, 40 us with 256).
// A short context is latency, not bandwidth: a body split of 2.5 tiles (a wave's fixed cost is
// about two tiles' worth) plus three splits for the sink and the tiles with fp16 rows (B=1, 4k
// tokens: 11.4 us with 16 splits, 13.5 with 12, 17.4 with 8; 16k tokens: 14.0 us with 54, 15.8 with
// 36), and then, if it can be had with body splits of 4 tiles or fewer, a launch of at most 3/4 of
// a workgroup per SIMD, in which no two waves share one (B=4, 8k tokens: 15.0 us with 24 splits,
// 16.8 with 32, 23.9 with 64), else one of at most six workgroups per compute unit (B=2, 32k tokens:
// 18.0 us with 96 splits, 19.5 with 48 or 68, 18.6 with 120; B=1, 64k: 18.8 with 192, 20.2 with 132).
// Sequences with their own lengths (per_sequence_counts) get at least 12 splits when they can be
// long: more, shorter splits even out the load.
extern "C" int kitty_decode_attn_default_splits(int B, int H_KV, int max_tiles, int per_sequence_counts) {
  if (B <= 0 || H_KV <= 0 || max_tiles <= 0) return 1;
  const int64_t units = (int64_t)B * H_KV;
  const int simds = device_simds(), slots = 2 * simds;
  int64_t s = (slots + units - 1) / units;
  if (max_tiles < 8 * s) s = (slots - slots / 16 + units - 1) / units;
  const int by_tiles = 2 * max_tiles / 5 + 3, by_tiles_long = (max_tiles + 3) / 4 + 3;
  if (s > by_tiles) {
    s = by_tiles;
    const int64_t calm = 3 * simds / 4 / units, six_per_cu = 3 * simds / 2 / units;
    if (s > calm) s = calm > by_tiles_long ? calm : (s < six_per_cu ? s : six_per_cu);
  }
  if (per_sequence_counts && s < 12 && max_tiles >= 48) s = 12;
  if (s > 512) s = 512;
  return s < 1 ? 1 : (int)s;
}

namespace {

// events for the next split pass launched by this thread (kitty_profile_next_split)
thread_local hipEvent_t g_ev_start = nullptr, g_ev_stop = nullptr;

int check_layer(const kitty_kv_layer* layer, const void* q, int B, int H_Q, int* max_tiles) {
  KITTY_REQUIRE(layer && q, KITTY_E_NULL, "layer / q is NULL");
  const kitty_kv_layer& L = *layer;
  KITTY_REQUIRE(head_dim_supported(L.D) && L.PAGE_SIZE == kPage, KITTY_E_SHAPE,
                "kernels are built for head_dim 64, 128 or 256 and page_size 128, got D=%d page_size=%d", L.D,
                L.PAGE_SIZE);
  KITTY_REQUIRE(L.H_KV >= 1 && H_Q >= L.H_KV && H_Q % L.H_KV == 0, KITTY_E_SHAPE,
                "H_Q=%d must be a positive multiple of H_KV=%d", H_Q, L.H_KV);
  KITTY_REQUIRE(H_Q / L.H_KV <= 16, KITTY_E_SHAPE, "KV_GROUP (%d) exceeds MAX_KV_GROUP (16)", H_Q / L.H_KV);
  KITTY_REQUIRE(L.D_BOOSTED >= 0 && L.D_BOOSTED <= L.D && L.D_BOOSTED <= 255 &&
                    k_head_bytes_d(L.D, L.D_BOOSTED) % 16 == 0,
                KITTY_E_SHAPE, "unsupported D_BOOSTED=%d", L.D_BOOSTED);
  KITTY_REQUIRE(L.S >= 0 && L.S <= kPage && L.MAX_PAGE >= 0, KITTY_E_SHAPE, "S=%d must be in [0, 128]", L.S);
  KITTY_REQUIRE(B >= 1 && B <= 65535 && L.H_KV <= 65535, KITTY_E_RANGE, "bad batch size %d", B);
  KITTY_REQUIRE(L.key_cache && L.key_meta && L.value_cache && L.value_meta && L.page_table_k && L.page_table_v &&
                    L.sink_k && L.sink_v && L.qbuf_k && L.qbuf_v && L.local_v,
                KITTY_E_NULL, "a cache tensor pointer is NULL");
  KITTY_REQUIRE(((uintptr_t)L.key_cache % 16) == 0 && L.key_cache_stride_page % 16 == 0 &&
                    ((uintptr_t)L.value_cache % 16) == 0 && L.value_cache_stride_page % 16 == 0 &&
                    ((uintptr_t)L.key_meta % 16) == 0 && L.key_meta_stride_page % 16 == 0 &&
                    ((uintptr_t)L.value_meta % 16) == 0 && L.value_meta_stride_page % 16 == 0 &&
                    ((uintptr_t)L.sink_k % 16) == 0 && ((uintptr_t)L.sink_v % 16) == 0 &&
                    ((uintptr_t)L.qbuf_k % 16) == 0 && ((uintptr_t)L.qbuf_v % 16) == 0 &&
                    ((uintptr_t)L.local_v % 16) == 0 && L.sink_stride_b % 16 == 0 && L.sink_stride_h % 16 == 0 &&
                    L.win_stride_b % 16 == 0 && L.win_stride_h % 16 == 0 && ((uintptr_t)q % 16) == 0,
                KITTY_E_ALIGN, "cache tensors and q need 16-byte alignment");
  KITTY_REQUIRE(L.cache_pages_k <= INT32_MAX && L.cache_pages_v <= INT32_MAX, KITTY_E_RANGE,
                "cache_pages_k / cache_pages_v beyond 2^31 - 1 (page ids travel as 32-bit numbers inside the kernels)");
  KITTY_REQUIRE(L.cache_pages_k >= 0 && L.cache_pages_v >= 0 && ((uintptr_t)L.status % 4) == 0 &&
                    ((uintptr_t)L.seq_counts % 4) == 0,
                KITTY_E_RANGE, "negative cache_pages_k / cache_pages_v, or misaligned status / seq_counts");
  KITTY_REQUIRE(L.key_cache_stride_page >= (int64_t)L.H_KV * k_head_bytes_d(L.D, L.D_BOOSTED) &&
                    L.value_cache_stride_page >= (int64_t)L.H_KV * v_head_bytes_d(L.D) &&
                    L.key_meta_stride_page >= (int64_t)L.H_KV * L.D * 4 &&
                    L.value_meta_stride_page >= (int64_t)L.H_KV * kPage * 4,
                KITTY_E_RANGE, "a page stride is smaller than one page");
  *max_tiles = 2 + L.MAX_PAGE;
  if (!L.seq_counts) {
    const int* c = L.counts;
    KITTY_REQUIRE(c[KITTY_CNT_SINK] >= 0 && c[KITTY_CNT_SINK] <= L.S && c[KITTY_CNT_PAGES_K] >= 0 &&
                      c[KITTY_CNT_PAGES_K] <= L.MAX_PAGE && c[KITTY_CNT_PAGES_V] >= 0 &&
                      c[KITTY_CNT_PAGES_V] <= L.MAX_PAGE && c[KITTY_CNT_QBUF_K] >= 0 &&
                      c[KITTY_CNT_QBUF_K] <= kPage && c[KITTY_CNT_QBUF_V] >= 0 && c[KITTY_CNT_QBUF_V] <= kPage &&
                      c[KITTY_CNT_LOCAL_V] >= 0 && c[KITTY_CNT_LOCAL_V] <= kPage && c[KITTY_CNT_LOCAL_OFF] >= 0 &&
                      c[KITTY_CNT_LOCAL_OFF] < kPage,
                  KITTY_E_RANGE, "a cache counter is out of range");
    const int nk = c[KITTY_CNT_PAGES_K] * kPage + c[KITTY_CNT_QBUF_K];
    const int nv = c[KITTY_CNT_PAGES_V] * kPage + c[KITTY_CNT_QBUF_V] + c[KITTY_CNT_LOCAL_V];
    KITTY_REQUIRE(nk == nv, KITTY_E_RANGE, "seqlen_K: %d, seqlen_V: %d", nk + c[KITTY_CNT_SINK],
                  nv + c[KITTY_CNT_SINK]);
    KITTY_REQUIRE((c[KITTY_CNT_PAGES_K] == 0 || L.cache_pages_k > 0) && (c[KITTY_CNT_PAGES_V] == 0 || L.cache_pages_v > 0),
                  KITTY_E_RANGE, "the counters name packed pages but cache_pages_k / cache_pages_v is 0");
    *max_tiles = 1 + (nk + kPage - 1) / kPage;
  }
  return 0;
}

int check_workspace(const void* workspace, size_t workspace_bytes, int B, int H_Q, int num_splits, int D = kD) {
  KITTY_REQUIRE(workspace != nullptr, KITTY_E_NULL, "workspace is NULL");
  KITTY_REQUIRE(((uintptr_t)workspace % 256) == 0, KITTY_E_ALIGN, "workspace needs 256-byte alignment");
  KITTY_REQUIRE(num_splits >= 1 && num_splits <= 65535, KITTY_E_RANGE, "num_splits=%d out of range", num_splits);
  KITTY_REQUIRE(workspace_bytes >= ws_total_bytes(B, H_Q, num_splits, D), KITTY_E_WORKSPACE,
                "workspace of %zu bytes is smaller than the %zu needed for %d splits", workspace_bytes,
                ws_total_bytes(B, H_Q, num_splits, D), num_splits);
  return 0;
}

}  // namespace

namespace kitty {
// check_layer for other translation units: the argument checks of every attention entry point, and
// the tile count (1 + the 128-token tiles after the sink of the longest sequence) the default split
// rule is evaluated on.
int decode_check_layer(const kitty_kv_layer* layer, const void* q, int B, int H_Q, int* max_tiles) {
  return check_layer(layer, q, B, H_Q, max_tiles);
}
}  // namespace kitty

extern "C" int kitty_decode_attn_split(const kitty_kv_layer* layer, const void* q, int B, int H_Q, float scaling,
                                       void* workspace, size_t workspace_bytes, int num_splits, int variant,
                                       void* stream) {
  // armed events belong to THIS call, whether it launches or is rejected: taken and disarmed before
  // anything can return, so that they never ride on a later, unrelated launch of this thread
  const hipEvent_t ev0 = g_ev_start, ev1 = g_ev_stop;
  g_ev_start = g_ev_stop = nullptr;
  int max_tiles = 0;
  if (int rc = check_layer(layer, q, B, H_Q, &max_tiles)) return rc;
  if (int rc = check_workspace(workspace, workspace_bytes, B, H_Q, num_splits, layer->D)) return rc;
  KITTY_REQUIRE(variant == 0 || variant == 1, KITTY_E_SHAPE, "unknown variant %d", variant);
  const kitty_kv_layer& L = *layer;
  float* ws_ml = (float*)workspace;
  float* ws_acc = (float*)((uint8_t*)workspace + ws_ml_bytes(B, H_Q, num_splits));
  if (L.D != kD) {   // one kernel for both variants: the reference's order of operations on the vector ALUs
    if (ev0) (void)hipEventRecord(ev0, (hipStream_t)stream);
    launch_decode_any(L, q, B, H_Q, scaling, ws_ml, ws_acc, num_splits, (hipStream_t)stream);
    if (ev1) (void)hipEventRecord(ev1, (hipStream_t)stream);
  } else if (variant == 0 && decode_mfma_supported(L, H_Q)) {
    uint32_t* ws_plan = (uint32_t*)((uint8_t*)ws_acc + ws_acc_bytes(B, H_Q, num_splits));
    launch_decode_mfma(L, q, B, H_Q, scaling, ws_ml, ws_acc, ws_plan, num_splits, device_simds(), (hipStream_t)stream,
                       ev0, ev1);
  } else {
    if (ev0) (void)hipEventRecord(ev0, (hipStream_t)stream);
    launch_decode_plain(L, q, B, H_Q, scaling, ws_ml, ws_acc, num_splits, (hipStream_t)stream);
    if (ev1) (void)hipEventRecord(ev1, (hipStream_t)stream);
  }
  return check_launch("kitty_decode_attn_split");
}

extern "C" int kitty_profile_next_split(void* start_event, void* stop_event) {
  KITTY_REQUIRE((start_event == nullptr) == (stop_event == nullptr), KITTY_E_NULL, "two events, or none to cancel");
  g_ev_start = (hipEvent_t)start_event;
  g_ev_stop = (hipEvent_t)stop_event;
  return 0;
}

extern "C" int kitty_decode_attn_merge(const void* workspace, size_t workspace_bytes, int B, int H_Q, int D,
                                       int num_splits, void* out, void* stream) {
  KITTY_REQUIRE(out != nullptr, KITTY_E_NULL, "out is NULL");
  KITTY_REQUIRE(head_dim_supported(D) && B >= 1 && B <= 65535 && H_Q >= 1 && H_Q <= 65535, KITTY_E_SHAPE,
                "bad B=%d H_Q=%d D=%d", B, H_Q, D);
  KITTY_REQUIRE(((uintptr_t)out % 16) == 0, KITTY_E_ALIGN, "out needs 16-byte alignment");
  if (int rc = check_workspace(workspace, workspace_bytes, B, H_Q, num_splits, D)) return rc;
  const float* ws_ml = (const float*)workspace;
  const float* ws_acc = (const float*)((const uint8_t*)workspace + ws_ml_bytes(B, H_Q, num_splits));
  if (D != kD) launch_merge_any(D, ws_ml, ws_acc, out, B, H_Q, num_splits, (hipStream_t)stream);
  else launch_decode_merge(ws_ml, ws_acc, out, B, H_Q, num_splits, (hipStream_t)stream);
  return check_launch("kitty_decode_attn_merge");
}

extern "C" int kitty_decode_attn(const kitty_kv_layer* layer, const void* q, int B, int H_Q, float scaling,
                                 void* out, void* workspace, size_t workspace_bytes, int num_splits, int variant,
                                 void* stream) {
  int max_tiles = 0;
  if (int rc = check_layer(layer, q, B, H_Q, &max_tiles)) return rc;
  if (num_splits <= 0)
    num_splits = kitty_decode_attn_default_splits(B, layer->H_KV, max_tiles, layer->seq_counts != nullptr);
  if (int rc = kitty_decode_attn_split(layer, q, B, H_Q, scaling, workspace, workspace_bytes, num_splits, variant,
                                       stream))
    return rc;
  return kitty_decode_attn_merge(workspace, workspace_bytes, B, H_Q, layer->D, num_splits, out, stream);
}

extern "C" int kitty_prefill_attn(const kitty_kv_layer* layer, const void* q, int64_t q_stride_b,
                                  int64_t q_stride_h, int64_t q_stride_t, const void* k_new, const void* v_new,
                                  int64_t new_stride_b, int64_t new_stride_h, int64_t new_stride_t, int B, int H_Q,
                                  int T_q, float scaling, void* out, void* stream) {
  int max_tiles = 0;
  if (int rc = check_layer(layer, q, B, H_Q, &max_tiles)) return rc;
  KITTY_REQUIRE(k_new && v_new && out, KITTY_E_NULL, "k_new / v_new / out is NULL");
  KITTY_REQUIRE(T_q >= 1 && T_q <= (1 << 24), KITTY_E_RANGE, "T_q=%d out of range", T_q);
  KITTY_REQUIRE(layer->D_BOOSTED % 4 == 0, KITTY_E_SHAPE, "unsupported D_BOOSTED=%d", layer->D_BOOSTED);
  KITTY_REQUIRE(((uintptr_t)k_new % 16) == 0 && ((uintptr_t)v_new % 16) == 0 && ((uintptr_t)out % 16) == 0 &&
                    q_stride_b % 16 == 0 && q_stride_h % 16 == 0 && q_stride_t % 16 == 0 &&
                    new_stride_b % 16 == 0 && new_stride_h % 16 == 0 && new_stride_t % 16 == 0,
                KITTY_E_ALIGN, "q, k_new, v_new and out need 16-byte aligned bases and strides");
  KITTY_REQUIRE(q_stride_t >= layer->D * 2 && new_stride_t >= layer->D * 2, KITTY_E_ALIGN,
                "a token stride is smaller than one row of D fp16 values");
  if (layer->D != kD) {
    launch_prefill_any(*layer, q, q_stride_b, q_stride_h, q_stride_t, k_new, v_new, new_stride_b, new_stride_h,
                       new_stride_t, B, H_Q, T_q, scaling, out, (hipStream_t)stream);
    return check_launch("kitty_prefill_attn");
  }
  launch_prefill_attn(*layer, q, q_stride_b, q_stride_h, q_stride_t, k_new, v_new, new_stride_b, new_stride_h,
                      new_stride_t, B, H_Q, T_q, scaling, out, (hipStream_t)stream);
  return check_launch("kitty_prefill_attn");
}
