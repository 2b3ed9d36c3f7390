// kitty_decode_attn_static: decode attention whose split-K partials live in an array that is part
// of the library's own device image, for callers that cannot allocate (code under HIP graph
// capture, serving loops and harnesses that forbid hipMalloc).  It runs the kernels of
// kitty_decode_attn; only the home of the partials differs.
#include <mutex>

#include "decode_common.h"

using namespace kitty;

// Split-K partials of one call: [B * H_Q * splits] x (2 + 128) floats.  16 MiB hold the default
// split counts of batch 16 at 32k tokens (4.3 MB), batch 64 ragged (12.8 MB) and one 128k sequence
// with 64 query heads (8 MB).  Every device the library runs on holds its own copy at its own
// address until the process ends.
static __device__ __align__(256) uint8_t scratch[KITTY_STATIC_WORKSPACE_BYTES];

namespace {

constexpr int kMaxDevices = 64;
std::mutex g_mutex;
void* g_scratch_of_device[kMaxDevices];   // the array's address on each device, asked once

// `scratch` itself is only a host-side handle: the device address comes from the runtime.
int scratch_of_current_device(void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return set_error((int)e, "kitty_decode_attn_static: hipGetDevice: %s", hipGetErrorString(e));
  KITTY_REQUIRE(dev >= 0 && dev < kMaxDevices, KITTY_E_RANGE, "device ordinal %d outside [0, %d)", dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(g_mutex);
  if (!g_scratch_of_device[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p)
      return set_error(e != hipSuccess ? (int)e : KITTY_E_NULL, "kitty_decode_attn_static: hipGetSymbolAddress: %s",
                       hipGetErrorString(e));
    g_scratch_of_device[dev] = p;
  }
  *out = g_scratch_of_device[dev];
  return 0;
}

}  // namespace

extern "C" int kitty_decode_attn_static(const kitty_kv_layer* layer, const void* q, int B, int H_Q, float scaling,
                                        void* out, int num_splits, int variant, void* stream) {
  KITTY_REQUIRE(layer && q && out, KITTY_E_NULL, "layer / q / out is NULL");
  KITTY_REQUIRE(B >= 1 && H_Q >= 1 && layer->H_KV >= 1, KITTY_E_RANGE, "bad B=%d, H_Q=%d or H_KV=%d", B, H_Q, layer->H_KV);
  const size_t per_split = ws_total_bytes(B, H_Q, 1) + 768;   // an upper bound of the growth per split
  if (num_splits <= 0) {
    // the default of kitty_decode_attn, cut back to what the array holds
    int max_tiles = 2 + layer->MAX_PAGE;
    if (!layer->seq_counts) {
      const int* c = layer->counts;
      max_tiles = 1 + (c[KITTY_CNT_PAGES_K] * kPage + c[KITTY_CNT_QBUF_K] + kPage - 1) / kPage;
    }
    num_splits = kitty_decode_attn_default_splits(B, layer->H_KV, max_tiles, layer->seq_counts != nullptr);
    const size_t fit = KITTY_STATIC_WORKSPACE_BYTES / per_split;
    if ((size_t)num_splits > fit) num_splits = (int)fit;
    KITTY_REQUIRE(num_splits >= 1, KITTY_E_WORKSPACE,
                  "B=%d x H_Q=%d query heads need %zu bytes of partials per split, the library's array holds %zu", B,
                  H_Q, ws_total_bytes(B, H_Q, 1), (size_t)KITTY_STATIC_WORKSPACE_BYTES);
  }
  KITTY_REQUIRE(num_splits <= 65535 && ws_total_bytes(B, H_Q, num_splits) <= KITTY_STATIC_WORKSPACE_BYTES,
                KITTY_E_WORKSPACE,
                "%d splits of B=%d x H_Q=%d query heads need %zu bytes of partials, the library's array holds %zu: "
                "ask for fewer splits or use kitty_decode_attn with a workspace of your own",
                num_splits, B, H_Q, ws_total_bytes(B, H_Q, num_splits), (size_t)KITTY_STATIC_WORKSPACE_BYTES);
  void* ws = nullptr;
  if (int rc = scratch_of_current_device(&ws)) return rc;
  return kitty_decode_attn(layer, q, B, H_Q, scaling, out, ws, KITTY_STATIC_WORKSPACE_BYTES, num_splits, variant, stream);
}
