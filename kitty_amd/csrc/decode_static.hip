// kitty_decode_attn_static: decode attention whose split-K partials live in an array that is part
// of the library's own device image, for callers that cannot allocate (code under HIP graph
// capture, serving loops and harnesses that forbid hipMalloc).  It runs the kernels of
// kitty_decode_attn; only the home of the partials differs.
#include <mutex>

#include "decode_common.h"

namespace kitty {
int decode_check_layer(const kitty_kv_layer* layer, const void* q, int B, int H_Q, int* max_tiles);
}
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
int scratch_of_current_device(void** out, hipStream_t stream) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return set_error((int)e, "kitty_decode_attn_static: hipGetDevice: %s", hipGetErrorString(e));
  KITTY_REQUIRE(dev >= 0 && dev < kMaxDevices, KITTY_E_RANGE, "device ordinal %d outside [0, %d)", dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(g_mutex);
  if (!g_scratch_of_device[dev]) {
    // The runtime call that resolves the address is not one a stream capture may contain: the first
    // call on a device has to come before the capture (any call, e.g. the eager warm-up run that a
    // capture follows anyway).  Said here rather than found out from a broken capture.
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &cap) == hipSuccess && cap != hipStreamCaptureStatusNone)
      return set_error(KITTY_E_RANGE,
                       "kitty_decode_attn_static: the first call on a device resolves the address of the library's "
                       "array and cannot be part of a stream capture; call it once on device %d before capturing", dev);
    (void)hipGetLastError();
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
  KITTY_REQUIRE(out != nullptr, KITTY_E_NULL, "out is NULL");
  // the checks, and the tile count behind the default split rule, are kitty_decode_attn's own
  int max_tiles = 0;
  if (int rc = decode_check_layer(layer, q, B, H_Q, &max_tiles)) return rc;
  const size_t per_split = ws_total_bytes(B, H_Q, 1, layer->D) + 768;   // an upper bound of the growth per split
  if (num_splits <= 0) {
    // the default of kitty_decode_attn, cut back to what the array holds
    num_splits = kitty_decode_attn_default_splits(B, layer->H_KV, max_tiles, layer->seq_counts != nullptr);
    const size_t fit = KITTY_STATIC_WORKSPACE_BYTES / per_split;
    if ((size_t)num_splits > fit) num_splits = (int)fit;
    KITTY_REQUIRE(num_splits >= 1, KITTY_E_WORKSPACE,
                  "B=%d x H_Q=%d query heads need %zu bytes of partials per split, the library's array holds %zu", B,
                  H_Q, ws_total_bytes(B, H_Q, 1, layer->D), (size_t)KITTY_STATIC_WORKSPACE_BYTES);
  }
  KITTY_REQUIRE(num_splits <= 65535 && ws_total_bytes(B, H_Q, num_splits, layer->D) <= KITTY_STATIC_WORKSPACE_BYTES,
                KITTY_E_WORKSPACE,
                "%d splits of B=%d x H_Q=%d query heads need %zu bytes of partials, the library's array holds %zu: "
                "ask for fewer splits or use kitty_decode_attn with a workspace of your own",
                num_splits, B, H_Q, ws_total_bytes(B, H_Q, num_splits, layer->D), (size_t)KITTY_STATIC_WORKSPACE_BYTES);
  void* ws = nullptr;
  if (int rc = scratch_of_current_device(&ws, (hipStream_t)stream)) return rc;
  return kitty_decode_attn(layer, q, B, H_Q, scaling, out, ws, KITTY_STATIC_WORKSPACE_BYTES, num_splits, variant, stream);
}
