// Decode attention, matrix-core variant (placeholder until the kernel lands).
#include "decode_common.h"

namespace kitty {
bool decode_mfma_supported(const kitty_kv_layer&, int) { return false; }
void launch_decode_mfma(const kitty_kv_layer&, const void*, int, int, float, float*, float*, int, hipStream_t) {}
}  // namespace kitty
