// TEST INFRASTRUCTURE: entry points of the one translation unit that is not part of the emulation build (the stream-K
// form, whose prefetch ring is inline assembly), as far as the staged sources refer to them.
#include <hip/hip_runtime.h>

#include "../../include/bgmoe.h"

// the balanced (stream-K) form is not emulated: "does not apply", the caller launches the plain form
int bgmoe_internal_fp8_streamk(const bgmoe_fp8_act*, const bgmoe_fp8_weight*, const bgmoe_fp8_weight*, const int32_t*,
                               const int32_t*, int, int, int, uint16_t*, uint8_t*, float*, int64_t, int64_t, int, int64_t,
                               void*, size_t, hipStream_t) {
  return BGMOE_ERR_WORKSPACE;
}

#include "bgmoe_common.h"

int bgmoe_internal_init_fp8_streamk() { return BGMOE_OK; }
