// TEST INFRASTRUCTURE: entry points of translation units that are not part of the emulation build, as far as the
// staged sources refer to them.
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

extern "C" int bgmoe_version(void) { return 1; }
extern "C" int bgmoe_init(void) {
  int rc = bgmoe_internal_init_fp8_skinny();
  if (rc == BGMOE_OK) rc = bgmoe_internal_init_fp8_tiled();
  if (rc == BGMOE_OK) rc = bgmoe_internal_init_mxfp4();
  if (rc == BGMOE_OK) rc = bgmoe_internal_init_router_gemm();
  if (rc == BGMOE_OK) rc = bgmoe_internal_init_permute();
  return rc;
}
