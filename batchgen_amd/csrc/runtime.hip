// Error reporting and small host utilities of libbgmoe.
#include <stdarg.h>
#include <stdio.h>

#include "bgmoe_common.h"

static thread_local char g_err[512] = "";

void bgmoe_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

int bgmoe_check_launch(const char* what) {
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) {
    bgmoe_set_error("%s: %s", what, hipGetErrorString(err));
    return BGMOE_ERR_HIP;
  }
  return BGMOE_OK;
}

extern "C" const char* bgmoe_last_error(void) { return g_err; }
extern "C" int bgmoe_version(void) { return 1; }

extern "C" int bgmoe_init(void) {
  int rc = bgmoe_internal_init_fp8_skinny();
  if (rc == BGMOE_OK) rc = bgmoe_internal_init_fp8_streamk();
  if (rc == BGMOE_OK) rc = bgmoe_internal_init_fp8_tiled();
  if (rc == BGMOE_OK) rc = bgmoe_internal_init_mxfp4();
  if (rc == BGMOE_OK) rc = bgmoe_internal_init_router_gemm();
  if (rc == BGMOE_OK) rc = bgmoe_internal_init_permute();
  return rc;
}

// ---- per-launch timing ------------------------------------------------------------
// When enabled, every kernel launch of the library is bracketed by a pair of HIP
// events on its own stream.  bgmoe_prof_collect() synchronises, sums the elapsed
// time per kernel id and clears the records.  Meant for benchmarks: the events
// serialise nothing, but a run with timing on should not be used for end-to-end
// numbers.
#include <vector>

bool g_bgmoe_prof_on = false;

namespace {
struct ProfRec { int id; hipEvent_t a, b; };
std::vector<ProfRec> g_recs;
std::vector<hipEvent_t> g_free;
hipEvent_t g_pending = nullptr;
const char* kNames[BGMOE_K_COUNT] = {
    "router", "perm_hist", "perm_scan", "perm_rank", "gather_rows", "act_quant", "combine", "compact",
    "s1_skinny16", "s1_skinny64", "s1_tiled", "gemm_skinny16", "gemm_skinny64", "gemm_tiled",
    "mxfp4_s1", "mxfp4_gemm", "bf16_gemm", "router_gemm", "router_gemm_reduce", "norm_quant", "situ_and_mul", "fp8_dense_gemm"};
hipEvent_t take_event() {
  if (!g_free.empty()) { hipEvent_t e = g_free.back(); g_free.pop_back(); return e; }
  hipEvent_t e = nullptr;
  (void)hipEventCreate(&e);
  return e;
}
}  // namespace

void bgmoe_prof_mark(int id, hipStream_t st, bool begin) {
  if (begin) {
    g_pending = take_event();
    (void)hipEventRecord(g_pending, st);
  } else {
    hipEvent_t b = take_event();
    (void)hipEventRecord(b, st);
    g_recs.push_back(ProfRec{id, g_pending, b});
    g_pending = nullptr;
  }
}

extern "C" int bgmoe_prof_enable(int on) {
  g_bgmoe_prof_on = on != 0;
  return BGMOE_OK;
}

extern "C" int bgmoe_prof_kernel_count(void) { return BGMOE_K_COUNT; }
extern "C" const char* bgmoe_prof_kernel_name(int id) { return (id >= 0 && id < BGMOE_K_COUNT) ? kNames[id] : ""; }

extern "C" int bgmoe_prof_collect(double* total_ms, int64_t* launches, int n) {
  if (hipDeviceSynchronize() != hipSuccess) {
    bgmoe_set_error("prof_collect: device synchronisation failed");
    return BGMOE_ERR_HIP;
  }
  for (int i = 0; i < n; ++i) { total_ms[i] = 0.0; launches[i] = 0; }
  for (const ProfRec& r : g_recs) {
    float ms = 0.0f;
    if (hipEventElapsedTime(&ms, r.a, r.b) == hipSuccess && r.id < n) {
      total_ms[r.id] += ms;
      launches[r.id] += 1;
    }
    g_free.push_back(r.a);
    g_free.push_back(r.b);
  }
  g_recs.clear();
  return BGMOE_OK;
}
