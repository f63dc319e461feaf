// Host-side plumbing shared by every entry point: thread-local error text, launch
// check, descriptor validation and layout classification.
#include "common.h"

#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <algorithm>
#include <mutex>

namespace mi355 {

static thread_local char g_error[512] = "";

int set_error(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

static Knobs g_knobs;
static std::once_flag g_knobs_once;

static void copy_knob(char* dst, size_t cap, const char* src) {
  if (src == nullptr) src = "";
  strncpy(dst, src, cap - 1);
  dst[cap - 1] = 0;
}

static void knobs_from_env() {
  copy_knob(g_knobs.gemm_tile, sizeof(g_knobs.gemm_tile), getenv("MI355_GEMM_TILE"));
  copy_knob(g_knobs.gemm_waves, sizeof(g_knobs.gemm_waves), getenv("MI355_GEMM_WAVES"));
  g_knobs.x16_spin_limit = kX16SpinLimitDefault;
  g_knobs.gemm_prefetch = -1;
}

const Knobs& knobs() {
  std::call_once(g_knobs_once, knobs_from_env);
  return g_knobs;
}

int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess)
    return set_error(MI355_ERR_LAUNCH, "%s: launch failed: %s", what, hipGetErrorString(e));
  return MI355_OK;
}

int check_tensor(const mi355_tensor* t, const char* op, const char* name) {
  if (t == nullptr) return set_error(MI355_ERR_INVALID, "%s: %s is NULL", op, name);
  if (t->ndim < 0 || t->ndim > MI355_MAX_DIMS)
    return set_error(MI355_ERR_INVALID, "%s: %s has ndim %d (max %d)", op, name, t->ndim,
                     MI355_MAX_DIMS);
  if (t->dtype < 0 || t->dtype >= MI355_DTYPE_COUNT)
    return set_error(MI355_ERR_INVALID, "%s: %s has unknown dtype %d", op, name, t->dtype);
  int64_t n = 1;
  for (int i = 0; i < t->ndim; ++i) {
    if (t->sizes[i] < 0)
      return set_error(MI355_ERR_INVALID, "%s: %s has negative size at dim %d", op, name, i);
    n *= t->sizes[i];
  }
  if (n > 0 && t->data == nullptr)
    return set_error(MI355_ERR_INVALID, "%s: %s has a NULL data pointer", op, name);
  return MI355_OK;
}

bool same_dense_layout(const mi355_tensor* const* ts, int nt) {
  const mi355_tensor* t0 = ts[0];
  for (int t = 1; t < nt; ++t) {
    if (!same_shape(t0, ts[t])) return false;
    for (int i = 0; i < t0->ndim; ++i)
      if (t0->sizes[i] != 1 && t0->strides[i] != ts[t]->strides[i]) return false;
  }
  // Sort dims by stride; dense iff each stride equals the product of the smaller sizes.
  int order[MI355_MAX_DIMS];
  int nd = 0;
  for (int i = 0; i < t0->ndim; ++i)
    if (t0->sizes[i] != 1) order[nd++] = i;
  std::sort(order, order + nd, [&](int a, int b) { return t0->strides[a] < t0->strides[b]; });
  int64_t expect = 1;
  for (int k = 0; k < nd; ++k) {
    if (t0->strides[order[k]] != expect) return false;
    expect *= t0->sizes[order[k]];
  }
  return true;
}

}  // namespace mi355

extern "C" int mi355_abi_version(void) { return MI355_ABI_VERSION; }

extern "C" int mi355_set_knob(const char* name, const char* value) {
  using namespace mi355;
  knobs();  // the environment first, so that a later call cannot overwrite this one
  if (name == nullptr) return set_error(MI355_ERR_INVALID, "mi355_set_knob: name is NULL");
  if (strcmp(name, "gemm_tile") == 0) {
    copy_knob(g_knobs.gemm_tile, sizeof(g_knobs.gemm_tile), value);
  } else if (strcmp(name, "gemm_waves") == 0) {
    copy_knob(g_knobs.gemm_waves, sizeof(g_knobs.gemm_waves), value);
  } else if (strcmp(name, "gemm_split") == 0) {
    copy_knob(g_knobs.gemm_split, sizeof(g_knobs.gemm_split), value);
  } else if (strcmp(name, "x16_spin_limit") == 0) {
    const long v = (value == nullptr || value[0] == 0) ? kX16SpinLimitDefault : strtol(value, nullptr, 10);
    if (v < 0 || v > (1L << 30)) return set_error(MI355_ERR_INVALID, "mi355_set_knob: x16_spin_limit %ld out of range", v);
    g_knobs.x16_spin_limit = (int)v;
  } else if (strcmp(name, "gemm_prefetch") == 0) {
    const long v = (value == nullptr || value[0] == 0) ? -1 : strtol(value, nullptr, 10);
    if (v < -1 || v > kNumCU) return set_error(MI355_ERR_INVALID, "mi355_set_knob: gemm_prefetch %ld out of range", v);
    g_knobs.gemm_prefetch = (int)v;
  } else {
    return set_error(MI355_ERR_INVALID, "mi355_set_knob: unknown knob '%s'", name);
  }
  return MI355_OK;
}

// Defined next to the state they cover.  (The GEMM-only measurement builds - MI355_GEMM_ONLY - hold no reduce.hip.)
namespace mi355 {
#ifndef MI355_GEMM_ONLY
int reduce_static_init();   // reduce.hip: address of the built-in scratch array on the current device
#else
static int reduce_static_init() { return MI355_OK; }
#endif
}

extern "C" int mi355_init(void) {
  using namespace mi355;
  knobs();
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return set_error(MI355_ERR_LAUNCH, "mi355_init: hipGetDevice failed: %s", hipGetErrorString(e));
  hipDeviceProp_t prop;
  e = hipGetDeviceProperties(&prop, dev);
  if (e != hipSuccess) return set_error(MI355_ERR_LAUNCH, "mi355_init: hipGetDeviceProperties failed: %s", hipGetErrorString(e));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return set_error(MI355_ERR_UNSUPPORTED, "mi355_init: device %d is %s; this library holds gfx950 code only", dev, prop.gcnArchName);
  // The persistent and split-K grids, the tile planner and the streaming kernels' grids are sized for
  // this many CUs; a partitioned or cut-down part would run them with idle or oversubscribed CUs.
  if (prop.multiProcessorCount != kNumCU)
    return set_error(MI355_ERR_UNSUPPORTED, "mi355_init: device %d has %d compute units, the launch heuristics are built for %d",
                     dev, prop.multiProcessorCount, kNumCU);
  return reduce_static_init();
}
extern "C" const char* mi355_last_error(void) { return mi355::g_error; }
