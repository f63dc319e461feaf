// Host-side plumbing shared by every entry point: thread-local error text, launch
// check, descriptor validation and layout classification.
#include "common.h"

#include <stdarg.h>
#include <stdio.h>
#include <algorithm>

namespace mi355 {

static thread_local char g_error[512] = "";

int set_error(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
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
extern "C" const char* mi355_last_error(void) { return mi355::g_error; }
