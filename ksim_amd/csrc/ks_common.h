// Shared host-side helpers for the C ABI (error text, launch checks).
#pragma once
#include <hip/hip_runtime.h>
#include <cstdarg>
#include <cstdio>
#include "../../include/ksim_hip.h"

namespace ks {

char* err_buf();  // thread-local, 256 bytes

inline int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(err_buf(), 256, fmt, ap);
  va_end(ap);
  return code;
}

inline int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(KS_ELAUNCH, "%s: %s", what, hipGetErrorString(e));
  return KS_OK;
}

constexpr int kWave = 64;

// defined beside the MLP handle: weight matrix (npad, kpad) of layer l in working precision and its transpose (after train_init)
int mlp_peek_layer(const KsMlp* h, int l, const void** W, const void** Wt, int* npad, int* kpad, int* dtype);

}  // namespace ks
