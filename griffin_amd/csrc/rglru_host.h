// Host-side helpers shared by the C-ABI translation units: error text, device facts, checks.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>
#include <cstdarg>
#include <cstdio>

#include "../../include/rglru_hip.h"

namespace rglru {

char* error_buffer();                       // thread-local, 512 bytes
int fail(int code, const char* fmt, ...);   // formats into error_buffer(), returns code
int num_compute_units();                    // of the current device (cached per device)
long long spin_limit();

static __global__ void clear_words_kernel(unsigned* p, long long n) {
  long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x;
  long long stride = (long long)gridDim.x * blockDim.x;
  for (; i < n; i += stride) p[i] = 0u;
}

inline int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(RGLRU_E_LAUNCH, "%s: %s", what, hipGetErrorString(e));
  return RGLRU_OK;
}

}  // namespace rglru
