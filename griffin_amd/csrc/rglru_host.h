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

// Zero `n` 32-bit words starting at a 16-byte aligned address (n a multiple of 4).
static __global__ void clear_words_kernel(unsigned* p, long long n) {
  uint4* q = reinterpret_cast<uint4*>(p);
  const long long n4 = n >> 2;
  long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x;
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (; i < n4; i += stride) q[i] = make_uint4(0u, 0u, 0u, 0u);
}

inline int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(RGLRU_E_LAUNCH, "%s: %s", what, hipGetErrorString(e));
  return RGLRU_OK;
}

}  // namespace rglru
