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

struct Geometry;
// The block-diagonal GEMMs of the gate projections and their gradients (rglru_gate_gemm.hip).
int gate_dw_splits(long long N, const Geometry& g);
int launch_gate_pre_gemm(const void* x, const void* wg, void* pre, long long N, const Geometry& g, hipStream_t s);
int launch_gate_gemms(const void* x, const void* du_a, const void* du_x, long long du_ld, long long du_blk,
                      const void* w2t, void* dx, float* dw_partial, long long N, const Geometry& g, int dtype,
                      int n_split, hipStream_t s);

// The same for two ranges in one launch.
static __global__ void clear_two_kernel(unsigned* p0, long long n0, unsigned* p1, long long n1) {
  long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x;
  const long long stride = (long long)gridDim.x * blockDim.x;
  const long long a = n0 >> 2, b = n1 >> 2;
  for (; i < a + b; i += stride) {
    if (i < a) reinterpret_cast<uint4*>(p0)[i] = make_uint4(0u, 0u, 0u, 0u);
    else reinterpret_cast<uint4*>(p1)[i - a] = make_uint4(0u, 0u, 0u, 0u);
  }
}

inline int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(RGLRU_E_LAUNCH, "%s: %s", what, hipGetErrorString(e));
  return RGLRU_OK;
}

}  // namespace rglru
