// Scan-only kernels: h_t = a_t * h_{t-1} + z_t in fp32, and its reverse-mode derivative.
// Contract of griffin/triton_scan.py:207-271 (fp32 a, z, h0; da, dz, dh0 out), but time is cut
// into chunks of 32 steps that run on different waves and exchange carries through the
// publish / look-back protocol, so the launch fills the chip instead of B * W / 256 programs.
//
// One wave owns one (sequence, chunk, 64-channel group) tile.  A lane owns one channel: each
// load or store instruction of the wave touches 64 consecutive floats of one time step.

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <cstring>

#include "rglru_device.h"
#include "rglru_host.h"
#include "rglru_layout.h"

namespace rglru {

// ------------------------------------------------------------------------------------------
// host helpers (defined once, here)
// ------------------------------------------------------------------------------------------
char* error_buffer() {
  static thread_local char buf[512] = {0};
  return buf;
}

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(error_buffer(), 512, fmt, ap);
  va_end(ap);
  return code;
}

int num_compute_units() {
  static std::atomic<int> cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  int v = cached[dev].load(std::memory_order_relaxed);
  if (v == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cached[dev].store(n, std::memory_order_relaxed);
    v = n;
  }
  return v;
}

static std::atomic<long long> g_spin_limit{1ll << 22};
long long spin_limit() { return g_spin_limit.load(std::memory_order_relaxed); }
long long exchange_spin_limit(long long v) { return g_spin_limit.exchange(v); }

// ------------------------------------------------------------------------------------------
struct ScanArgs {
  const float* a; const float* z; const float* h0; float* h;      // forward
  const float* dh; const float* h_saved; float* da; float* dz; float* dh0;   // backward
  rec_t* rec_a; unsigned* ticket; unsigned* fail;
  int B, T, W, nC, groups;
  long long tiles, limit;
};

__global__ __launch_bounds__(kThreads) void scan_fwd_kernel(ScanArgs p) {
  const int lane = threadIdx.x & 63;
  // one ticket counter per chain (sequence x channel group): the waves bound to a chain take its
  // chunks in chain order
  const long long gw = (long long)blockIdx.x * kWaves + (threadIdx.x >> 6);
  if (gw >= p.tiles) return;
  const int chains = p.B * p.groups;
  const int chain_id = (int)(gw % chains);
  unsigned tk = 0;
  if (lane == 0) tk = atomicAdd(p.ticket + chain_id, 1u);
  tk = __builtin_amdgcn_readfirstlane(tk);
  const int c = (int)tk;
  const int b = chain_id / p.groups, grp = chain_id - b * p.groups;
  const int ch = grp * 64 + lane;
  const bool ok = ch < p.W;
  const int t0 = c * kChunk;
  const long long W = p.W;

  float a[kChunk], z[kChunk];
  const long long base = ((long long)b * p.T + t0) * W + ch;
#pragma unroll
  for (int e = 0; e < kChunk; ++e) {
    bool in = ok && (t0 + e < p.T);
    a[e] = in ? p.a[base + e * W] : 1.f;
    z[e] = in ? p.z[base + e * W] : 0.f;
  }
  float A = 1.f, H = 0.f;
#pragma unroll
  for (int e = 0; e < kChunk; ++e) { H = fmaf(a[e], H, z[e]); A *= a[e]; }

  CarryChain chain;
  const long long seq = (long long)b * p.nC * W + (ok ? ch : 0);
  chain.rec = p.rec_a + seq; chain.stride = W;

  float h_in;
  if (c == 0) {
    h_in = ok ? p.h0[(long long)b * W + ch] : 0.f;
  } else {
    if (ok) carry_publish(chain, c, A, H, false);
    h_in = carry_lookback(chain, c, -1, -1, 0.f, ok, p.limit, p.fail);
  }
  if (ok) carry_publish(chain, c, 0.f, fmaf(A, h_in, H), true);

  float h = h_in;
#pragma unroll
  for (int e = 0; e < kChunk; ++e) {
    h = fmaf(a[e], h, z[e]);
    if (ok && (t0 + e < p.T)) p.h[base + e * W] = h;
  }
}

__global__ __launch_bounds__(kThreads) void scan_bwd_kernel(ScanArgs p) {
  const int lane = threadIdx.x & 63;
  const long long gw = (long long)blockIdx.x * kWaves + (threadIdx.x >> 6);
  if (gw >= p.tiles) return;
  const int chains = p.B * p.groups;
  const int chain_id = (int)(gw % chains);
  unsigned tk = 0;
  if (lane == 0) tk = atomicAdd(p.ticket + chain_id, 1u);
  tk = __builtin_amdgcn_readfirstlane(tk);
  const int c = p.nC - 1 - (int)tk;                  // the chain runs from the last chunk to the first
  const int b = chain_id / p.groups, grp = chain_id - b * p.groups;
  const int ch = grp * 64 + lane;
  const bool ok = ch < p.W;
  const int t0 = c * kChunk;
  const long long W = p.W;

  float a[kChunk], g[kChunk], hp[kChunk];
  const long long base = ((long long)b * p.T + t0) * W + ch;
#pragma unroll
  for (int e = 0; e < kChunk; ++e) {
    const int t = t0 + e;
    bool in = ok && (t < p.T);
    a[e] = in ? p.a[base + e * W] : 1.f;
    g[e] = in ? p.dh[base + e * W] : 0.f;
    hp[e] = in ? (t == 0 ? p.h0[(long long)b * W + ch] : p.h_saved[base + (e - 1) * W]) : 0.f;
  }
  float A = 1.f, carry = 0.f;
#pragma unroll
  for (int e = kChunk - 1; e >= 0; --e) { float d = g[e] + carry; carry = a[e] * d; A *= a[e]; }
  const float H = carry;

  CarryChain chain;
  const long long seq = (long long)b * p.nC * W + (ok ? ch : 0);
  chain.rec = p.rec_a + seq; chain.stride = W;

  float d_in;
  if (c == p.nC - 1) {
    d_in = 0.f;
  } else {
    if (ok) carry_publish(chain, c, A, H, false);
    d_in = carry_lookback(chain, c, +1, p.nC, 0.f, ok, p.limit, p.fail);
  }
  const float d_out = fmaf(A, d_in, H);
  if (ok) carry_publish(chain, c, 0.f, d_out, true);
  if (c == 0 && ok) p.dh0[(long long)b * W + ch] = d_out;

  carry = d_in;
#pragma unroll
  for (int e = kChunk - 1; e >= 0; --e) {
    float d = g[e] + carry;
    carry = a[e] * d;
    if (ok && (t0 + e < p.T)) {
      p.dz[base + e * W] = d;
      p.da[base + e * W] = d * hp[e];
    }
  }
}

static int scan_common(ScanArgs& p, void* ws, int64_t B, int64_t T, int64_t W, hipStream_t s) {
  if (B <= 0 || T <= 0 || W <= 0) return fail(RGLRU_E_ARG, "scan: B, T, W must be positive (got %lld, %lld, %lld)", (long long)B, (long long)T, (long long)W);
  if (!ws) return fail(RGLRU_E_ARG, "scan: workspace pointer is null");
  if (B * T * W >= (1ll << 40)) return fail(RGLRU_E_UNSUPPORTED, "scan: tensor too large");
  ScanLayout L = make_scan_layout(B, T, W);
  if (B * L.nC * L.groups >= (1ll << 31)) return fail(RGLRU_E_UNSUPPORTED, "scan: too many tiles");
  char* base = (char*)ws;
  p.rec_a = (rec_t*)(base + L.rec_a);
  p.ticket = (unsigned*)(base + L.ticket); p.fail = (unsigned*)(base + L.fail);
  p.B = (int)B; p.T = (int)T; p.W = (int)W; p.nC = (int)L.nC; p.groups = (int)L.groups;
  p.tiles = B * L.nC * L.groups;
  p.limit = spin_limit();
  long long words = (long long)L.total / 4;
  int cb = (int)((words + 1023) / 1024); if (cb > 2048) cb = 2048;
  hipLaunchKernelGGL(clear_words_kernel, dim3(cb), dim3(256), 0, s, (unsigned*)base, words);
  return check_launch("scan workspace clear");
}

}  // namespace rglru

using namespace rglru;

extern "C" {

int rglru_hip_abi_version(void) { return RGLRU_ABI_VERSION; }
const char* rglru_hip_last_error(void) { return error_buffer(); }

int64_t rglru_hip_set_spin_limit(int64_t polls) {
  if (polls < 1) polls = 1;
  return (int64_t)g_spin_limit.exchange((long long)polls);
}

size_t rglru_hip_scan_workspace_bytes(int64_t B, int64_t T, int64_t W) {
  if (B <= 0 || T <= 0 || W <= 0) return 0;
  return make_scan_layout(B, T, W).total;
}

int rglru_hip_scan_fwd(const float* a, const float* z, const float* h0, float* h, void* ws,
                       int64_t B, int64_t T, int64_t W, void* stream) {
  if (!a || !z || !h0 || !h) return fail(RGLRU_E_ARG, "scan_fwd: null tensor pointer");
  ScanArgs p;
  memset(&p, 0, sizeof(p));
  hipStream_t s = (hipStream_t)stream;
  int rc = scan_common(p, ws, B, T, W, s);
  if (rc) return rc;
  p.a = a; p.z = z; p.h0 = h0; p.h = h;
  unsigned blocks = (unsigned)((p.tiles + kWaves - 1) / kWaves);
  hipLaunchKernelGGL(scan_fwd_kernel, dim3(blocks), dim3(kThreads), 0, s, p);
  return check_launch("scan_fwd");
}

int rglru_hip_scan_bwd(const float* a, const float* h0, const float* h, const float* dh,
                       float* da, float* dz, float* dh0, void* ws,
                       int64_t B, int64_t T, int64_t W, void* stream) {
  if (!a || !h0 || !h || !dh || !da || !dz || !dh0) return fail(RGLRU_E_ARG, "scan_bwd: null tensor pointer");
  ScanArgs p;
  memset(&p, 0, sizeof(p));
  hipStream_t s = (hipStream_t)stream;
  int rc = scan_common(p, ws, B, T, W, s);
  if (rc) return rc;
  p.a = a; p.h0 = h0; p.h_saved = h; p.dh = dh; p.da = da; p.dz = dz; p.dh0 = dh0;
  unsigned blocks = (unsigned)((p.tiles + kWaves - 1) / kWaves);
  hipLaunchKernelGGL(scan_bwd_kernel, dim3(blocks), dim3(kThreads), 0, s, p);
  return check_launch("scan_bwd");
}

}  // extern "C"
