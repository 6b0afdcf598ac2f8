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
static std::atomic<int> g_reproducible{0};
// what the kernels get as `limit`: negative selects the look-back that accepts final records only
long long spin_limit() {
  const long long polls = g_spin_limit.load(std::memory_order_relaxed);
  return g_reproducible.load(std::memory_order_relaxed) ? -polls : polls;
}
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

// ------------------------------------------------------------------------------------------
// Vector variant (rows 16-byte aligned, width a multiple of 4): a lane owns four consecutive
// channels and moves 16 bytes per access; a wave owns kVecTokens consecutive tokens of 256 channels
// and a workgroup of kVecWaves waves a run of kVecWaves * kVecTokens tokens of one sequence.  The
// waves of a workgroup exchange their maps through LDS (one barrier), so only one carry per run and
// channel crosses workgroups: four times fewer records, tickets and look-backs than one wave per
// 32-token chunk, and every wave has its whole tile in flight before anything is computed.  Measured
// at B8 T2048 W1024 (forward / forward + backward, eager): 8 waves x 16 tokens 47 / 119 us, 16 x 8
// 49 / 123 us, 8 x 8 58 / 141 us, 4 x 8 80 / 178 us; one wave per 32-token chunk and scalar accesses
// took 57 / 148 us.
// ------------------------------------------------------------------------------------------
constexpr int kVecTokens = 16;
constexpr int kVecWaves = 8;
constexpr int kVecRun = kVecTokens * kVecWaves;          // tokens per workgroup
constexpr int kVecThreads = 64 * kVecWaves;

struct Map4 { float4 a, h; };

RGLRU_DEVICE float4 fma4(float4 a, float4 b, float4 c) {
  return make_float4(fmaf(a.x, b.x, c.x), fmaf(a.y, b.y, c.y), fmaf(a.z, b.z, c.z), fmaf(a.w, b.w, c.w));
}
RGLRU_DEVICE float4 mul4(float4 a, float4 b) { return make_float4(a.x * b.x, a.y * b.y, a.z * b.z, a.w * b.w); }

// carry_in of run `c` for the lane's four channels (records at rec + q * stride + 0..3), walking
// `step` from run c until a final record or the boundary (where the carry is `boundary`).  A run
// publishes its four records back to back; a reader treats them as published only when all four are.
RGLRU_DEVICE float4 carry_lookback4(const rec_t* rec, long long stride, int c, int step, int end, float4 boundary,
                                    bool lane_ok, long long limit, unsigned* fail_word) {
  float acc_a[4] = {1.f, 1.f, 1.f, 1.f}, acc_h[4] = {0.f, 0.f, 0.f, 0.f};
  const float bnd[4] = {boundary.x, boundary.y, boundary.z, boundary.w};
  bool done = !lane_ok;
  int q = c + step;
  long long polls = 0;
  const bool finals_only = limit < 0;                    // see carry_compose
  if (finals_only) limit = -limit;
  while (!__all(done)) {
    if (q == end) {                                      // wave-uniform
      if (!done) {
#pragma unroll
        for (int i = 0; i < 4; ++i) { acc_h[i] = fmaf(acc_a[i], bnd[i], acc_h[i]); acc_a[i] = 0.f; }
        done = true;
      }
      break;
    }
    rec_t r[4] = {0, 0, 0, 0};
    if (!done) {
#pragma unroll
      for (int i = 0; i < 4; ++i) r[i] = rec_load(rec + (long long)q * stride + i);
    }
    const bool ready = done || (finals_only ? ((unsigned)r[0] == 1u && (unsigned)r[1] == 1u && (unsigned)r[2] == 1u && (unsigned)r[3] == 1u)
                                            : ((unsigned)r[0] != 0u && (unsigned)r[1] != 0u && (unsigned)r[2] != 0u && (unsigned)r[3] != 0u));
    if (!__all(ready)) {
      if (++polls > limit) {
        if ((threadIdx.x & 63) == 0) atomicOr(fail_word, 1u);
        if (!done) { acc_h[0] = acc_h[1] = acc_h[2] = acc_h[3] = __builtin_nanf(""); }
        break;
      }
      __builtin_amdgcn_s_sleep(1);
      continue;
    }
    if (!done) {
      bool all_final = true;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const unsigned lo = (unsigned)r[i];
        if (acc_a[i] != 0.f) {                           // this channel still needs carries from further back
          acc_h[i] = fmaf(acc_a[i], __uint_as_float((unsigned)(r[i] >> 32)), acc_h[i]);
          acc_a[i] = lo == 1u ? 0.f : acc_a[i] * __uint_as_float(lo);
        }
        all_final = all_final && acc_a[i] == 0.f;
      }
      done = all_final;
    }
    q += step;
  }
  return make_float4(acc_h[0], acc_h[1], acc_h[2], acc_h[3]);
}

RGLRU_DEVICE void rec_store4(rec_t* rec, float4 a, float4 h, bool final) {
  rec_store(rec + 0, final ? 0.f : a.x, h.x);
  rec_store(rec + 1, final ? 0.f : a.y, h.y);
  rec_store(rec + 2, final ? 0.f : a.z, h.z);
  rec_store(rec + 3, final ? 0.f : a.w, h.w);
}

// FORWARD = true: h_t = a_t h_{t-1} + z_t (out0 = h).  FORWARD = false: the reverse scan
// delta_t = dh_t + a_{t+1} delta_{t+1}; out0 = da = delta * h_{t-1}, out1 = dz = delta, dh0 = a_0 delta_0.
template <bool FORWARD>
__global__ __launch_bounds__(kVecThreads, 2) void scan_vec_kernel(ScanArgs p) {
  __shared__ float4 s_a[kVecWaves][64], s_h[kVecWaves][64];
  __shared__ float4 s_carry[64];
  __shared__ unsigned s_ticket;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int groups4 = (p.W + 255) / 256;
  const int chains = p.B * groups4;
  const int nR = (p.T + kVecRun - 1) / kVecRun;          // runs per chain
  const int chain_id = (int)(blockIdx.x % chains);
  if (threadIdx.x == 0) s_ticket = atomicAdd(p.ticket + chain_id, 1u);
  __syncthreads();
  const int tk = (int)s_ticket;
  const int c = FORWARD ? tk : nR - 1 - tk;              // chain order: first run first / last run first
  const int b = chain_id / groups4, grp = chain_id - b * groups4;
  const int ch = grp * 256 + lane * 4;
  const bool ok = ch < p.W;                              // W is a multiple of 4: a lane's channels are all in or all out
  const long long W = p.W;
  const int t0 = c * kVecRun + wave * kVecTokens;
  const long long base = ((long long)b * p.T + t0) * W + ch;

  float4 a[kVecTokens], v[kVecTokens], hp[FORWARD ? 1 : kVecTokens];
  const float4 one = make_float4(1.f, 1.f, 1.f, 1.f), zero = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
  for (int e = 0; e < kVecTokens; ++e) {
    const bool in = ok && (t0 + e < p.T);
    if constexpr (FORWARD) {
      // Both loads are made on every path, from the start of the tensor where the lane has no token, and the
      // defaults are selected afterwards, component by component.  (For `in ? *p : zero` on the four-component struct the
      // compiler selected between the address and a
      // copy of `zero` in scratch memory and loaded through the result: 31 flat loads of 4 and 12 bytes in place of
      // 16 global loads of 16.)
      const long long at = in ? base + e * W : 0;
      const float4 av = *reinterpret_cast<const float4*>(p.a + at), zv = *reinterpret_cast<const float4*>(p.z + at);
      a[e] = make_float4(in ? av.x : 1.f, in ? av.y : 1.f, in ? av.z : 1.f, in ? av.w : 1.f);
      v[e] = make_float4(in ? zv.x : 0.f, in ? zv.y : 0.f, in ? zv.z : 0.f, in ? zv.w : 0.f);
    } else {
      a[e] = in ? *reinterpret_cast<const float4*>(p.a + base + e * W) : one;
      v[e] = in ? *reinterpret_cast<const float4*>(p.dh + base + e * W) : zero;
      hp[e] = zero;
      if (in) hp[e] = (t0 + e == 0) ? *reinterpret_cast<const float4*>(p.h0 + (long long)b * W + ch)
                                    : *reinterpret_cast<const float4*>(p.h_saved + base + (e - 1) * W);
    }
  }
  // the wave's own map: carry_out = A carry_in + H
  float4 A = one, H = zero;
  if constexpr (FORWARD) {
#pragma unroll
    for (int e = 0; e < kVecTokens; ++e) { H = fma4(a[e], H, v[e]); A = mul4(A, a[e]); }
  } else {
#pragma unroll
    for (int e = kVecTokens - 1; e >= 0; --e) {
      const float4 d = make_float4(v[e].x + H.x, v[e].y + H.y, v[e].z + H.z, v[e].w + H.w);
      H = mul4(a[e], d); A = mul4(A, a[e]);
    }
  }
  s_a[wave][lane] = A; s_h[wave][lane] = H;
  __syncthreads();
  // map of the waves in front of this one inside the run (chain order), and of the whole run
  float4 PA = one, PH = zero;
  if constexpr (FORWARD) {
    for (int u = 0; u < wave; ++u) { PH = fma4(s_a[u][lane], PH, s_h[u][lane]); PA = mul4(PA, s_a[u][lane]); }
  } else {
    for (int u = kVecWaves - 1; u > wave; --u) { PH = fma4(s_a[u][lane], PH, s_h[u][lane]); PA = mul4(PA, s_a[u][lane]); }
  }
  const int last_wave = FORWARD ? kVecWaves - 1 : 0;     // the wave at the end of the run in chain order
  if (wave == last_wave) {
    const float4 RA = mul4(PA, A), RH = fma4(A, PH, H);  // the run's map
    rec_t* rec = p.rec_a + (long long)b * p.nC * W + (ok ? ch : 0);
    const int first_run = FORWARD ? 0 : nR - 1;
    float4 carry;
    if (c == first_run) {
      carry = zero;
      if (FORWARD && ok) carry = *reinterpret_cast<const float4*>(p.h0 + (long long)b * W + ch);
    } else {
      if (ok) rec_store4(rec + (long long)c * W, RA, RH, false);
      carry = carry_lookback4(rec, W, c, FORWARD ? -1 : +1, FORWARD ? -1 : nR, zero, ok, p.limit, p.fail);
    }
    const float4 out = fma4(RA, carry, RH);
    if (ok) rec_store4(rec + (long long)c * W, RA, out, true);
    if (!FORWARD && c == 0 && ok) *reinterpret_cast<float4*>(p.dh0 + (long long)b * W + ch) = out;
    s_carry[lane] = carry;
  }
  __syncthreads();
  const float4 run_in = s_carry[lane];
  float4 h = fma4(PA, run_in, PH);                        // carry into this wave's tokens
  if constexpr (FORWARD) {
#pragma unroll
    for (int e = 0; e < kVecTokens; ++e) {
      h = fma4(a[e], h, v[e]);
      if (ok && (t0 + e < p.T)) *reinterpret_cast<float4*>(p.h + base + e * W) = h;
    }
  } else {
#pragma unroll
    for (int e = kVecTokens - 1; e >= 0; --e) {
      const float4 d = make_float4(v[e].x + h.x, v[e].y + h.y, v[e].z + h.z, v[e].w + h.w);
      h = mul4(a[e], d);
      if (ok && (t0 + e < p.T)) {
        *reinterpret_cast<float4*>(p.dz + base + e * W) = d;
        *reinterpret_cast<float4*>(p.da + base + e * W) = mul4(d, hp[e]);
      }
    }
  }
}

static bool pointers_aligned16(const void* const* ptrs, int n) {
  for (int i = 0; i < n; ++i) if ((uintptr_t)ptrs[i] % 16 != 0) return false;
  return true;
}

// Fills the workspace part of the arguments and clears what is asked for.  `vec`: the vector kernels run (rows
// of 128-token runs instead of 32-token chunks in the record array).  `region`: 0 = forward, 1 = backward.
// `clear`: 0 = nothing (the region is known to be clear), 1 = this pass's region, 2 = both regions (forward).
static int scan_common(ScanArgs& p, void* ws, int64_t B, int64_t T, int64_t W, bool vec, int region, int clear, hipStream_t s) {
  if (B <= 0 || T <= 0 || W <= 0) return fail(RGLRU_E_ARG, "scan: B, T, W must be positive (got %lld, %lld, %lld)", (long long)B, (long long)T, (long long)W);
  if (!ws) return fail(RGLRU_E_ARG, "scan: workspace pointer is null");
  if (B * T * W >= (1ll << 40)) return fail(RGLRU_E_UNSUPPORTED, "scan: tensor too large");
  ScanLayout L = make_scan_layout(B, T, W);
  if (B * L.nC * L.groups >= (1ll << 31)) return fail(RGLRU_E_UNSUPPORTED, "scan: too many tiles");
  char* base = (char*)ws + (size_t)region * L.region;
  p.rec_a = (rec_t*)(base + L.rec_a);
  p.ticket = (unsigned*)(base + L.ticket); p.fail = (unsigned*)((char*)ws + L.fail);
  p.B = (int)B; p.T = (int)T; p.W = (int)W; p.groups = (int)L.groups;
  p.nC = vec ? (int)((T + kVecRun - 1) / kVecRun) : (int)L.nC;       // rows per sequence of the record array
  p.tiles = B * L.nC * L.groups;
  p.limit = spin_limit();
  if (clear == 0) return RGLRU_OK;
  // tickets, failure word and the records in use; the other pass of a pair may run the other kernel variant
  // (its tensors decide), so a forward call clears the second region for the variant with more records
  const long long own = ((long long)L.rec_a + round_up(B * (long long)p.nC * W * 8, 16)) / 4;
  const long long full = ((long long)L.rec_a + round_up(B * L.nC * W * 8, 16)) / 4;
  const long long words = clear == 2 ? own + full : own;
  int cb = (int)((words + 1023) / 1024); if (cb > 2048) cb = 2048;
  if (clear == 2) hipLaunchKernelGGL(clear_two_kernel, dim3(cb), dim3(256), 0, s, (unsigned*)base, own, (unsigned*)(base + L.region), full);
  else hipLaunchKernelGGL(clear_words_kernel, dim3(cb), dim3(256), 0, s, (unsigned*)base, own);
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

int rglru_hip_set_reproducible(int enable) { return g_reproducible.exchange(enable ? 1 : 0); }

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
  const void* ptrs[] = {a, z, h0, h};
  const bool vec = W % 4 == 0 && pointers_aligned16(ptrs, 4);
  int rc = scan_common(p, ws, B, T, W, vec, 0, 2, s);
  if (rc) return rc;
  p.a = a; p.z = z; p.h0 = h0; p.h = h;
  if (vec) {
    const long long runs = (long long)B * ((W + 255) / 256) * ((T + kVecRun - 1) / kVecRun);
    hipLaunchKernelGGL(scan_vec_kernel<true>, dim3((unsigned)runs), dim3(kVecThreads), 0, s, p);
    return check_launch("scan_fwd");
  }
  unsigned blocks = (unsigned)((p.tiles + kWaves - 1) / kWaves);
  hipLaunchKernelGGL(scan_fwd_kernel, dim3(blocks), dim3(kThreads), 0, s, p);
  return check_launch("scan_fwd");
}

int rglru_hip_scan_bwd(const float* a, const float* h0, const float* h, const float* dh,
                       float* da, float* dz, float* dh0, void* ws, int ws_fresh,
                       int64_t B, int64_t T, int64_t W, void* stream) {
  if (!a || !h0 || !h || !dh || !da || !dz || !dh0) return fail(RGLRU_E_ARG, "scan_bwd: null tensor pointer");
  ScanArgs p;
  memset(&p, 0, sizeof(p));
  hipStream_t s = (hipStream_t)stream;
  const void* ptrs[] = {a, h0, h, dh, da, dz, dh0};
  const bool vec = W % 4 == 0 && pointers_aligned16(ptrs, 7);
  int rc = scan_common(p, ws, B, T, W, vec, 1, ws_fresh ? 0 : 1, s);
  if (rc) return rc;
  p.a = a; p.h0 = h0; p.h_saved = h; p.dh = dh; p.da = da; p.dz = dz; p.dh0 = dh0;
  if (vec) {
    const long long runs = (long long)B * ((W + 255) / 256) * ((T + kVecRun - 1) / kVecRun);
    hipLaunchKernelGGL(scan_vec_kernel<false>, dim3((unsigned)runs), dim3(kVecThreads), 0, s, p);
    return check_launch("scan_bwd");
  }
  unsigned blocks = (unsigned)((p.tiles + kWaves - 1) / kWaves);
  hipLaunchKernelGGL(scan_bwd_kernel, dim3(blocks), dim3(kThreads), 0, s, p);
  return check_launch("scan_bwd");
}

}  // extern "C"
