// Kernels for the two elementwise stages of the recurrent block that sit directly in front of and
// behind the RG-LRU (griffin/griffin.py:439-529): the causal depthwise temporal convolution
// (:474-487, the all-tokens-active path) and the output gate h * gelu_tanh(v) (:464, :520), each
// forward and backward.  Both are pure streaming, bounded by HBM.
//
// Convolution:
//   out[b,t,c] = bias[c] + sum_{lag<K} taps[c][K-1-lag] * [segment_pos[b,t] >= lag] * padded[b,t-lag,c]
// where padded is the K-1 rows of carried state followed by the T rows of the input.  A thread owns
// V consecutive channels (one 16-byte vector, or one element when the rows are not 16-byte
// aligned) and a run of consecutive tokens of one sequence, keeps the last K-1 rows in registers
// and touches every input and output element once.  All global accesses go through buffer
// descriptors of one sequence: rows past its end read as zero and stores to them are dropped, so
// the token loops carry no bounds branches.

#include <hip/hip_runtime.h>

#include <cstring>
#include <initializer_list>

#include "rglru_device.h"
#include "rglru_host.h"

namespace rglru {

constexpr int kConvMaxTaps = 4;        // kernel sizes 1..4 (the reference uses 4)
constexpr int kConvRunFwd = 16;        // tokens per thread, forward
constexpr int kConvRunBwd = 16;        // tokens per thread, backward (one partial sum per run; 32 left half the chip's load slots idle)
constexpr int kConvThreads = 256;
constexpr int kConvBatch = 8;          // rows requested together, forward
constexpr int kConvBatchBwd = 4;       // backward (two streams, more live state)
constexpr int kConvBwdVecs = 32;       // backward: channel vectors per workgroup ...
constexpr int kConvBwdRuns = kConvThreads / kConvBwdVecs;   // ... and runs, whose partial sums it adds up

struct ConvArgs {
  const void* u; const void* state; const void* taps; const void* bias; const long long* segpos;
  void* out; void* new_state;                               // forward
  const void* dout; void* du; void* dstate; float* partial;  // backward
  long long ld_du;                                          // elements between rows of du (>= W)
  // Right-padded batches whose active tokens are a prefix of the row run on these kernels too: rows[b] = number of
  // active tokens, rows[2 * B + b] != 0 where the row is such a prefix (the others are left to the kernels for
  // arbitrary masks).  Null: every row has T tokens.
  const int* rows;
  int B, T, W, K, nvec, runs, vec_dtype;
};

// Tokens of row b these kernels work on (inputs past them read as zero), or -1 where the row is not theirs.
RGLRU_DEVICE int conv_row_tokens(const ConvArgs& p, int b) {
  if (!p.rows) return p.T;
  return p.rows[2 * p.B + b] ? p.rows[b] : -1;
}

// V values of one row.  `Raw` is the row as loaded (requests are issued in batches before any of
// them is used); unpack turns it into floats.
template <typename IO, int V> struct ConvRow;
template <> struct ConvRow<__bf16, 8> {
  typedef bf16x8 Raw;
  static RGLRU_DEVICE Raw request(rsrc_t r, unsigned off) { return buf_load_frag<bf16x8>(r, off); }
  static RGLRU_DEVICE void unpack(float (&v)[8], const Raw& f) {
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = (float)f[i];
  }
  static RGLRU_DEVICE void load(float (&v)[8], rsrc_t r, unsigned off) { unpack(v, request(r, off)); }
  static RGLRU_DEVICE void store(const float (&v)[8], rsrc_t r, unsigned off) {
    bf16x8 f;
#pragma unroll
    for (int i = 0; i < 8; ++i) f[i] = (__bf16)v[i];
    buf_store_b128(__builtin_bit_cast(i32x4, f), r, off);
  }
};
template <> struct ConvRow<float, 4> {
  typedef f32x4 Raw;
  static RGLRU_DEVICE Raw request(rsrc_t r, unsigned off) { return buf_load_frag<f32x4>(r, off); }
  static RGLRU_DEVICE void unpack(float (&v)[4], const Raw& f) {
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = f[i];
  }
  static RGLRU_DEVICE void load(float (&v)[4], rsrc_t r, unsigned off) { unpack(v, request(r, off)); }
  static RGLRU_DEVICE void store(const float (&v)[4], rsrc_t r, unsigned off) {
    f32x4 f;
#pragma unroll
    for (int i = 0; i < 4; ++i) f[i] = v[i];
    buf_store_b128(__builtin_bit_cast(i32x4, f), r, off);
  }
};
template <typename IO> struct ConvRow<IO, 1> {
  typedef float Raw;
  static RGLRU_DEVICE Raw request(rsrc_t r, unsigned off) { return BufIo<IO>::load(r, off, 0u); }
  static RGLRU_DEVICE void unpack(float (&v)[1], const Raw& f) { v[0] = f; }
  static RGLRU_DEVICE void load(float (&v)[1], rsrc_t r, unsigned off) { v[0] = request(r, off); }
  static RGLRU_DEVICE void store(const float (&v)[1], rsrc_t r, unsigned off) { BufIo<IO>::store((IO)v[0], r, off, 0u); }
};

RGLRU_DEVICE float conv_param(const void* base, long long i, int vec_dtype) {
  return vec_dtype == RGLRU_BF16 ? (float)((const __bf16*)base)[i] : ((const float*)base)[i];
}

// N consecutive parameters starting at element `first`, as fp32.  With 16-byte alignment (of the
// pointer, of the first element and of the length) they come as 16-byte loads: element-wise loads
// of a lane's 8 channels x 4 taps touch 32 cache lines per instruction and wave.
template <int N>
RGLRU_DEVICE void conv_params(const void* base, long long first, int vec_dtype, float (&out)[N]) {
  const int es = vec_dtype == RGLRU_BF16 ? 2 : 4;
  if ((N * es) % 16 == 0 && (first * es) % 16 == 0 && (uintptr_t)base % 16 == 0) {
    const uint4* src = reinterpret_cast<const uint4*>((const char*)base + first * es);
    if (vec_dtype == RGLRU_BF16) {
#pragma unroll
      for (int q = 0; q < (N * 2 + 15) / 16; ++q) {
        const uint4 v = src[q];
        const unsigned w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (8 * q + 2 * i < N) out[8 * q + 2 * i] = __uint_as_float(w[i] << 16);
          if (8 * q + 2 * i + 1 < N) out[8 * q + 2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
        }
      }
    } else {
#pragma unroll
      for (int q = 0; q < (N * 4 + 15) / 16; ++q) {
        const uint4 v = src[q];
        const unsigned w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (4 * q + i < N) out[4 * q + i] = __uint_as_float(w[i]);
      }
    }
  } else if (vec_dtype == RGLRU_BF16) {                    // one branch on the type, then all loads in flight together
    __bf16 raw[N];
#pragma unroll
    for (int i = 0; i < N; ++i) raw[i] = ((const __bf16*)base)[first + i];
#pragma unroll
    for (int i = 0; i < N; ++i) out[i] = (float)raw[i];
  } else {
#pragma unroll
    for (int i = 0; i < N; ++i) out[i] = ((const float*)base)[first + i];
  }
}

// Taps [channel][K] and biases of the V channels that start at c0: tap[j][v], bias[v] (zero without a bias).
template <int V, int K>
RGLRU_DEVICE void conv_load_taps(const void* taps, const void* bias_ptr, int c0, int vec_dtype,
                                 float (&tap)[K][V], float (&bias)[V]) {
  float flat[V * K];
  conv_params<V * K>(taps, (long long)c0 * K, vec_dtype, flat);
#pragma unroll
  for (int v = 0; v < V; ++v)
#pragma unroll
    for (int j = 0; j < K; ++j) tap[j][v] = flat[v * K + j];
  if (bias_ptr) {
    conv_params<V>(bias_ptr, c0, vec_dtype, bias);
  } else {
#pragma unroll
    for (int v = 0; v < V; ++v) bias[v] = 0.f;
  }
}

// Which (sequence, run, channel vector) a thread owns.  A workgroup stays inside one sequence
// (blocks_per_seq workgroups each), so that the sequence, and with it every buffer descriptor built
// from it, is the same in all lanes; vectors vary fastest, so the lanes of a wave read consecutive
// addresses of one row.
struct ConvItem { int b, run, c0; bool ok; };
__host__ __device__ inline long long conv_blocks_per_seq(int runs, int nvec) {
  return ((long long)runs * nvec + kConvThreads - 1) / kConvThreads;
}
RGLRU_DEVICE ConvItem conv_item(const ConvArgs& p) {
  ConvItem it;
  const unsigned per_seq = (unsigned)conv_blocks_per_seq(p.runs, p.nvec);
  it.b = (int)(blockIdx.x / per_seq);
  const long long item = (long long)(blockIdx.x - (unsigned)it.b * per_seq) * kConvThreads + threadIdx.x;
  it.ok = item < (long long)p.runs * p.nvec;
  const long long safe = it.ok ? item : 0;
  it.run = (int)(safe / p.nvec);
  it.c0 = (int)(safe - (long long)it.run * p.nvec) * (p.W / p.nvec);
  return it;
}

// Row `t` of the padded input of one sequence (t < 0: carried state, zeros when there is none).  Both
// sources are asked, the one that does not hold the row past its end, so that neither the descriptor
// nor the control flow depends on the lane; `ok` false gives zeros.  `rs` is conv_state_rsrc().
template <typename IO, int V, int K>
RGLRU_DEVICE void padded_row(const ConvArgs& p, rsrc_t ru, rsrc_t rs, bool ok, int t, int c0, float (&v)[V]) {
  const unsigned es = (unsigned)sizeof(IO);
  const bool from_state = t < 0;
  const unsigned off_u = ok && t >= 0 ? ((unsigned)t * (unsigned)p.W + (unsigned)c0) * es : kOutOfRange;
  const unsigned off_s = ok && from_state && K - 1 + t >= 0 ? ((unsigned)(K - 1 + t) * (unsigned)p.W + (unsigned)c0) * es
                                                            : kOutOfRange;
  const typename ConvRow<IO, V>::Raw raw_u = ConvRow<IO, V>::request(ru, off_u);
  const typename ConvRow<IO, V>::Raw raw_s = ConvRow<IO, V>::request(rs, off_s);
  float from_u[V], from_s[V];
  ConvRow<IO, V>::unpack(from_u, raw_u);
  ConvRow<IO, V>::unpack(from_s, raw_s);
#pragma unroll
  for (int i = 0; i < V; ++i) v[i] = from_state ? from_s[i] : from_u[i];
}

// The carried state of sequence b as a buffer (empty without one, so that its loads return zero).
template <typename IO, int K>
RGLRU_DEVICE rsrc_t conv_state_rsrc(const ConvArgs& p, int b) {
  return make_rsrc(p.state ? (const IO*)p.state + (long long)b * (K - 1) * p.W : (const IO*)p.u,
                   p.state ? (unsigned)((K - 1) * p.W) * (unsigned)sizeof(IO) : 0u);
}

template <typename IO, int V, int K>
__global__ __launch_bounds__(kConvThreads) void conv_fwd_kernel(ConvArgs p) {
  const ConvItem it = conv_item(p);
  if (!it.ok) return;
  const int b = it.b, c0 = it.c0, t0 = it.run * kConvRunFwd;
  const int n = conv_row_tokens(p, b);
  if (n < 0) return;
  const unsigned es = (unsigned)sizeof(IO), uW = (unsigned)p.W;
  float tap[K][V], bias[V];
  conv_load_taps<V, K>(p.taps, p.bias, c0, p.vec_dtype, tap, bias);
  const unsigned seq_bytes = (unsigned)p.T * uW * es;
  const rsrc_t ru = make_rsrc((const IO*)p.u + (long long)b * p.T * p.W, (unsigned)n * uW * es);
  const rsrc_t ro = make_rsrc((const IO*)p.out + (long long)b * p.T * p.W, seq_bytes);
  const rsrc_t rs = conv_state_rsrc<IO, K>(p, b);
  const long long* sp_row = p.segpos + (long long)b * p.T;

  float win[K > 1 ? K - 1 : 1][V];                         // win[j] = padded row t - 1 - j
#pragma unroll
  for (int j = 0; j < K - 1; ++j) padded_row<IO, V, K>(p, ru, rs, true, t0 - 1 - j, c0, win[j]);
  for (int t1 = 0; t1 < kConvRunFwd; t1 += kConvBatch) {
   typename ConvRow<IO, V>::Raw raw[kConvBatch];
   long long spb[kConvBatch];
#pragma unroll
   for (int i = 0; i < kConvBatch; ++i) {
     const int t = t0 + t1 + i;
     raw[i] = ConvRow<IO, V>::request(ru, ((unsigned)t * uW + (unsigned)c0) * es);
     spb[i] = sp_row[t < p.T ? t : p.T - 1];
   }
#pragma unroll
   for (int i = 0; i < kConvBatch; ++i) {
    const int t = t0 + t1 + i;
    const unsigned off = ((unsigned)t * uW + (unsigned)c0) * es;
    float cur[V], acc[V];
    ConvRow<IO, V>::unpack(cur, raw[i]);
    const long long sp = spb[i];
#pragma unroll
    for (int v = 0; v < V; ++v) {
      float a = bias[v];
      if (sp >= 0) a = fmaf(cur[v], tap[K - 1][v], a);
#pragma unroll
      for (int lag = 1; lag < K; ++lag)
        if (sp >= lag) a = fmaf(win[lag - 1][v], tap[K - 1 - lag][v], a);
      acc[v] = t < n ? a : 0.f;                            // padding behind the row's tokens
    }
    ConvRow<IO, V>::store(acc, ro, off);
#pragma unroll
    for (int j = K - 2; j > 0; --j)
#pragma unroll
      for (int v = 0; v < V; ++v) win[j][v] = win[j - 1][v];
    if (K > 1) {
#pragma unroll
      for (int v = 0; v < V; ++v) win[0][v] = cur[v];
    }
   }
  }
  // carried state for the next call: the last K-1 rows of the padded input
  if (K > 1 && p.new_state && it.run == p.runs - 1) {
    const rsrc_t rn = make_rsrc((IO*)p.new_state + (long long)b * (K - 1) * p.W, (unsigned)((K - 1) * p.W) * es);
#pragma unroll
    for (int j = 0; j < K - 1; ++j) {
      float row[V];
      padded_row<IO, V, K>(p, ru, rs, true, p.T - (K - 1) + j, c0, row);
      ConvRow<IO, V>::store(row, rn, ((unsigned)j * uW + (unsigned)c0) * es);
    }
  }
}

// Backward: du, the gradient at the carried state (optional) and partial sums of the tap and bias
// gradients.  A workgroup covers kConvBwdVecs channel vectors and kConvBwdRuns consecutive runs of
// one sequence and adds the sums of its runs up in LDS:
//   partial[((b * run_groups + run_group) * (K + 1) + j) * W + c],  j = K for the bias.
template <typename IO, int V, int K>
__global__ __launch_bounds__(kConvThreads) void conv_bwd_kernel(ConvArgs p) {
  __shared__ float red[kConvBwdRuns][(K + 1) * V][kConvBwdVecs + 1];
  const int vec_groups = (p.nvec + kConvBwdVecs - 1) / kConvBwdVecs;
  const int run_groups = (p.runs + kConvBwdRuns - 1) / kConvBwdRuns;
  const int vg = blockIdx.x % vec_groups;
  const int rest = blockIdx.x / vec_groups;
  const int rgp = rest % run_groups, b = rest / run_groups;
  const int lane_vec = threadIdx.x % kConvBwdVecs, lane_run = threadIdx.x / kConvBwdVecs;
  const int vec = vg * kConvBwdVecs + lane_vec, run = rgp * kConvBwdRuns + lane_run;
  const bool ok = vec < p.nvec && run < p.runs;
  const int c0 = (vec < p.nvec ? vec : 0) * V, t0 = run * kConvRunBwd;
  const unsigned es = (unsigned)sizeof(IO), uW = (unsigned)p.W;
  float tap[K][V], bias_unused[V];
  conv_load_taps<V, K>(p.taps, nullptr, c0, p.vec_dtype, tap, bias_unused);
  // The descriptors are the same in all lanes.  A thread without work addresses past their end:
  // its loads return zero and its stores are dropped.
  const int n = conv_row_tokens(p, b);
  if (n < 0) return;                                       // the whole workgroup: it lies inside one sequence
  const unsigned seq_bytes = (unsigned)n * uW * es;        // the gradient of a padded output is not read: it counts as zero
  const rsrc_t ru = make_rsrc((const IO*)p.u + (long long)b * p.T * p.W, seq_bytes);
  const rsrc_t rd = make_rsrc((const IO*)p.dout + (long long)b * p.T * p.W, seq_bytes);
  const unsigned ld_du = (unsigned)p.ld_du;
  const rsrc_t rg = make_rsrc((const IO*)p.du + (long long)b * p.T * p.ld_du, ((unsigned)(p.T - 1) * ld_du + uW) * es);
  const rsrc_t rs_in = conv_state_rsrc<IO, K>(p, b);
  const long long* sp_row = p.segpos + (long long)b * p.T;
  auto position = [&](int t) { return sp_row[t < p.T ? t : p.T - 1]; };
  auto at = [&](int t) { return ok ? ((unsigned)t * uW + (unsigned)c0) * es : kOutOfRange; };
  auto at_du = [&](int t) { return ok ? ((unsigned)t * ld_du + (unsigned)c0) * es : kOutOfRange; };

  float dwin[K][V];                                        // dwin[j] = dout row t + j
  long long spw[K];
  float uwin[K > 1 ? K - 1 : 1][V];                        // uwin[j] = padded row t - 1 - j
  float acc_tap[K][V], acc_bias[V];
#pragma unroll
  for (int v = 0; v < V; ++v) {
    acc_bias[v] = 0.f;
#pragma unroll
    for (int j = 0; j < K; ++j) acc_tap[j][v] = 0.f;
  }
#pragma unroll
  for (int j = 0; j < K - 1; ++j) {
    ConvRow<IO, V>::load(dwin[j], rd, at(t0 + j));
    spw[j] = position(t0 + j);
    padded_row<IO, V, K>(p, ru, rs_in, ok, t0 - 1 - j, c0, uwin[j]);
  }
  for (int t1 = 0; t1 < kConvRunBwd; t1 += kConvBatchBwd) {
    typename ConvRow<IO, V>::Raw raw_u[kConvBatchBwd], raw_d[kConvBatchBwd];
    long long spb[kConvBatchBwd];
#pragma unroll
    for (int i = 0; i < kConvBatchBwd; ++i) {
      const int t = t0 + t1 + i;
      raw_u[i] = ConvRow<IO, V>::request(ru, at(t));
      raw_d[i] = ConvRow<IO, V>::request(rd, at(t + K - 1));
      spb[i] = position(t + K - 1);
    }
#pragma unroll
    for (int i = 0; i < kConvBatchBwd; ++i) {
      const int t = t0 + t1 + i;
      const unsigned off = at_du(t);
      ConvRow<IO, V>::unpack(dwin[K - 1], raw_d[i]);
      spw[K - 1] = spb[i];
      float cur[V], g[V];
      ConvRow<IO, V>::unpack(cur, raw_u[i]);
#pragma unroll
      for (int v = 0; v < V; ++v) {
        // input gradient: token t feeds the outputs t .. t + K - 1
        float a = 0.f;
#pragma unroll
        for (int lag = 0; lag < K; ++lag)
          if (spw[lag] >= lag) a = fmaf(dwin[lag][v], tap[K - 1 - lag][v], a);
        g[v] = a;
        // parameter gradients of output t
        const float d = dwin[0][v];
        acc_bias[v] += d;
        if (spw[0] >= 0) acc_tap[K - 1][v] = fmaf(d, cur[v], acc_tap[K - 1][v]);
#pragma unroll
        for (int lag = 1; lag < K; ++lag)
          if (spw[0] >= lag) acc_tap[K - 1 - lag][v] = fmaf(d, uwin[lag - 1][v], acc_tap[K - 1 - lag][v]);
      }
      ConvRow<IO, V>::store(g, rg, off);
#pragma unroll
      for (int j = 0; j < K - 1; ++j) {
        spw[j] = spw[j + 1];
#pragma unroll
        for (int v = 0; v < V; ++v) dwin[j][v] = dwin[j + 1][v];
      }
#pragma unroll
      for (int j = K - 2; j > 0; --j)
#pragma unroll
        for (int v = 0; v < V; ++v) uwin[j][v] = uwin[j - 1][v];
      if (K > 1) {
#pragma unroll
        for (int v = 0; v < V; ++v) uwin[0][v] = cur[v];
      }
    }
  }

  // gradient at the carried state: state row j stands at time j - (K - 1) < 0
  if (K > 1 && p.dstate && ok && run == 0) {
    const rsrc_t rs = make_rsrc((IO*)p.dstate + (long long)b * (K - 1) * p.W, (unsigned)((K - 1) * p.W) * es);
#pragma unroll
    for (int j = 0; j < K - 1; ++j) {
      const int tau = j - (K - 1);
      float a[V];
#pragma unroll
      for (int v = 0; v < V; ++v) a[v] = 0.f;
#pragma unroll
      for (int lag = 1; lag < K; ++lag) {
        const int t = tau + lag;
        if (t >= 0 && t < p.T && position(t) >= lag) {
          float d[V];
          ConvRow<IO, V>::load(d, rd, ((unsigned)t * uW + (unsigned)c0) * es);
#pragma unroll
          for (int v = 0; v < V; ++v) a[v] = fmaf(d[v], tap[K - 1 - lag][v], a[v]);
        }
      }
      ConvRow<IO, V>::store(a, rs, ((unsigned)j * uW + (unsigned)c0) * es);
    }
  }

  // sums of the workgroup's runs (threads without work hold zeros)
#pragma unroll
  for (int j = 0; j < K; ++j)
#pragma unroll
    for (int v = 0; v < V; ++v) red[lane_run][j * V + v][lane_vec] = acc_tap[j][v];
#pragma unroll
  for (int v = 0; v < V; ++v) red[lane_run][K * V + v][lane_vec] = acc_bias[v];
  __syncthreads();
  float* part = p.partial + ((long long)(b * run_groups + rgp) * (K + 1)) * p.W;
  for (int idx = threadIdx.x; idx < (K + 1) * V * kConvBwdVecs; idx += kConvThreads) {
    const int row = idx / kConvBwdVecs, lv = idx - row * kConvBwdVecs;   // row = j * V + v
    const int j = row / V, v = row - j * V;
    const int ch = (vg * kConvBwdVecs + lv) * V + v;
    if (ch < p.W) {
      float sum = 0.f;
#pragma unroll
      for (int q = 0; q < kConvBwdRuns; ++q) sum += red[q][row][lv];
      part[(long long)j * p.W + ch] = sum;
    }
  }
}

// Sums the per-run partials: one thread per (tap or bias, channel).
struct ConvFinishArgs { const float* partial; void* dtaps; void* dbias; int W, K, slots, grad_dtype; };
__global__ __launch_bounds__(256) void conv_finish_kernel(ConvFinishArgs p) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= (long long)(p.K + 1) * p.W) return;
  const int j = (int)(i / p.W), c = (int)(i - (long long)j * p.W);
  const float* src = p.partial + (long long)j * p.W + c;
  const long long stride = (long long)(p.K + 1) * p.W;
  float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
  int n = 0;
  for (; n + 16 <= p.slots; n += 16) {                   // sixteen loads in flight: latency, not bytes, is what this kernel waits for
    float v[16];
#pragma unroll
    for (int u = 0; u < 16; ++u) v[u] = src[(long long)(n + u) * stride];
#pragma unroll
    for (int u = 0; u < 16; u += 4) { s0 += v[u]; s1 += v[u + 1]; s2 += v[u + 2]; s3 += v[u + 3]; }
  }
  for (; n < p.slots; ++n) s0 += src[(long long)n * stride];
  const float s = (s0 + s1) + (s2 + s3);
  void* dst = j < p.K ? p.dtaps : p.dbias;
  if (!dst) return;
  const long long at = j < p.K ? (long long)c * p.K + j : c;
  if (p.grad_dtype == RGLRU_BF16) ((__bf16*)dst)[at] = (__bf16)s; else ((float*)dst)[at] = s;
}

// ------------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------------
static int conv_check(const char* who, int64_t B, int64_t T, int64_t W, int64_t K, int dtype, int vec_dtype) {
  if (dtype != RGLRU_F32 && dtype != RGLRU_BF16) return fail(RGLRU_E_ARG, "%s: dtype must be RGLRU_F32 or RGLRU_BF16, got %d", who, dtype);
  if (vec_dtype != RGLRU_F32 && vec_dtype != RGLRU_BF16) return fail(RGLRU_E_ARG, "%s: unknown parameter dtype %d", who, vec_dtype);
  if (B <= 0 || T <= 0 || W <= 0) return fail(RGLRU_E_ARG, "%s: empty shape B=%lld T=%lld W=%lld", who, (long long)B, (long long)T, (long long)W);
  if (K < 1 || K > kConvMaxTaps) return fail(RGLRU_E_UNSUPPORTED, "%s: kernel size %lld outside 1..%d", who, (long long)K, kConvMaxTaps);
  const int64_t es = dtype == RGLRU_BF16 ? 2 : 4;
  if ((T + kConvRunBwd + K) * W * es >= (1ll << 31)) return fail(RGLRU_E_UNSUPPORTED, "%s: one sequence exceeds 2 GiB", who);
  if (B * ((T + kConvRunFwd - 1) / kConvRunFwd) * W >= (1ll << 40)) return fail(RGLRU_E_UNSUPPORTED, "%s: tensor too large", who);
  return RGLRU_OK;
}

static bool conv_vector_ok(int64_t W, int dtype, std::initializer_list<const void*> ptrs) {
  const int v = dtype == RGLRU_BF16 ? 8 : 4;
  if (W % v) return false;
  for (const void* q : ptrs) if (q && (uintptr_t)q % 16) return false;
  return true;
}

#define RGLRU_CONV_K(KERNEL, IO, V, grid, s, a)                                                     \
  switch ((a).K) {                                                                                  \
    case 1: hipLaunchKernelGGL((KERNEL<IO, V, 1>), grid, dim3(kConvThreads), 0, s, a); break;       \
    case 2: hipLaunchKernelGGL((KERNEL<IO, V, 2>), grid, dim3(kConvThreads), 0, s, a); break;       \
    case 3: hipLaunchKernelGGL((KERNEL<IO, V, 3>), grid, dim3(kConvThreads), 0, s, a); break;       \
    default: hipLaunchKernelGGL((KERNEL<IO, V, 4>), grid, dim3(kConvThreads), 0, s, a); break;      \
  }
#define RGLRU_CONV_DISPATCH(KERNEL, dtype, vec, grid, s, a)                                          \
  do {                                                                                              \
    if ((dtype) == RGLRU_BF16) { if (vec) { RGLRU_CONV_K(KERNEL, __bf16, 8, grid, s, a) } else { RGLRU_CONV_K(KERNEL, __bf16, 1, grid, s, a) } } \
    else { if (vec) { RGLRU_CONV_K(KERNEL, float, 4, grid, s, a) } else { RGLRU_CONV_K(KERNEL, float, 1, grid, s, a) } } \
  } while (0)


// ------------------------------------------------------------------------------------------
// Convolution over right-padded batches (griffin/griffin.py:488-510), forward only.  The reference
// walks the tokens one by one with a window of the last K-1 ACTIVE inputs, cleared where an active
// token starts a document.  Here the walk is split in two parallel kernels:
//   conv_padded_index_kernel  one wave per row: the ordinal of every active token among the active
//       ones, the ordinal at which its document started (-1: no start inside this call) and the
//       list ordinal -> token, by ballots and population counts over 64 tokens at a time;
//   conv_padded_fwd_kernel    per token and channel vector, like the dense kernel, gathering the
//       rows of the K-1 previous active tokens (or carried state rows, or zeros) through that list.
// A row whose active tokens are a prefix of it (a right-padded batch: every row of one) needs none of
// that: there the ordinal is the token, and the convolution is the dense one over the first `count` tokens
// with the position `ordinal - document start` (unbounded where no document starts inside the call).  The
// index kernel writes those positions as well and marks such rows; conv_fwd_kernel / conv_bwd_kernel take
// them (ConvArgs::rows) and the two kernels here leave them alone.
// Scratch: position[B][T] (64-bit), then 32-bit words ord[B][T], start[B][T], list[B][T], count[B],
// final_start[B], prefix[B].
// ------------------------------------------------------------------------------------------
struct PaddedArgs {
  const void* u; const void* state; const void* taps; const void* bias;
  const long long* segpos; const unsigned char* active;
  void* out; void* new_state; int* scratch;
  const void* dout; void* du; void* dstate; float* partial;   // backward
  int B, T, W, K, nvec, runs, vec_dtype;
};

// The parts of the index of sequence b.
struct PaddedIndex { long long* position; int* ord; int* start; int* list; int* tail; };
RGLRU_DEVICE PaddedIndex padded_index(const PaddedArgs& p, int b) {
  PaddedIndex x;
  const long long cells = (long long)p.B * p.T;
  x.position = reinterpret_cast<long long*>(p.scratch) + (long long)b * p.T;
  int* words = p.scratch + 2 * cells;
  x.ord = words + (long long)b * p.T;
  x.start = words + cells + (long long)b * p.T;
  x.list = words + 2 * cells + (long long)b * p.T;
  x.tail = words + 3 * cells;
  return x;
}
constexpr long long kUnboundedPosition = 1ll << 30;        // no document start in front of the token inside this call

__global__ __launch_bounds__(64) void conv_padded_index_kernel(PaddedArgs p) {
  const int b = blockIdx.x, lane = threadIdx.x;
  const PaddedIndex x = padded_index(p, b);
  int* ord = x.ord; int* start = x.start; int* list = x.list; int* tail = x.tail;
  int count = 0, doc_start = -1, last_active = -1;         // wave-uniform running values
  // The walk is a chain of wave-uniform values, so a chunk's loads must not wait behind the chunk in front of
  // it: the flags and positions of kAhead chunks are requested together (clamped index, so every load is
  // unconditional), then the chunks are walked from registers.
  constexpr int kAhead = 8;
  const unsigned char* act_row = p.active + (long long)b * p.T;
  const long long* pos_row = p.segpos + (long long)b * p.T;
  for (int base = 0; base < p.T; base += 64 * kAhead) {
    unsigned char act_v[kAhead];
    long long pos_v[kAhead];
#pragma unroll
    for (int q = 0; q < kAhead; ++q) {
      const int tq = base + 64 * q + lane;
      const int tc = tq < p.T ? tq : p.T - 1;
      act_v[q] = act_row[tc];
      pos_v[q] = pos_row[tc];
    }
#pragma unroll
    for (int q = 0; q < kAhead; ++q) {
    const int t0 = base + 64 * q;
    if (t0 >= p.T) break;
    const int t = t0 + lane;
    const bool in = t < p.T;
    const bool act = in && act_v[q] != 0;
    const bool rst = act && pos_v[q] == 0;
    const unsigned long long am = __ballot(act), rm = __ballot(rst);
    const unsigned long long below = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
    const int my_ord = count + __popcll(am & below);
    // last document start at or before this token inside the chunk, else the running one
    const unsigned long long upto = rm & (below | (1ull << lane));
    int my_start = doc_start;
    if (upto) {
      const int at = 63 - __clzll(upto);
      my_start = count + __popcll(am & ((at == 0) ? 0ull : (~0ull >> (64 - at))));
    }
    if (in) {
      ord[t] = act ? my_ord : -1; start[t] = my_start;
      x.position[t] = my_start < 0 ? kUnboundedPosition : (long long)(my_ord - my_start);   // read for prefix rows only
    }
    if (act) list[my_ord] = t;
    if (am) last_active = t0 + 63 - __clzll(am);
    if (rm) {
      const int at = 63 - __clzll(rm);
      doc_start = count + __popcll(am & ((at == 0) ? 0ull : (~0ull >> (64 - at))));
    }
    count += __popcll(am);
    }
  }
  if (lane == 0) { tail[b] = count; tail[p.B + b] = doc_start; tail[2 * p.B + b] = count == last_active + 1 ? 1 : 0; }
}

__host__ __device__ inline long long padded_blocks_per_seq(int T, int nvec) {
  return ((long long)(T + 1) * nvec + kConvThreads - 1) / kConvThreads;
}

// Row that stands `lag` active tokens before ordinal i of sequence b, as floats.
template <typename IO, int V, int K>
RGLRU_DEVICE void padded_source(const PaddedArgs& p, rsrc_t ru, rsrc_t rs, const int* list, int i, int lag, int doc_start,
                                int c0, float (&v)[V]) {
  const int j = i - lag;
  const unsigned es = (unsigned)sizeof(IO), uW = (unsigned)p.W;
  // both sources are asked (the one that does not apply at an offset that reads as zero) and the row is selected
  // afterwards: a descriptor chosen per lane would turn the load into a loop over the lanes' choices
  unsigned off_u = kOutOfRange, off_s = kOutOfRange;
  bool from_state = false;
  if (j >= 0 && j >= doc_start) off_u = ((unsigned)list[j] * uW + (unsigned)c0) * es;
  else if (doc_start < 0 && j < 0 && K - 1 + j >= 0) { off_s = ((unsigned)(K - 1 + j) * uW + (unsigned)c0) * es; from_state = true; }
  float s[V];
  ConvRow<IO, V>::load(v, ru, off_u);
  ConvRow<IO, V>::load(s, rs, off_s);
#pragma unroll
  for (int e = 0; e < V; ++e) v[e] = from_state ? s[e] : v[e];
}

template <typename IO, int V, int K>
__global__ __launch_bounds__(kConvThreads) void conv_padded_fwd_kernel(PaddedArgs p) {
  // a workgroup stays inside one sequence, so the descriptors below are the same in all its lanes
  const long long per_seq = (long long)(p.T + 1) * p.nvec;    // one extra "token" per row writes the new state
  const unsigned wg_per_seq = (unsigned)padded_blocks_per_seq(p.T, p.nvec);
  const int b = __builtin_amdgcn_readfirstlane((int)(blockIdx.x / wg_per_seq));   // the quotient comes out of the vector unit
  const long long rest = (long long)(blockIdx.x - (unsigned)b * wg_per_seq) * kConvThreads + threadIdx.x;
  if (rest >= per_seq) return;
  const int t = (int)(rest / p.nvec), c0 = (int)(rest - (long long)t * p.nvec) * V;
  const unsigned es = (unsigned)sizeof(IO), uW = (unsigned)p.W;
  const PaddedIndex x = padded_index(p, b);
  const int* ord = x.ord; const int* start = x.start; const int* list = x.list; const int* tail = x.tail;
  if (t < p.T && tail[2 * p.B + b]) return;                // a prefix row: the dense kernel writes its outputs
  const rsrc_t ru = make_rsrc((const IO*)p.u + (long long)b * p.T * p.W, (unsigned)p.T * uW * es);
  const rsrc_t rs = make_rsrc(p.state ? (const IO*)p.state + (long long)b * (K - 1) * p.W : (const IO*)p.u,
                              p.state ? (unsigned)((K - 1) * p.W) * es : 0u);
  if (t == p.T) {
    // carried state: the last K-1 active inputs since the last document start, oldest first
    if (K > 1 && p.new_state) {
      const int n = tail[b], doc_start = tail[p.B + b];
      const rsrc_t rn = make_rsrc((IO*)p.new_state + (long long)b * (K - 1) * p.W, (unsigned)((K - 1) * p.W) * es);
#pragma unroll
      for (int lag = 1; lag < K; ++lag) {
        float row[V];
        padded_source<IO, V, K>(p, ru, rs, list, n, lag, doc_start, c0, row);
        ConvRow<IO, V>::store(row, rn, ((unsigned)(K - 1 - lag) * uW + (unsigned)c0) * es);
      }
    }
    return;
  }
  const rsrc_t ro = make_rsrc((IO*)p.out + (long long)b * p.T * p.W, (unsigned)p.T * uW * es);
  const unsigned off = ((unsigned)t * uW + (unsigned)c0) * es;
  const int i = ord[t];
  float acc[V];
  if (i < 0) {
#pragma unroll
    for (int v = 0; v < V; ++v) acc[v] = 0.f;
  } else {
    const int doc_start = start[t];
    float cur[V], tap[K][V], bias[V];
    ConvRow<IO, V>::load(cur, ru, off);
    conv_load_taps<V, K>(p.taps, p.bias, c0, p.vec_dtype, tap, bias);
#pragma unroll
    for (int v = 0; v < V; ++v) acc[v] = fmaf(cur[v], tap[K - 1][v], bias[v]);
#pragma unroll
    for (int lag = 1; lag < K; ++lag) {
      float row[V];
      padded_source<IO, V, K>(p, ru, rs, list, i, lag, doc_start, c0, row);
#pragma unroll
      for (int v = 0; v < V; ++v) acc[v] = fmaf(row[v], tap[K - 1 - lag][v], acc[v]);
    }
  }
  ConvRow<IO, V>::store(acc, ro, off);
}

// Reverse mode of the padded convolution.  In ordinal space (the active tokens of a row in order) the
// forward pass is a plain causal convolution whose taps are cut at the output's document start, so the
// gradient of the input at ordinal j collects the outputs at ordinals j .. j + K - 1 whose document
// started at or before j; the carried state rows stand at ordinals -(K-1) .. -1 and feed only outputs
// without a document start in front of them.  Threads are laid out as in conv_bwd_kernel (a thread owns
// a run of kConvRunBwd consecutive tokens of one channel vector; tap and bias gradients are summed per
// workgroup and written as one partial row per (sequence, group of runs)).
template <typename IO, int V, int K>
__global__ __launch_bounds__(kConvThreads) void conv_padded_bwd_kernel(PaddedArgs p) {
  __shared__ float red[kConvBwdRuns][(K + 1) * V][kConvBwdVecs + 1];
  const int vec_groups = (p.nvec + kConvBwdVecs - 1) / kConvBwdVecs;
  const int run_groups = (p.runs + kConvBwdRuns - 1) / kConvBwdRuns;
  // quotients of workgroup-uniform values come out of the vector unit (integer division runs there): said to be
  // uniform here, so that the sequence's descriptors live in scalar registers
  const int vg = __builtin_amdgcn_readfirstlane((int)(blockIdx.x % vec_groups));
  const int rest = __builtin_amdgcn_readfirstlane((int)(blockIdx.x / vec_groups));
  const int rgp = __builtin_amdgcn_readfirstlane(rest % run_groups), b = __builtin_amdgcn_readfirstlane(rest / run_groups);
  const int lane_vec = threadIdx.x % kConvBwdVecs, lane_run = threadIdx.x / kConvBwdVecs;
  const int vec = vg * kConvBwdVecs + lane_vec, run = rgp * kConvBwdRuns + lane_run;
  const bool ok = vec < p.nvec && run < p.runs;
  const int c0 = (vec < p.nvec ? vec : 0) * V, t0 = run * kConvRunBwd;
  const unsigned es = (unsigned)sizeof(IO), uW = (unsigned)p.W;
  const PaddedIndex x = padded_index(p, b);
  const int* ord = x.ord; const int* start = x.start; const int* list = x.list; const int* tail = x.tail;
  if (tail[2 * p.B + b]) return;                           // a prefix row: the dense kernel does it, partial sums included
  const int n = tail[b];                                   // active tokens of the row
  float tap[K][V], bias_unused[V];
  conv_load_taps<V, K>(p.taps, nullptr, c0, p.vec_dtype, tap, bias_unused);
  // the descriptors are the same in every lane (a thread without work leaves the token loop at once and takes no
  // part in the state gradient), so no access through them becomes a loop over the lanes' values
  const unsigned seq_bytes = (unsigned)p.T * uW * es;
  const rsrc_t ru = make_rsrc((const IO*)p.u + (long long)b * p.T * p.W, seq_bytes);
  const rsrc_t rd = make_rsrc((const IO*)p.dout + (long long)b * p.T * p.W, seq_bytes);
  const rsrc_t rg = make_rsrc((const IO*)p.du + (long long)b * p.T * p.W, seq_bytes);
  const rsrc_t rs = make_rsrc(p.state ? (const IO*)p.state + (long long)b * (K - 1) * p.W : (const IO*)p.u,
                              p.state ? (unsigned)((K - 1) * p.W) * es : 0u);
  float acc_tap[K][V], acc_bias[V];
#pragma unroll
  for (int v = 0; v < V; ++v) {
    acc_bias[v] = 0.f;
#pragma unroll
    for (int j = 0; j < K; ++j) acc_tap[j][v] = 0.f;
  }
  for (int t1 = 0; t1 < kConvRunBwd; ++t1) {
    const int t = t0 + t1;
    if (!ok || t >= p.T) break;
    const unsigned off = ((unsigned)t * uW + (unsigned)c0) * es;
    const int i = ord[t];
    float g[V];
#pragma unroll
    for (int v = 0; v < V; ++v) g[v] = 0.f;
    if (i >= 0) {
      // input gradient: ordinal i feeds the outputs at ordinals i .. i + K - 1 of its document
#pragma unroll
      for (int lag = 0; lag < K; ++lag) {
        const int i2 = i + lag;
        if (i2 < n) {
          const int t2 = list[i2];
          if (start[t2] <= i) {
            float d[V];
            ConvRow<IO, V>::load(d, rd, ((unsigned)t2 * uW + (unsigned)c0) * es);
#pragma unroll
            for (int v = 0; v < V; ++v) g[v] = fmaf(d[v], tap[K - 1 - lag][v], g[v]);
          }
        }
      }
      // parameter gradients of the output at this token
      float d[V];
      ConvRow<IO, V>::load(d, rd, off);
      const int doc_start = start[t];
#pragma unroll
      for (int v = 0; v < V; ++v) acc_bias[v] += d[v];
#pragma unroll
      for (int lag = 0; lag < K; ++lag) {
        float row[V];
        padded_source<IO, V, K>(p, ru, rs, list, i, lag, doc_start, c0, row);
#pragma unroll
        for (int v = 0; v < V; ++v) acc_tap[K - 1 - lag][v] = fmaf(d[v], row[v], acc_tap[K - 1 - lag][v]);
      }
    }
    ConvRow<IO, V>::store(g, rg, off);
  }

  // gradient at the carried state: row j stands at ordinal j - (K - 1) < 0
  if (K > 1 && p.dstate && ok && run == 0) {
    const rsrc_t rds = make_rsrc((IO*)p.dstate + (long long)b * (K - 1) * p.W, (unsigned)((K - 1) * p.W) * es);
#pragma unroll
    for (int j = 0; j < K - 1; ++j) {
      const int tau = j - (K - 1);
      float a[V];
#pragma unroll
      for (int v = 0; v < V; ++v) a[v] = 0.f;
#pragma unroll
      for (int lag = 1; lag < K; ++lag) {
        const int i2 = tau + lag;
        if (i2 >= 0 && i2 < n) {
          const int t2 = list[i2];
          if (start[t2] < 0) {
            float d[V];
            ConvRow<IO, V>::load(d, rd, ((unsigned)t2 * uW + (unsigned)c0) * es);
#pragma unroll
            for (int v = 0; v < V; ++v) a[v] = fmaf(d[v], tap[K - 1 - lag][v], a[v]);
          }
        }
      }
      ConvRow<IO, V>::store(a, rds, ((unsigned)j * uW + (unsigned)c0) * es);
    }
  }

  // sums of the workgroup's runs (threads without work hold zeros)
#pragma unroll
  for (int j = 0; j < K; ++j)
#pragma unroll
    for (int v = 0; v < V; ++v) red[lane_run][j * V + v][lane_vec] = acc_tap[j][v];
#pragma unroll
  for (int v = 0; v < V; ++v) red[lane_run][K * V + v][lane_vec] = acc_bias[v];
  __syncthreads();
  float* part = p.partial + ((long long)(b * run_groups + rgp) * (K + 1)) * p.W;
  for (int idx = threadIdx.x; idx < (K + 1) * V * kConvBwdVecs; idx += kConvThreads) {
    const int row = idx / kConvBwdVecs, lv = idx - row * kConvBwdVecs;   // row = j * V + v
    const int j = row / V, v = row - j * V;
    const int ch = (vg * kConvBwdVecs + lv) * V + v;
    if (ch < p.W) {
      float sum = 0.f;
#pragma unroll
      for (int q = 0; q < kConvBwdRuns; ++q) sum += red[q][row][lv];
      part[(long long)j * p.W + ch] = sum;
    }
  }
}

// ------------------------------------------------------------------------------------------
// Everything a single-token step of the recurrent block needs in front of the RG-LRU step kernel,
// in one launch (griffin/griffin.py:459-510 with one token per row): the row's position
// (previous + 1, or the one given), its flags for the step kernel (reset at position 0, inactive),
// the convolved input, the shifted convolution state and the position to carry on.  Without an
// `active` array the rows follow the all-active path (:476-487: taps masked by the position, the
// state simply shifted); with one they follow the padded path (:488-510: a document start clears
// the history first, every tap counts, an inactive row keeps its state and position and gets a
// zero input).
// ------------------------------------------------------------------------------------------
struct DecodeArgs {
  const void* u; const void* state; const void* taps; const void* bias;
  const long long* prev_pos; const long long* seg_pos; const unsigned char* active;
  void* x; void* new_state; long long* new_pos; unsigned char* flags;
  long long ldu;                                          // elements between rows of u (>= W)
  int B, W, K, nvec, vec_dtype;
};

template <typename IO, int V, int K>
__global__ __launch_bounds__(kConvThreads) void decode_prepare_kernel(DecodeArgs p) {
  typedef ConvRow<IO, V> Row;
  const long long item = (long long)blockIdx.x * kConvThreads + threadIdx.x;
  if (item >= (long long)p.B * p.nvec) return;
  const int vec = (int)(item % p.nvec), b = (int)(item / p.nvec);
  const int c0 = vec * V;
  const unsigned es = (unsigned)sizeof(IO), uW = (unsigned)p.W;
  // The step is a chain of latencies, so everything it reads is requested before anything is used: the row's
  // activity byte and positions (from a readable dummy where the caller passes none; a load under a condition sits
  // in a block of its own and waits there), then the input row and the carried rows.  The descriptors span the
  // whole tensors with the row in the lane offset: a descriptor per row differs from lane to lane, and every access
  // through one becomes a loop over the wave's distinct rows that ends in a wait for all memory operations.
  const unsigned char* active_src = p.active ? p.active + b : p.flags + b;
  const long long* before_src = p.prev_pos ? p.prev_pos + b : p.new_pos + b;
  const long long* pos_src = p.seg_pos ? p.seg_pos + b : p.new_pos + b;
  const unsigned char active_raw = *active_src;
  const long long before_raw = *before_src, pos_raw = *pos_src;
  const rsrc_t ru = make_rsrc(p.u, (unsigned)(((long long)(p.B - 1) * p.ldu + p.W) * es));
  const rsrc_t rx = make_rsrc(p.x, (unsigned)p.B * uW * es);
  const unsigned off = (unsigned)c0 * es;
  const unsigned row_x = (unsigned)b * uW * es, row_s = (unsigned)b * (unsigned)(K - 1) * uW * es;
  float cur[V], acc[V], hist[K > 1 ? K - 1 : 1][V];          // hist[j] = state row j (oldest first)
  const rsrc_t rs = make_rsrc(p.state ? p.state : p.u, p.state ? (unsigned)p.B * (unsigned)(K - 1) * uW * es : 0u);
  const typename Row::Raw cur_raw = Row::request(ru, (unsigned)((long long)b * p.ldu * es) + off);
  typename Row::Raw hist_raw[K > 1 ? K - 1 : 1];
#pragma unroll
  for (int j = 0; j < K - 1; ++j) hist_raw[j] = Row::request(rs, row_s + ((unsigned)j * uW + (unsigned)c0) * es);
  float tap[K][V], bias[V];
  conv_load_taps<V, K>(p.taps, p.bias, c0, p.vec_dtype, tap, bias);
  const bool live = p.active ? active_raw != 0 : true;
  const long long before = p.prev_pos ? before_raw : -1;
  const long long pos = p.seg_pos ? pos_raw : before + (live ? 1 : 0);
  if (vec == 0) {
    p.new_pos[b] = live ? pos : before;
    p.flags[b] = (unsigned char)((live && pos == 0 ? RGLRU_FLAG_RESET : 0u) | (live ? 0u : RGLRU_FLAG_INACTIVE));
  }
  Row::unpack(cur, cur_raw);
#pragma unroll
  for (int j = 0; j < K - 1; ++j) Row::unpack(hist[j], hist_raw[j]);
  const bool padded = p.active != nullptr;
  if (padded && live && pos == 0) {                         // griffin/griffin.py:491-492
#pragma unroll
    for (int j = 0; j < K - 1; ++j)
#pragma unroll
      for (int v = 0; v < V; ++v) hist[j][v] = 0.f;
  }
#pragma unroll
  for (int v = 0; v < V; ++v) {
    float a = bias[v];
    if (padded || pos >= 0) a = fmaf(cur[v], tap[K - 1][v], a);
#pragma unroll
    for (int lag = 1; lag < K; ++lag)
      if (padded || pos >= lag) a = fmaf(hist[K - 1 - lag][v], tap[K - 1 - lag][v], a);
    acc[v] = live ? a : 0.f;
  }
  Row::store(acc, rx, row_x + off);
  if (K > 1) {
    const rsrc_t rn = make_rsrc(p.new_state, (unsigned)p.B * (unsigned)(K - 1) * uW * es);
#pragma unroll
    for (int j = 0; j < K - 1; ++j) {
      float row[V];
#pragma unroll
      for (int v = 0; v < V; ++v) {
        const float shifted = (j + 1 < K - 1) ? hist[j + 1 < K - 1 ? j + 1 : 0][v] : cur[v];
        row[v] = live ? shifted : hist[j][v];
      }
      Row::store(row, rn, row_s + ((unsigned)j * uW + (unsigned)c0) * es);
    }
  }
}

// ------------------------------------------------------------------------------------------
// Output gate: out = h * gelu_tanh(v) and its reverse mode, flat over n elements.
//   gelu_tanh(v) = v/2 * (1 + tanh(u)),  u = sqrt(2/pi) * (v + 0.044715 v^3)
// A thread handles 16-byte vectors in a grid-stride loop, four vectors requested at a time.
// ------------------------------------------------------------------------------------------
constexpr int kGateThreads = 256;
constexpr int kGateBatch = 4;

struct GateArgs {
  const void* h; const void* v; const void* dout; void* out; void* dh; void* dv; long long n;
  long long ld_dv; int row_vecs; unsigned dv_bytes;         // backward with dv rows ld_dv elements apart (row_vecs vectors per row); 0: flat
  unsigned row_magic;                                       // ceil(2^32 / row_vecs) where (vectors + row_vecs) * row_vecs < 2^32 (the multiply-high is then exact), else 0
};

template <typename IO, int V, bool BACKWARD>
__global__ __launch_bounds__(kGateThreads) void gelu_gate_kernel(GateArgs p) {
  typedef ConvRow<IO, V> Row;
  const long long nvec = p.n / V;
  const long long stride = (long long)gridDim.x * kGateThreads;
  // descriptors cover at most 2 GiB: the loop walks windows of that size
  constexpr long long WIN = (1ll << 30) / (long long)sizeof(IO) / V * V;    // elements per window (1 GiB)
  for (long long w0 = 0; w0 < p.n; w0 += WIN) {
    const long long wn = (p.n - w0) < WIN ? (p.n - w0) : WIN;
    const unsigned bytes = (unsigned)(wn * (long long)sizeof(IO));
    const rsrc_t rh = make_rsrc((const IO*)p.h + w0, bytes);
    const rsrc_t rv = make_rsrc((const IO*)p.v + w0, bytes);
    const rsrc_t rd = make_rsrc(BACKWARD ? (const IO*)p.dout + w0 : (const IO*)p.h, BACKWARD ? bytes : 0u);
    const rsrc_t ro = make_rsrc(BACKWARD ? (IO*)p.dh + w0 : (IO*)p.out + w0, bytes);
    // dv is flat like the rest, or has rows of its own stride (then the tensor is one window)
    const bool dv_rows = BACKWARD && p.row_vecs > 0;
    const rsrc_t rw = make_rsrc(BACKWARD ? (dv_rows ? (IO*)p.dv : (IO*)p.dv + w0) : (IO*)p.out, BACKWARD ? (dv_rows ? p.dv_bytes : bytes) : 0u);
    const long long wvec = (wn + V - 1) / V;
    (void)nvec;
    for (long long i0 = (long long)blockIdx.x * kGateThreads + threadIdx.x; i0 < wvec; i0 += stride * kGateBatch) {
      typename Row::Raw raw_h[kGateBatch], raw_v[kGateBatch], raw_d[kGateBatch];
#pragma unroll
      for (int j = 0; j < kGateBatch; ++j) {
        const long long i = i0 + (long long)j * stride;
        const unsigned off = i < wvec ? (unsigned)(i * V * (long long)sizeof(IO)) : kOutOfRange;
        raw_h[j] = Row::request(rh, off);
        raw_v[j] = Row::request(rv, off);
        if (BACKWARD) raw_d[j] = Row::request(rd, off);
      }
#pragma unroll
      for (int j = 0; j < kGateBatch; ++j) {
        const long long i = i0 + (long long)j * stride;
        const unsigned off = i < wvec ? (unsigned)(i * V * (long long)sizeof(IO)) : kOutOfRange;
        float h[V], v[V], a[V], b[V];
        Row::unpack(h, raw_h[j]);
        Row::unpack(v, raw_v[j]);
        if (BACKWARD) {
          float d[V];
          Row::unpack(d, raw_d[j]);
#pragma unroll
          for (int e = 0; e < V; ++e) {
            const GeluParts g = gelu_tanh_parts(v[e]);
            a[e] = d[e] * g.gelu;
            b[e] = (d[e] * h[e]) * g.dgelu;
          }
          Row::store(a, ro, off);
          unsigned off_dv = off;
          if (dv_rows && i < wvec) {
            const unsigned row = p.row_magic ? __umulhi((unsigned)i, p.row_magic) : (unsigned)i / (unsigned)p.row_vecs;
            const unsigned cv = (unsigned)i - row * (unsigned)p.row_vecs;
            off_dv = (row * (unsigned)p.ld_dv + cv * V) * (unsigned)sizeof(IO);
          }
          Row::store(b, rw, off_dv);
        } else {
#pragma unroll
          for (int e = 0; e < V; ++e) a[e] = h[e] * gelu_tanh_parts(v[e]).gelu;
          Row::store(a, ro, off);
        }
      }
    }
  }
}

static int gate_launch(const char* who, bool backward, GateArgs a, int dtype, void* stream) {
  if (dtype != RGLRU_F32 && dtype != RGLRU_BF16) return fail(RGLRU_E_ARG, "%s: dtype must be RGLRU_F32 or RGLRU_BF16, got %d", who, dtype);
  if (a.n <= 0) return fail(RGLRU_E_ARG, "%s: empty tensor", who);
  const int v = dtype == RGLRU_BF16 ? 8 : 4;
  const bool vec = conv_vector_ok(a.n, dtype, {a.h, a.v, a.dout, a.out, a.dh, a.dv});
  const long long items = vec ? (a.n + v - 1) / v : a.n;
  long long blocks = (items + (long long)kGateThreads * kGateBatch - 1) / ((long long)kGateThreads * kGateBatch);
  const long long cap = (long long)num_compute_units() * 16;
  if (blocks > cap) blocks = cap;
  if (blocks < 1) blocks = 1;
  dim3 grid((unsigned)blocks);
  hipStream_t s = (hipStream_t)stream;
#define RGLRU_GATE_LAUNCH(IO, V)                                                                      \
  do {                                                                                                \
    if (backward) hipLaunchKernelGGL((gelu_gate_kernel<IO, V, true>), grid, dim3(kGateThreads), 0, s, a);  \
    else hipLaunchKernelGGL((gelu_gate_kernel<IO, V, false>), grid, dim3(kGateThreads), 0, s, a);     \
  } while (0)
  if (dtype == RGLRU_BF16) { if (vec) RGLRU_GATE_LAUNCH(__bf16, 8); else RGLRU_GATE_LAUNCH(__bf16, 1); }
  else { if (vec) RGLRU_GATE_LAUNCH(float, 4); else RGLRU_GATE_LAUNCH(float, 1); }
#undef RGLRU_GATE_LAUNCH
  return check_launch(who);
}


// ------------------------------------------------------------------------------------------
// RMSNorm in front of the block (griffin/griffin.py:68-80): y = x * rsqrt(mean(x^2) + eps) * (1 + g)
// over the last axis, and its reverse mode.  One wave per row at a time (grid-stride over rows); a
// lane holds the row's 16-byte vectors lane, lane + 64, ... in registers, so a row is read once.
//   dx = inv * (w dy - x inv^2 mean(w dy x)),  w = 1 + g,  inv = rsqrt(mean(x^2) + eps)
//   dg = sum over rows of dy x inv            (per-wave partial sums, reduced by a second kernel)
// ------------------------------------------------------------------------------------------
constexpr int kNormThreads = 256;
constexpr int kNormSlots = 16;                 // most vectors per lane: rows of up to 64 * 16 vectors (1, 2, 4, 8 or 16 are compiled)

struct NormArgs {
  const void* x; const void* g; const void* dy; const float* inv_in;
  void* y; void* dx; float* inv_out; float* partial;
  long long rows; int D, nvec, vec_dtype; float eps;
};

RGLRU_DEVICE float wave_sum(float v) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, 64);
  return v;
}

template <typename IO, int V, int SLOTS, bool BACKWARD>
__global__ __launch_bounds__(kNormThreads) void rmsnorm_kernel(NormArgs p) {
  typedef ConvRow<IO, V> Row;
  constexpr int kNormSlots = SLOTS;                        // shadows the global maximum inside the kernel
  const int lane = threadIdx.x & 63;
  const long long wave = (long long)blockIdx.x * (kNormThreads / 64) + (threadIdx.x >> 6);
  const long long n_waves = (long long)gridDim.x * (kNormThreads / 64);
  const unsigned row_bytes = (unsigned)p.D * (unsigned)sizeof(IO);
  // The widest backward variant would hold x, dy, the scale and its gradient sums of 128 elements per lane, more
  // than the register file: there the scale is fetched again for every row (it stays in the cache).
  constexpr bool kHoldScale = !(BACKWARD && SLOTS * V > 64);
  float w[kHoldScale ? kNormSlots : 1][V], dg[kNormSlots][V];
  auto scale_of = [&](int s, float (&out)[V]) {
    const bool has = lane + 64 * s < p.nvec;
    float g[V];
    conv_params<V>(p.g, has ? (long long)(lane + 64 * s) * V : 0, p.vec_dtype, g);
#pragma unroll
    for (int v = 0; v < V; ++v) out[v] = has ? 1.0f + g[v] : 0.f;
  };
#pragma unroll
  for (int s = 0; s < kNormSlots; ++s) {
    if constexpr (kHoldScale) scale_of(s, w[s]);
#pragma unroll
    for (int v = 0; v < V; ++v) dg[s][v] = 0.f;
  }
  const float inv_d = 1.0f / (float)p.D;
  for (long long row = wave; row < p.rows; row += n_waves) {
    const rsrc_t rx = make_rsrc((const IO*)p.x + row * p.D, row_bytes);
    typename Row::Raw raw_x[kNormSlots], raw_d[kNormSlots];
#pragma unroll
    for (int s = 0; s < kNormSlots; ++s) {
      const unsigned off = (lane + 64 * s < p.nvec) ? (unsigned)((lane + 64 * s) * V) * (unsigned)sizeof(IO) : kOutOfRange;
      raw_x[s] = Row::request(rx, off);
      if (BACKWARD) raw_d[s] = Row::request(make_rsrc((const IO*)p.dy + row * p.D, row_bytes), off);
    }
    // the row as floats, except in the widest backward variant, which keeps the rows as loaded and converts a
    // slot each time it needs it (x, dy and the gradient sums as floats would not fit the registers)
    float x[kHoldScale ? kNormSlots : 1][V];
    auto x_of = [&](int s, float (&out)[V]) {
      if constexpr (kHoldScale) {
#pragma unroll
        for (int v = 0; v < V; ++v) out[v] = x[s][v];
      } else {
        Row::unpack(out, raw_x[s]);
      }
    };
    float acc = 0.f;
#pragma unroll
    for (int s = 0; s < kNormSlots; ++s) {
      float xs[V];
      Row::unpack(xs, raw_x[s]);
#pragma unroll
      for (int v = 0; v < V; ++v) {
        if constexpr (kHoldScale) x[s][v] = xs[v];
        acc = fmaf(xs[v], xs[v], acc);
      }
    }
    if (!BACKWARD) {
      const float inv = __builtin_amdgcn_rsqf(wave_sum(acc) * inv_d + p.eps);
      if (lane == 0 && p.inv_out) p.inv_out[row] = inv;
      const rsrc_t ry = make_rsrc((IO*)p.y + row * p.D, row_bytes);
#pragma unroll
      for (int s = 0; s < kNormSlots; ++s) {
        float y[V];
#pragma unroll
        for (int v = 0; v < V; ++v) y[v] = x[s][v] * inv * w[s][v];
        Row::store(y, ry, (lane + 64 * s < p.nvec) ? (unsigned)((lane + 64 * s) * V) * (unsigned)sizeof(IO) : kOutOfRange);
      }
    } else {
      const float inv = p.inv_in[row];
      float d[kHoldScale ? kNormSlots : 1][V];
      float dot = 0.f;
#pragma unroll
      for (int s = 0; s < kNormSlots; ++s) {
        float ds[V], xs[V];
        Row::unpack(ds, raw_d[s]);
        x_of(s, xs);
        float ws[V];
        if constexpr (kHoldScale) {
#pragma unroll
          for (int v = 0; v < V; ++v) ws[v] = w[s][v];
        } else {
          scale_of(s, ws);
        }
#pragma unroll
        for (int v = 0; v < V; ++v) {
          dg[s][v] = fmaf(ds[v] * inv, xs[v], dg[s][v]);
          ds[v] *= ws[v];
          if constexpr (kHoldScale) d[s][v] = ds[v];
          dot = fmaf(ds[v], xs[v], dot);
        }
      }
      const float k = wave_sum(dot) * inv_d * inv * inv;
      const rsrc_t rdx = make_rsrc((IO*)p.dx + row * p.D, row_bytes);
#pragma unroll
      for (int s = 0; s < kNormSlots; ++s) {
        float g[V], xs[V], ds[V];
        x_of(s, xs);
        if constexpr (kHoldScale) {
#pragma unroll
          for (int v = 0; v < V; ++v) ds[v] = d[s][v];
        } else {
          float ws[V];
          Row::unpack(ds, raw_d[s]);
          scale_of(s, ws);
#pragma unroll
          for (int v = 0; v < V; ++v) ds[v] *= ws[v];
        }
#pragma unroll
        for (int v = 0; v < V; ++v) g[v] = inv * fmaf(-k, xs[v], ds[v]);
        Row::store(g, rdx, (lane + 64 * s < p.nvec) ? (unsigned)((lane + 64 * s) * V) * (unsigned)sizeof(IO) : kOutOfRange);
      }
    }
  }
  if constexpr (BACKWARD) {
    // the workgroup's waves add their sums up in LDS, one after the other; one partial row per workgroup
    __shared__ float red[SLOTS * 64 * V];
    for (int turn = 0; turn < kNormThreads / 64; ++turn) {
      if ((int)(threadIdx.x >> 6) == turn) {
#pragma unroll
        for (int s = 0; s < kNormSlots; ++s)
#pragma unroll
          for (int v = 0; v < V; ++v) {
            const int at = (lane + 64 * s) * V + v;
            red[at] = turn == 0 ? dg[s][v] : red[at] + dg[s][v];
          }
      }
      __syncthreads();
    }
    float* part = p.partial + (long long)blockIdx.x * p.D;
    for (int c = threadIdx.x; c < p.D; c += kNormThreads) part[c] = red[c];
  }
}

// Sums the per-workgroup partial rows: a workgroup owns 32 columns, eight threads share a column.
struct NormFinishArgs { const float* partial; void* dg; int D, slots, grad_dtype; };
__global__ __launch_bounds__(256) void rmsnorm_finish_kernel(NormFinishArgs p) {
  __shared__ float red[8][32];
  const int col = threadIdx.x & 31, share = threadIdx.x >> 5;
  const int c = blockIdx.x * 32 + col;
  float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
  if (c < p.D) {
    // sixteen loads in flight per thread: the kernel is a chain of memory round trips, not of bytes
    int n = share;
    for (; n + 120 < p.slots; n += 128) {
      float v[16];
#pragma unroll
      for (int u = 0; u < 16; ++u) v[u] = p.partial[(long long)(n + 8 * u) * p.D + c];
#pragma unroll
      for (int u = 0; u < 16; u += 4) { s0 += v[u]; s1 += v[u + 1]; s2 += v[u + 2]; s3 += v[u + 3]; }
    }
    for (; n < p.slots; n += 8) s0 += p.partial[(long long)n * p.D + c];
  }
  red[share][col] = (s0 + s1) + (s2 + s3);
  __syncthreads();
  if (share == 0 && c < p.D) {
    float s = 0.f;
#pragma unroll
    for (int q = 0; q < 8; ++q) s += red[q][col];
    if (p.grad_dtype == RGLRU_BF16) ((__bf16*)p.dg)[c] = (__bf16)s; else ((float*)p.dg)[c] = s;
  }
}

// Column sums of a [rows, D] matrix (the bias gradient of a Linear layer: db = sum over rows of dy).  A
// workgroup owns 32 vectors of columns and a slot of rows; its 8 row lanes stride through the slot with all
// their loads in flight, add up in LDS and leave one partial row per slot, which rmsnorm_finish_kernel
// sums in fixed order.
constexpr int kColsumVecs = 32, kColsumLanes = 8, kColsumRowsPerLane = 8;
struct ColsumArgs { const void* x; float* partial; long long rows; int D, nvec, vec_groups; };
template <typename IO, int V>
__global__ __launch_bounds__(256) void colsum_kernel(ColsumArgs p) {
  __shared__ float red[kColsumLanes][V][kColsumVecs + 1];
  const int lv = threadIdx.x % kColsumVecs, rl = threadIdx.x / kColsumVecs;
  const int vg = blockIdx.x % p.vec_groups;
  const long long slot = blockIdx.x / p.vec_groups;
  const int vec = vg * kColsumVecs + lv;
  const long long row0 = slot * (kColsumLanes * kColsumRowsPerLane) + rl;
  float acc[V];
#pragma unroll
  for (int v = 0; v < V; ++v) acc[v] = 0.f;
  if (vec < p.nvec) {
    const unsigned es = (unsigned)sizeof(IO);
    // the slot's rows through one descriptor: rows past the end read as zero
    const long long first = slot * (kColsumLanes * kColsumRowsPerLane);
    const long long left = p.rows - first;
    const unsigned rows_here = (unsigned)(left < kColsumLanes * kColsumRowsPerLane ? left : kColsumLanes * kColsumRowsPerLane);
    const rsrc_t r = make_rsrc((const IO*)p.x + first * p.D, rows_here * (unsigned)p.D * es);
    float row[kColsumRowsPerLane][V];
#pragma unroll
    for (int i = 0; i < kColsumRowsPerLane; ++i)
      ConvRow<IO, V>::load(row[i], r, ((unsigned)(rl + kColsumLanes * i) * (unsigned)p.D + (unsigned)vec * V) * es);
#pragma unroll
    for (int i = 0; i < kColsumRowsPerLane; ++i)
#pragma unroll
      for (int v = 0; v < V; ++v) acc[v] += row[i][v];
  }
  (void)row0;
#pragma unroll
  for (int v = 0; v < V; ++v) red[rl][v][lv] = acc[v];
  __syncthreads();
  for (int idx = threadIdx.x; idx < V * kColsumVecs; idx += 256) {
    const int v = idx / kColsumVecs, l = idx - v * kColsumVecs;
    const int c = (vg * kColsumVecs + l) * V + v;
    if (c < p.D) {
      float sum = 0.f;
#pragma unroll
      for (int q = 0; q < kColsumLanes; ++q) sum += red[q][v][l];
      p.partial[slot * p.D + c] = sum;
    }
  }
}

// Sum of `sets` arrays of n elements each, x[s * n + i] -> out[i]: what is left of a weight gradient whose
// contraction over the tokens was split into a batch of shorter GEMMs.  A thread owns V consecutive elements and
// asks for up to eight sets at once; fp32 accumulation in the order of the sets.
struct SumSetsArgs { const void* x; void* out; long long n; int sets; };
template <typename IO, int V>
__global__ __launch_bounds__(256) void sum_sets_kernel(SumSetsArgs p) {
  typedef typename ConvRow<IO, V>::Raw Raw;
  const long long i = ((long long)blockIdx.x * 256 + threadIdx.x) * V;
  if (i >= p.n) return;
  const IO* src = (const IO*)p.x + i;
  float acc[V];
#pragma unroll
  for (int v = 0; v < V; ++v) acc[v] = 0.f;
  for (int s0 = 0; s0 < p.sets; s0 += 8) {
    Raw raw[8];
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      const int s = s0 + q < p.sets ? s0 + q : p.sets - 1;   // a set past the last is asked again and not added
      if constexpr (V == 1) raw[q] = (float)src[(long long)s * p.n];
      else raw[q] = *reinterpret_cast<const Raw*>(src + (long long)s * p.n);
    }
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      float v[V];
      ConvRow<IO, V>::unpack(v, raw[q]);
      if (s0 + q < p.sets) {
#pragma unroll
        for (int e = 0; e < V; ++e) acc[e] += v[e];
      }
    }
  }
  IO* dst = (IO*)p.out + i;
  if constexpr (V == 1) {
    dst[0] = (IO)acc[0];
  } else {
    typedef IO Vec __attribute__((ext_vector_type(V)));
    Vec o;
#pragma unroll
    for (int e = 0; e < V; ++e) o[e] = (IO)acc[e];
    *reinterpret_cast<Vec*>(dst) = o;
  }
}

template <typename IO, int V, bool BACKWARD>
static void norm_launch(int nvec, dim3 grid, hipStream_t s, const NormArgs& a) {
  const int slots = (nvec + 63) / 64;
  if (slots <= 1) hipLaunchKernelGGL((rmsnorm_kernel<IO, V, 1, BACKWARD>), grid, dim3(kNormThreads), 0, s, a);
  else if (slots <= 2) hipLaunchKernelGGL((rmsnorm_kernel<IO, V, 2, BACKWARD>), grid, dim3(kNormThreads), 0, s, a);
  else if (slots <= 4) hipLaunchKernelGGL((rmsnorm_kernel<IO, V, 4, BACKWARD>), grid, dim3(kNormThreads), 0, s, a);
  else if (slots <= 8) hipLaunchKernelGGL((rmsnorm_kernel<IO, V, 8, BACKWARD>), grid, dim3(kNormThreads), 0, s, a);
  else hipLaunchKernelGGL((rmsnorm_kernel<IO, V, 16, BACKWARD>), grid, dim3(kNormThreads), 0, s, a);
}

static int norm_grid(long long rows) {
  long long blocks = (rows + (kNormThreads / 64) - 1) / (kNormThreads / 64);
  const long long cap = (long long)num_compute_units() * 4;
  if (blocks > cap) blocks = cap;
  return (int)(blocks < 1 ? 1 : blocks);
}

static int norm_check(const char* who, int64_t rows, int64_t D, int dtype, int vec_dtype, bool* vec, int* nvec,
                      std::initializer_list<const void*> ptrs) {
  if (dtype != RGLRU_F32 && dtype != RGLRU_BF16) return fail(RGLRU_E_ARG, "%s: dtype must be RGLRU_F32 or RGLRU_BF16, got %d", who, dtype);
  if (vec_dtype != RGLRU_F32 && vec_dtype != RGLRU_BF16) return fail(RGLRU_E_ARG, "%s: unknown parameter dtype %d", who, vec_dtype);
  if (rows <= 0 || D <= 0) return fail(RGLRU_E_ARG, "%s: empty shape rows=%lld D=%lld", who, (long long)rows, (long long)D);
  *vec = conv_vector_ok(D, dtype, ptrs);
  const int v = *vec ? (dtype == RGLRU_BF16 ? 8 : 4) : 1;
  *nvec = (int)(D / v);
  if (*nvec > 64 * kNormSlots) return fail(RGLRU_E_UNSUPPORTED, "%s: rows of %lld elements exceed the supported %d", who, (long long)D, 64 * kNormSlots * v);
  if (rows * D >= (1ll << 40)) return fail(RGLRU_E_UNSUPPORTED, "%s: tensor too large", who);
  return RGLRU_OK;
}

}  // namespace rglru

using namespace rglru;

extern "C" {

int rglru_hip_conv_max_kernel_size(void) { return kConvMaxTaps; }

int rglru_hip_conv_fwd(const void* u, const void* state, const void* taps, const void* bias,
                       const int64_t* segment_pos, void* out, void* new_state,
                       int64_t B, int64_t T, int64_t W, int64_t K, int dtype, int vec_dtype, void* stream) {
  int rc = conv_check("conv_fwd", B, T, W, K, dtype, vec_dtype);
  if (rc) return rc;
  if (!u || !taps || !segment_pos || !out) return fail(RGLRU_E_ARG, "conv_fwd: null pointer");
  ConvArgs a;
  memset(&a, 0, sizeof(a));
  a.u = u; a.state = state; a.taps = taps; a.bias = bias; a.segpos = (const long long*)segment_pos;
  a.out = out; a.new_state = new_state;
  a.B = (int)B; a.T = (int)T; a.W = (int)W; a.K = (int)K; a.vec_dtype = vec_dtype;
  const bool vec = conv_vector_ok(W, dtype, {u, state, out, new_state});
  a.nvec = (int)(vec ? W / (dtype == RGLRU_BF16 ? 8 : 4) : W);
  a.runs = (int)((T + kConvRunFwd - 1) / kConvRunFwd);
  const long long blocks = B * conv_blocks_per_seq(a.runs, a.nvec);
  if (blocks >= (1ll << 31)) return fail(RGLRU_E_UNSUPPORTED, "conv_fwd: tensor too large");
  dim3 grid((unsigned)blocks);
  hipStream_t s = (hipStream_t)stream;
  RGLRU_CONV_DISPATCH(conv_fwd_kernel, dtype, vec, grid, s, a);
  return check_launch("conv_fwd");
}

size_t rglru_hip_conv_scratch_bytes(int64_t B, int64_t T, int64_t W, int64_t K) {
  if (B <= 0 || T <= 0 || W <= 0 || K < 1 || K > kConvMaxTaps) return 0;
  const int64_t runs = (T + kConvRunBwd - 1) / kConvRunBwd;
  const int64_t run_groups = (runs + kConvBwdRuns - 1) / kConvBwdRuns;
  return (size_t)(B * run_groups * (K + 1) * W * 4);
}

int rglru_hip_conv_bwd(const void* u, const void* state, const void* taps, const int64_t* segment_pos,
                       const void* dout, void* scratch, void* du, int64_t du_stride, void* dstate, void* dtaps, void* dbias,
                       int64_t B, int64_t T, int64_t W, int64_t K, int dtype, int vec_dtype, int grad_dtype,
                       void* stream) {
  int rc = conv_check("conv_bwd", B, T, W, K, dtype, vec_dtype);
  if (rc) return rc;
  if (du_stride == 0) du_stride = W;
  if (du_stride < W) return fail(RGLRU_E_ARG, "conv_bwd: du_stride %lld is smaller than the width %lld", (long long)du_stride, (long long)W);
  rc = conv_check("conv_bwd", B, T, du_stride, K, dtype, vec_dtype);      // the strided rows obey the same per-sequence limit
  if (rc) return rc;
  if (grad_dtype != RGLRU_F32 && grad_dtype != RGLRU_BF16) return fail(RGLRU_E_ARG, "conv_bwd: unknown gradient dtype %d", grad_dtype);
  if (!u || !taps || !segment_pos || !dout || !scratch || !du) return fail(RGLRU_E_ARG, "conv_bwd: null pointer");
  ConvArgs a;
  memset(&a, 0, sizeof(a));
  a.u = u; a.state = state; a.taps = taps; a.segpos = (const long long*)segment_pos;
  a.dout = dout; a.du = du; a.dstate = dstate; a.partial = (float*)scratch; a.ld_du = du_stride;
  a.B = (int)B; a.T = (int)T; a.W = (int)W; a.K = (int)K; a.vec_dtype = vec_dtype;
  const bool vec = conv_vector_ok(W, dtype, {u, state, dout, du, dstate}) && (du_stride * (dtype == RGLRU_BF16 ? 2 : 4)) % 16 == 0;
  a.nvec = (int)(vec ? W / (dtype == RGLRU_BF16 ? 8 : 4) : W);
  a.runs = (int)((T + kConvRunBwd - 1) / kConvRunBwd);
  const long long run_groups = (a.runs + kConvBwdRuns - 1) / kConvBwdRuns;
  const long long vec_groups = (a.nvec + kConvBwdVecs - 1) / kConvBwdVecs;
  if (B * run_groups * vec_groups >= (1ll << 31)) return fail(RGLRU_E_UNSUPPORTED, "conv_bwd: tensor too large");
  dim3 grid((unsigned)(B * run_groups * vec_groups));
  hipStream_t s = (hipStream_t)stream;
  RGLRU_CONV_DISPATCH(conv_bwd_kernel, dtype, vec, grid, s, a);
  rc = check_launch("conv_bwd");
  if (rc) return rc;
  if (dtaps || dbias) {
    ConvFinishArgs f;
    f.partial = a.partial; f.dtaps = dtaps; f.dbias = dbias; f.W = (int)W; f.K = (int)K;
    f.slots = (int)(B * run_groups); f.grad_dtype = grad_dtype;
    const long long n = (long long)(K + 1) * W;
    hipLaunchKernelGGL(conv_finish_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, f);
    rc = check_launch("conv_bwd finish");
  }
  return rc;
}

// Host-side view of the index (see padded_index): the positions of prefix rows and the per-row words.
static const long long* padded_positions(const void* scratch) { return (const long long*)scratch; }
static const int* padded_rows(const void* scratch, int64_t B, int64_t T) { return (const int*)scratch + 5 * B * T; }

int rglru_hip_conv_padded_bwd(const void* u, const void* state, const void* taps,
                              const int64_t* segment_pos, const uint8_t* active, const void* dout,
                              void* index_scratch, void* scratch, void* du, void* dstate, void* dtaps, void* dbias,
                              int64_t B, int64_t T, int64_t W, int64_t K, int dtype, int vec_dtype, int grad_dtype,
                              void* stream) {
  int rc = conv_check("conv_padded_bwd", B, T, W, K, dtype, vec_dtype);
  if (rc) return rc;
  if (grad_dtype != RGLRU_F32 && grad_dtype != RGLRU_BF16) return fail(RGLRU_E_ARG, "conv_padded_bwd: unknown gradient dtype %d", grad_dtype);
  if (!u || !taps || !segment_pos || !active || !dout || !index_scratch || !scratch || !du)
    return fail(RGLRU_E_ARG, "conv_padded_bwd: null pointer");
  if ((uintptr_t)index_scratch % 8) return fail(RGLRU_E_ARG, "conv_padded_bwd: index scratch must be 8-byte aligned");
  if (B * T >= (1ll << 29)) return fail(RGLRU_E_UNSUPPORTED, "conv_padded_bwd: tensor too large");
  PaddedArgs a;
  memset(&a, 0, sizeof(a));
  a.u = u; a.state = state; a.taps = taps; a.segpos = (const long long*)segment_pos; a.active = active;
  a.scratch = (int*)index_scratch; a.dout = dout; a.du = du; a.dstate = dstate; a.partial = (float*)scratch;
  a.B = (int)B; a.T = (int)T; a.W = (int)W; a.K = (int)K; a.vec_dtype = vec_dtype;
  const bool vec = conv_vector_ok(W, dtype, {u, state, dout, du, dstate});
  a.nvec = (int)(vec ? W / (dtype == RGLRU_BF16 ? 8 : 4) : W);
  a.runs = (int)((T + kConvRunBwd - 1) / kConvRunBwd);
  hipStream_t s = (hipStream_t)stream;
  hipLaunchKernelGGL(conv_padded_index_kernel, dim3((unsigned)B), dim3(64), 0, s, a);
  rc = check_launch("conv_padded_bwd index");
  if (rc) return rc;
  const long long run_groups = (a.runs + kConvBwdRuns - 1) / kConvBwdRuns;
  const long long vec_groups = (a.nvec + kConvBwdVecs - 1) / kConvBwdVecs;
  if (B * run_groups * vec_groups >= (1ll << 31)) return fail(RGLRU_E_UNSUPPORTED, "conv_padded_bwd: tensor too large");
  dim3 grid((unsigned)(B * run_groups * vec_groups));
  RGLRU_CONV_DISPATCH(conv_padded_bwd_kernel, dtype, vec, grid, s, a);
  rc = check_launch("conv_padded_bwd");
  if (rc) return rc;
  {
    // rows whose active tokens are a prefix: the dense kernel, same grid and same partial rows
    ConvArgs d;
    memset(&d, 0, sizeof(d));
    d.u = u; d.state = state; d.taps = taps; d.dout = dout; d.du = du; d.dstate = dstate; d.partial = a.partial;
    d.ld_du = W; d.segpos = padded_positions(index_scratch); d.rows = padded_rows(index_scratch, B, T);
    d.B = (int)B; d.T = (int)T; d.W = (int)W; d.K = (int)K; d.vec_dtype = vec_dtype; d.nvec = a.nvec; d.runs = a.runs;
    RGLRU_CONV_DISPATCH(conv_bwd_kernel, dtype, vec, grid, s, d);
    rc = check_launch("conv_padded_bwd prefix rows");
    if (rc) return rc;
  }
  if (dtaps || dbias) {
    ConvFinishArgs f;
    f.partial = a.partial; f.dtaps = dtaps; f.dbias = dbias; f.W = (int)W; f.K = (int)K;
    f.slots = (int)(B * run_groups); f.grad_dtype = grad_dtype;
    const long long n = (long long)(K + 1) * W;
    hipLaunchKernelGGL(conv_finish_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, f);
    rc = check_launch("conv_padded_bwd finish");
  }
  return rc;
}

// Flag bytes of the block forward from the token positions: reset where a document starts, and in bits 2-3
// the number of convolution lags that reach in front of the document, 3 - min(position, 3).
__global__ __launch_bounds__(256) void block_flags_kernel(const long long* pos, unsigned char* flags, long long n) {
  const long long stride = (long long)gridDim.x * 256;
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) {
    const long long p = pos[i];
    const unsigned near = p < 0 ? 3u : p < 3 ? (unsigned)(3 - p) : 0u;
    flags[i] = (unsigned char)((p == 0 ? RGLRU_FLAG_RESET : 0u) | (near << 2));
  }
}

int rglru_hip_block_flags(const int64_t* segment_pos, uint8_t* flags, int64_t n, void* stream) {
  if (!segment_pos || !flags) return fail(RGLRU_E_ARG, "block_flags: null pointer");
  if (n <= 0) return fail(RGLRU_E_ARG, "block_flags: empty tensor");
  long long blocks = (n + 255) / 256; if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(block_flags_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                     (const long long*)segment_pos, (unsigned char*)flags, (long long)n);
  return check_launch("block_flags");
}

int rglru_hip_gelu_gate_fwd(const void* h, const void* v, void* out, int64_t n, int dtype, void* stream) {
  if (!h || !v || !out) return fail(RGLRU_E_ARG, "gelu_gate_fwd: null pointer");
  GateArgs a;
  memset(&a, 0, sizeof(a));
  a.h = h; a.v = v; a.out = out; a.n = n;
  return gate_launch("gelu_gate_fwd", false, a, dtype, stream);
}

int rglru_hip_gelu_gate_bwd(const void* dout, const void* h, const void* v, void* dh, void* dv,
                            int64_t n, int64_t W, int64_t dv_stride, int dtype, void* stream) {
  if (!dout || !h || !v || !dh || !dv) return fail(RGLRU_E_ARG, "gelu_gate_bwd: null pointer");
  GateArgs a;
  memset(&a, 0, sizeof(a));
  a.h = h; a.v = v; a.dout = dout; a.dh = dh; a.dv = dv; a.n = n;
  if (dv_stride != 0 && dv_stride != W) {
    if (dtype != RGLRU_F32 && dtype != RGLRU_BF16) return fail(RGLRU_E_ARG, "gelu_gate_bwd: dtype must be RGLRU_F32 or RGLRU_BF16, got %d", dtype);
    if (W <= 0 || n <= 0 || n % W || dv_stride < W) return fail(RGLRU_E_ARG, "gelu_gate_bwd: n = %lld is not rows of W = %lld elements, or dv_stride %lld < W", (long long)n, (long long)W, (long long)dv_stride);
    const int64_t es = dtype == RGLRU_BF16 ? 2 : 4, rows = n / W;
    if (rows * dv_stride * es >= (1ll << 31) || n * es > (1ll << 30)) return fail(RGLRU_E_UNSUPPORTED, "gelu_gate_bwd: a strided dv must stay below 2 GiB");
    const int vlen = dtype == RGLRU_BF16 ? 8 : 4;
    const bool vec = conv_vector_ok(n, dtype, {h, v, dout, dh, dv}) && W % vlen == 0 && (dv_stride * es) % 16 == 0;
    // rows of 16-byte vectors, or single elements: the launch below takes the vector kernel exactly when `vec` holds
    if (!vec && conv_vector_ok(n, dtype, {h, v, dout, dh, dv})) return fail(RGLRU_E_UNSUPPORTED, "gelu_gate_bwd: a strided dv needs W and dv_stride in whole 16-byte vectors");
    a.ld_dv = dv_stride; a.row_vecs = (int)(vec ? W / vlen : W);
    a.dv_bytes = (unsigned)(((rows - 1) * dv_stride + W) * es);
    const long long vectors = rows * a.row_vecs;
    if (a.row_vecs > 1 && (vectors + a.row_vecs) * a.row_vecs < (1ll << 32)) a.row_magic = (unsigned)(((1ull << 32) + a.row_vecs - 1) / a.row_vecs);
  }
  return gate_launch("gelu_gate_bwd", true, a, dtype, stream);
}

int rglru_hip_decode_prepare(const void* u, int64_t u_stride, const void* conv_state, const void* taps, const void* bias,
                             const int64_t* prev_pos, const int64_t* segment_pos, const uint8_t* active,
                             void* x, void* new_conv_state, int64_t* new_pos, uint8_t* flags,
                             int64_t B, int64_t W, int64_t K, int dtype, int vec_dtype, void* stream) {
  int rc = conv_check("decode_prepare", B, 1, W, K, dtype, vec_dtype);
  if (rc) return rc;
  if (!u || !taps || !x || !new_pos || !flags || (K > 1 && !new_conv_state))
    return fail(RGLRU_E_ARG, "decode_prepare: null pointer");
  if (u_stride == 0) u_stride = W;
  if (u_stride < W) return fail(RGLRU_E_ARG, "decode_prepare: row stride %lld of u is smaller than the width %lld", (long long)u_stride, (long long)W);
  // the kernel addresses whole tensors through one descriptor each, with 32-bit offsets
  if (B * u_stride * 4 >= (1ll << 32) || B * (K > 1 ? K - 1 : 1) * W * 4 >= (1ll << 32))
    return fail(RGLRU_E_UNSUPPORTED, "decode_prepare: tensors of 4 GiB or more");
  DecodeArgs a;
  memset(&a, 0, sizeof(a));
  a.u = u; a.state = conv_state; a.taps = taps; a.bias = bias;
  a.prev_pos = (const long long*)prev_pos; a.seg_pos = (const long long*)segment_pos; a.active = active;
  a.x = x; a.new_state = new_conv_state; a.new_pos = (long long*)new_pos; a.flags = flags;
  a.B = (int)B; a.W = (int)W; a.K = (int)K; a.vec_dtype = vec_dtype; a.ldu = u_stride;
  const bool vec = conv_vector_ok(W, dtype, {u, conv_state, x, new_conv_state}) &&
                   (u_stride * (dtype == RGLRU_BF16 ? 2 : 4)) % 16 == 0;
  a.nvec = (int)(vec ? W / (dtype == RGLRU_BF16 ? 8 : 4) : W);
  const long long items = (long long)B * a.nvec;
  dim3 grid((unsigned)((items + kConvThreads - 1) / kConvThreads));
  hipStream_t s = (hipStream_t)stream;
  RGLRU_CONV_DISPATCH(decode_prepare_kernel, dtype, vec, grid, s, a);
  return check_launch("decode_prepare");
}

size_t rglru_hip_conv_padded_scratch_bytes(int64_t B, int64_t T) {
  if (B <= 0 || T <= 0) return 0;
  return (size_t)(B * T * 8 + (3 * B * T + 3 * B) * 4);
}

int rglru_hip_conv_padded_fwd(const void* u, const void* state, const void* taps, const void* bias,
                              const int64_t* segment_pos, const uint8_t* active, void* scratch,
                              void* out, void* new_state,
                              int64_t B, int64_t T, int64_t W, int64_t K, int dtype, int vec_dtype, void* stream) {
  int rc = conv_check("conv_padded_fwd", B, T, W, K, dtype, vec_dtype);
  if (rc) return rc;
  if (!u || !taps || !segment_pos || !active || !scratch || !out) return fail(RGLRU_E_ARG, "conv_padded_fwd: null pointer");
  if ((uintptr_t)scratch % 8) return fail(RGLRU_E_ARG, "conv_padded_fwd: scratch must be 8-byte aligned");
  if (B * T >= (1ll << 29)) return fail(RGLRU_E_UNSUPPORTED, "conv_padded_fwd: tensor too large");
  PaddedArgs a;
  memset(&a, 0, sizeof(a));
  a.u = u; a.state = state; a.taps = taps; a.bias = bias; a.segpos = (const long long*)segment_pos; a.active = active;
  a.out = out; a.new_state = new_state; a.scratch = (int*)scratch;
  a.B = (int)B; a.T = (int)T; a.W = (int)W; a.K = (int)K; a.vec_dtype = vec_dtype;
  const bool vec = conv_vector_ok(W, dtype, {u, state, out, new_state});
  a.nvec = (int)(vec ? W / (dtype == RGLRU_BF16 ? 8 : 4) : W);
  hipStream_t s = (hipStream_t)stream;
  hipLaunchKernelGGL(conv_padded_index_kernel, dim3((unsigned)B), dim3(64), 0, s, a);
  rc = check_launch("conv_padded_fwd index");
  if (rc) return rc;
  const long long blocks = (long long)B * padded_blocks_per_seq((int)T, a.nvec);
  if (blocks > 0x7fffffffll) return fail(RGLRU_E_UNSUPPORTED, "conv_padded_fwd: problem too large for one launch");
  dim3 grid((unsigned)blocks);
  RGLRU_CONV_DISPATCH(conv_padded_fwd_kernel, dtype, vec, grid, s, a);
  rc = check_launch("conv_padded_fwd");
  if (rc) return rc;
  // rows whose active tokens are a prefix: the dense kernel over the positions the index kernel derived
  ConvArgs d;
  memset(&d, 0, sizeof(d));
  d.u = u; d.state = state; d.taps = taps; d.bias = bias; d.out = out;
  d.segpos = padded_positions(scratch); d.rows = padded_rows(scratch, B, T);
  d.B = (int)B; d.T = (int)T; d.W = (int)W; d.K = (int)K; d.vec_dtype = vec_dtype; d.nvec = a.nvec;
  d.runs = (int)((T + kConvRunFwd - 1) / kConvRunFwd);
  const long long dense_blocks = B * conv_blocks_per_seq(d.runs, d.nvec);
  if (dense_blocks >= (1ll << 31)) return fail(RGLRU_E_UNSUPPORTED, "conv_padded_fwd: tensor too large");
  dim3 dense_grid((unsigned)dense_blocks);
  RGLRU_CONV_DISPATCH(conv_fwd_kernel, dtype, vec, dense_grid, s, d);
  return check_launch("conv_padded_fwd prefix rows");
}

int rglru_hip_rmsnorm_max_width(int dtype, int aligned) {
  const int v = aligned ? (dtype == RGLRU_BF16 ? 8 : 4) : 1;
  return 64 * kNormSlots * v;
}

int rglru_hip_rmsnorm_fwd(const void* x, const void* g, void* y, float* inv, int64_t rows, int64_t D, float eps,
                          int dtype, int vec_dtype, void* stream) {
  if (!x || !g || !y) return fail(RGLRU_E_ARG, "rmsnorm_fwd: null pointer");
  bool vec; int nvec;
  int rc = norm_check("rmsnorm_fwd", rows, D, dtype, vec_dtype, &vec, &nvec, {x, y});
  if (rc) return rc;
  NormArgs a;
  memset(&a, 0, sizeof(a));
  a.x = x; a.g = g; a.y = y; a.inv_out = inv; a.rows = rows; a.D = (int)D; a.nvec = nvec; a.vec_dtype = vec_dtype; a.eps = eps;
  dim3 grid((unsigned)norm_grid(rows));
  hipStream_t s = (hipStream_t)stream;
  if (dtype == RGLRU_BF16) {
    if (vec) norm_launch<__bf16, 8, false>(nvec, grid, s, a); else norm_launch<__bf16, 1, false>(nvec, grid, s, a);
  } else {
    if (vec) norm_launch<float, 4, false>(nvec, grid, s, a); else norm_launch<float, 1, false>(nvec, grid, s, a);
  }
  return check_launch("rmsnorm_fwd");
}

size_t rglru_hip_rmsnorm_scratch_bytes(int64_t rows, int64_t D) {
  if (rows <= 0 || D <= 0) return 0;
  return (size_t)norm_grid(rows) * (size_t)D * 4;
}

int rglru_hip_rmsnorm_bwd(const void* x, const void* g, const float* inv, const void* dy, void* scratch,
                          void* dx, void* dg, int64_t rows, int64_t D, int dtype, int vec_dtype, int grad_dtype,
                          void* stream) {
  if (!x || !g || !inv || !dy || !scratch || !dx) return fail(RGLRU_E_ARG, "rmsnorm_bwd: null pointer");
  if (grad_dtype != RGLRU_F32 && grad_dtype != RGLRU_BF16) return fail(RGLRU_E_ARG, "rmsnorm_bwd: unknown gradient dtype %d", grad_dtype);
  bool vec; int nvec;
  int rc = norm_check("rmsnorm_bwd", rows, D, dtype, vec_dtype, &vec, &nvec, {x, dy, dx});
  if (rc) return rc;
  NormArgs a;
  memset(&a, 0, sizeof(a));
  a.x = x; a.g = g; a.dy = dy; a.inv_in = inv; a.dx = dx; a.partial = (float*)scratch;
  a.rows = rows; a.D = (int)D; a.nvec = nvec; a.vec_dtype = vec_dtype;
  const int blocks = norm_grid(rows);
  dim3 grid((unsigned)blocks);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == RGLRU_BF16) {
    if (vec) norm_launch<__bf16, 8, true>(nvec, grid, s, a); else norm_launch<__bf16, 1, true>(nvec, grid, s, a);
  } else {
    if (vec) norm_launch<float, 4, true>(nvec, grid, s, a); else norm_launch<float, 1, true>(nvec, grid, s, a);
  }
  rc = check_launch("rmsnorm_bwd");
  if (rc || !dg) return rc;
  NormFinishArgs f;
  f.partial = a.partial; f.dg = dg; f.D = (int)D; f.slots = blocks; f.grad_dtype = grad_dtype;
  hipLaunchKernelGGL(rmsnorm_finish_kernel, dim3((unsigned)((D + 31) / 32)), dim3(256), 0, s, f);
  return check_launch("rmsnorm_bwd finish");
}

static long long colsum_slots(int64_t rows) {
  return (rows + kColsumLanes * kColsumRowsPerLane - 1) / (kColsumLanes * kColsumRowsPerLane);
}

int rglru_hip_sum_sets(const void* x, void* out, int64_t sets, int64_t n, int dtype, void* stream) {
  if (!x || !out) return fail(RGLRU_E_ARG, "sum_sets: null pointer");
  if (dtype != RGLRU_F32 && dtype != RGLRU_BF16) return fail(RGLRU_E_ARG, "sum_sets: dtype must be RGLRU_F32 or RGLRU_BF16, got %d", dtype);
  if (sets <= 0 || n <= 0) return fail(RGLRU_E_ARG, "sum_sets: sets and n must be positive (got %lld, %lld)", (long long)sets, (long long)n);
  if (sets >= (1 << 20) || n >= (1ll << 38)) return fail(RGLRU_E_UNSUPPORTED, "sum_sets: problem too large");
  const bool vec = conv_vector_ok(n, dtype, {x, out});
  const int V = vec ? (dtype == RGLRU_BF16 ? 8 : 4) : 1;
  SumSetsArgs a;
  a.x = x; a.out = out; a.n = n; a.sets = (int)sets;
  const long long blocks = ((n + V - 1) / V + 255) / 256;
  if (blocks >= (1ll << 31)) return fail(RGLRU_E_UNSUPPORTED, "sum_sets: problem too large");
  dim3 grid((unsigned)blocks);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == RGLRU_BF16) {
    if (vec) hipLaunchKernelGGL((sum_sets_kernel<__bf16, 8>), grid, dim3(256), 0, s, a);
    else hipLaunchKernelGGL((sum_sets_kernel<__bf16, 1>), grid, dim3(256), 0, s, a);
  } else {
    if (vec) hipLaunchKernelGGL((sum_sets_kernel<float, 4>), grid, dim3(256), 0, s, a);
    else hipLaunchKernelGGL((sum_sets_kernel<float, 1>), grid, dim3(256), 0, s, a);
  }
  return check_launch("sum_sets");
}

size_t rglru_hip_colsum_scratch_bytes(int64_t rows, int64_t D) {
  if (rows <= 0 || D <= 0) return 0;
  return (size_t)colsum_slots(rows) * (size_t)D * 4;
}

int rglru_hip_colsum(const void* x, void* scratch, void* out, int64_t rows, int64_t D, int dtype, int out_dtype,
                     void* stream) {
  if (!x || !scratch || !out) return fail(RGLRU_E_ARG, "colsum: null pointer");
  if (dtype != RGLRU_F32 && dtype != RGLRU_BF16) return fail(RGLRU_E_ARG, "colsum: dtype must be RGLRU_F32 or RGLRU_BF16, got %d", dtype);
  if (out_dtype != RGLRU_F32 && out_dtype != RGLRU_BF16) return fail(RGLRU_E_ARG, "colsum: unknown output dtype %d", out_dtype);
  if (rows <= 0 || D <= 0) return fail(RGLRU_E_ARG, "colsum: rows and D must be positive (got %lld, %lld)", (long long)rows, (long long)D);
  const long long slots = colsum_slots(rows);
  if (D >= (1 << 24) || slots >= (1ll << 24)) return fail(RGLRU_E_UNSUPPORTED, "colsum: matrix too large");
  const bool vec = conv_vector_ok(D, dtype, {x});
  const int V = vec ? (dtype == RGLRU_BF16 ? 8 : 4) : 1;
  ColsumArgs a;
  a.x = x; a.partial = (float*)scratch; a.rows = rows; a.D = (int)D; a.nvec = (int)((D + V - 1) / V);
  a.vec_groups = (a.nvec + kColsumVecs - 1) / kColsumVecs;
  if (slots * a.vec_groups >= (1ll << 31)) return fail(RGLRU_E_UNSUPPORTED, "colsum: matrix too large");
  dim3 grid((unsigned)(slots * a.vec_groups));
  hipStream_t s = (hipStream_t)stream;
  if (dtype == RGLRU_BF16) {
    if (vec) hipLaunchKernelGGL((colsum_kernel<__bf16, 8>), grid, dim3(256), 0, s, a);
    else hipLaunchKernelGGL((colsum_kernel<__bf16, 1>), grid, dim3(256), 0, s, a);
  } else {
    if (vec) hipLaunchKernelGGL((colsum_kernel<float, 4>), grid, dim3(256), 0, s, a);
    else hipLaunchKernelGGL((colsum_kernel<float, 1>), grid, dim3(256), 0, s, a);
  }
  int rc = check_launch("colsum");
  if (rc) return rc;
  NormFinishArgs f;
  f.partial = a.partial; f.dg = out; f.D = (int)D; f.slots = (int)slots; f.grad_dtype = out_dtype;
  hipLaunchKernelGGL(rmsnorm_finish_kernel, dim3((unsigned)((D + 31) / 32)), dim3(256), 0, s, f);
  return check_launch("colsum finish");
}

}  // extern "C"
