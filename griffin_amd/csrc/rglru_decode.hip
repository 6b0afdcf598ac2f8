// RG-LRU decode for gfx950: one recurrence step per launch (rglru_hip_step, rglru_hip_step_gated) and K
// teacher-forced steps in one launch (rglru_hip_steps).  Rows are sequences; there is no scan.

#include "rglru_fused.h"

namespace rglru {

// ------------------------------------------------------------------------------------------
// Decode step: rows are sequences, no scan; h is updated in place.
// ------------------------------------------------------------------------------------------
template <typename IO, int NKG>
__global__ __launch_bounds__(kThreads) void step_kernel(FusedArgs p) {
  constexpr int MT = 1, TR = 32, EL = 16;
  typedef Io<IO> Tr;
  typedef typename Tr::Frag Frag;
  constexpr int KC = NKG > 0 ? NKG * Tr::KG : Tr::KCMAX;
  constexpr int LDSROW = KC + Tr::HW;
  __shared__ __attribute__((aligned(16))) IO lds[TR * LDSROW];

  const WaveId w = wave_identity(p, blockIdx.x);
  const int hf = w.hf, tid = threadIdx.x;
  const IO* wg = (const IO*)p.wg;
  const IO* w_a_row = wg + ((long long)(0 * p.nb + w.k) * p.bwp + (w.slab_ok ? w.o : 0)) * p.bwp + hf * Tr::HW;
  const IO* w_x_row = wg + ((long long)(1 * p.nb + w.k) * p.bwp + (w.slab_ok ? w.o : 0)) * p.bwp + hf * Tr::HW;
  const float bias_a = p.bias[w.kp], bias_x = p.bias[p.Wp + w.kp];
  const float sp = w.ch_ok ? p.sp[w.kp] : 0.f;
  const long long W = p.W;
  const long long row0 = (long long)w.wg_in_unit * TR;

  float h_old[EL], gate[EL];
  unsigned fls[EL];
  auto load_state = [&]() {
#pragma unroll
    for (int e = 0; e < EL; ++e) {
      const long long row = row0 + hf * EL + e;
      const bool ok = w.ch_ok && row < p.B;
      const long long at = ok ? row * W + w.ch : 0;
      h_old[e] = ok ? p.h_prev[at] : 0.f;
      gate[e] = (ok && p.gate_v) ? (float)((const IO*)p.gate_v)[row * p.ld_gate + w.ch] : 0.f;
      fls[e] = (ok && p.flags) ? (unsigned)p.flags[row] : 0u;
    }
  };
  f32x16 ua[MT], ux[MT];
  float xv[EL];
  if constexpr (NKG > 0) {
    // Loads return in issue order and the step is a chain of latencies, not of bytes: the x tile (which
    // has to pass through LDS and a barrier) is requested first, the weights next, the lane's previous
    // states, gate values and flags last; they arrive while the projections are computed.  (9.05 us per
    // step with the states requested first, 7.66 us in this order, B256 W1024 in a HIP graph; x rows
    // loaded straight into MFMA fragments instead of through LDS: 8.2 us, 32 rows per load instruction.)
    constexpr int VPR = KC / Tr::HW;
    constexpr int NVX = (TR * VPR + kThreads - 1) / kThreads;
    Frag xin[NVX];
#pragma unroll
    for (int i = 0; i < NVX; ++i) {
      const int idx = tid + i * kThreads;
      const int row = idx / VPR, cv = idx - row * VPR;
      xin[i] = idx < TR * VPR ? load_x_frag<IO>(p, (const IO*)p.x, row0 + row, p.B, w.k, cv * Tr::HW) : Tr::zero();
    }
    HeldWeights<IO, NKG> hw;
    hw.load(w_a_row, w_x_row);
    load_state();
#pragma unroll
    for (int i = 0; i < NVX; ++i) {
      const int idx = tid + i * kThreads;
      const int row = idx / VPR, cv = idx - row * VPR;
      if (idx < TR * VPR) *reinterpret_cast<Frag*>(lds + row * LDSROW + cv * Tr::HW) = xin[i];
    }
    __syncthreads();
    if (w.slab_ok) gate_mfma_held<IO, MT, NKG>(lds, hw, 0, w.slab, w.r, hf, bias_a, bias_x, ua[0], ux[0], xv);
  } else {
    load_state();
    gate_tile_generic<IO, MT>(p, (const IO*)p.x, row0, p.B, w.k, w.slab, w.slab_ok, w_a_row, w_x_row,
                              bias_a, bias_x, lds, ua, ux, xv);
  }
  if (!w.ch_ok) return;
  IO* y = (IO*)p.y;
#pragma unroll
  for (int e = 0; e < EL; ++e) {
    const long long row = row0 + hf * EL + e;
    if (row >= p.B) break;
    GateOut go = gate_forward<Precise<IO>::value, true>(ua[0][e], ux[0][e], xv[e], sp, fls[e]);
    const long long at = row * W + w.ch;
    float h = fmaf(go.a, h_old[e], go.z);
    p.h_state[at] = h;
    if (p.gate_v) h *= gelu_tanh_parts(gate[e]).gelu;
    y[at] = (IO)h;
  }
}

// Decode step for 16-bit storage and gate blocks of 32 to 384 channels in steps of 32, on 16 x 16 MFMA tiles: a wave
// owns 16 sequences x 16 channels, a lane 4 sequences of one channel.  The step is a chain of latencies
// (launch, loads, products, gate math, stores), so the work is cut as fine as the matrix unit allows:
// four elements of gate math per lane instead of sixteen, 8 KB of weights per wave instead of 16, x rows
// straight into A fragments (16 rows of 64 contiguous bytes per load instruction; no LDS, no barrier),
// and at B256 W1024 one workgroup on every compute unit instead of on a quarter of them.
template <int NKS>
__global__ __launch_bounds__(kThreads) void step16_kernel(FusedArgs p) {
  typedef __bf16 IO;
  typedef bf16x8 Frag;
  typedef float f32x4v __attribute__((ext_vector_type(4)));
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, n = lane & 15, q = lane >> 4;
  // Grid: x = groups of four channel tiles (one per wave), y = tiles of 16 sequences.  No division on the way to the
  // first load: what this kernel takes is latency, and a 64-bit division by the tile count alone was 150 instructions.
  const int ct = (int)blockIdx.x * kWaves + wave;
  if (ct * 16 >= p.W) return;
  const long long row0 = (long long)blockIdx.y * 16;
  const long long W = p.W;
  const int ch = ct * 16 + n;                              // the lane's channel; a tile lies inside one gate block
  const int k = (int)__umulhi((unsigned)(ct * 16), p.bw_magic), o = ch - k * p.bw;
  const int kp = k * p.bwp + o;
  // A fragments: row m = lane % 16 is sequence row0 + m, element j of K step ks is input channel 32 ks + 8 q + j
  const long long arow = row0 + n;
  const bool arow_ok = arow < p.B;
  const IO* xr = (const IO*)p.x + (arow_ok ? arow : 0) * W + k * p.bw + 8 * q;
  Frag xa[NKS], fa[NKS], fx[NKS];
#pragma unroll
  for (int ks = 0; ks < NKS; ++ks) xa[ks] = *reinterpret_cast<const Frag*>(xr + 32 * ks);   // a row past the end reads row 0: its products are not used
  // B fragments: column n is output channel o, same K elements: rows of the two weight matrices
  const IO* wa = (const IO*)p.wg + ((long long)(0 * p.nb + k) * p.bwp + o) * p.bwp + 8 * q;
  const IO* wx = (const IO*)p.wg + ((long long)(1 * p.nb + k) * p.bwp + o) * p.bwp + 8 * q;
#pragma unroll
  for (int ks = 0; ks < NKS; ++ks) {
    fa[ks] = *reinterpret_cast<const Frag*>(wa + 32 * ks);
    fx[ks] = *reinterpret_cast<const Frag*>(wx + 32 * ks);
  }
  // accumulator register v of the lane is sequence row0 + 4 q + v
  float h_old[4], gate[4], xv[4];
  unsigned fls[4];
  // Every load below is made on every path, from row 0 where the lane's row does not exist (its value is never used)
  // and from x where there is no gate or flag tensor: loads under a condition end up in blocks of their own, each
  // waiting for its data before the next block issues its loads -- eight memory round trips in a row in a kernel that
  // is nothing but latency.  Unconditional, all of them are in flight together behind the fragment loads.
  const IO* gate_src = p.gate_v ? (const IO*)p.gate_v : (const IO*)p.x;
  const long long gate_ld = p.gate_v ? p.ld_gate : W;
  const unsigned char* flag_src = p.flags ? p.flags : (const unsigned char*)p.x;
  IO x_raw[4], gate_raw[4];
  unsigned char fl_raw[4];
#pragma unroll
  for (int v = 0; v < 4; ++v) {
    const long long row = row0 + 4 * q + v;
    const long long rr = row < p.B ? row : 0;
    h_old[v] = p.h_prev[rr * W + ch];
    x_raw[v] = ((const IO*)p.x)[rr * W + ch];
    gate_raw[v] = gate_src[rr * gate_ld + ch];
    fl_raw[v] = flag_src[rr];
  }
  const float bias_a = p.bias[kp], bias_x = p.bias[p.Wp + kp], sp = p.sp[kp];
  __builtin_amdgcn_sched_barrier(0);                       // or the compiler issues some of them behind the matrix products
#pragma unroll
  for (int v = 0; v < 4; ++v) {
    xv[v] = (float)x_raw[v];
    gate[v] = (float)gate_raw[v];
    fls[v] = p.flags ? (unsigned)fl_raw[v] : 0u;
  }
  f32x4v ua = {bias_a, bias_a, bias_a, bias_a}, ux = {bias_x, bias_x, bias_x, bias_x};
#pragma unroll
  for (int ks = 0; ks < NKS; ++ks) {
    ua = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa[ks], fa[ks], ua, 0, 0, 0);
    ux = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa[ks], fx[ks], ux, 0, 0, 0);
  }
  IO* y = (IO*)p.y;
  // the four elements side by side (their transcendental chains overlap), then the stores of the rows that exist
  float h_new[4], out[4];
#pragma unroll
  for (int v = 0; v < 4; ++v) {
    const GateOut go = gate_forward<Precise<IO>::value, true>(ua[v], ux[v], xv[v], sp, fls[v]);
    h_new[v] = fmaf(go.a, h_old[v], go.z);
    out[v] = p.gate_v ? h_new[v] * gelu_tanh_parts(gate[v]).gelu : h_new[v];
  }
#pragma unroll
  for (int v = 0; v < 4; ++v) {
    const long long row = row0 + 4 * q + v;
    if (row < p.B) {
      const long long at = row * W + ch;
      p.h_state[at] = h_new[v];
      y[at] = (IO)out[v];
    }
  }
}

// K consecutive decode steps on the tiling of step16_kernel: weights and the lane's four states stay in
// registers, the next step's x fragments, own x values and flags are requested before the current step
// is computed.
template <int NKS>
__global__ __launch_bounds__(kThreads) void steps16_kernel(FusedArgs p) {
  typedef __bf16 IO;
  typedef bf16x8 Frag;
  typedef float f32x4v __attribute__((ext_vector_type(4)));
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, n = lane & 15, q = lane >> 4;
  const int ctiles = p.W / 16;
  const long long wv = (long long)blockIdx.x * kWaves + wave;
  const int ct = (int)(wv % ctiles);
  const long long row0 = (wv / ctiles) * 16;
  if (row0 >= p.B) return;
  const long long W = p.W;
  const int ch = ct * 16 + n;
  const int k = ch / p.bw, o = ch - k * p.bw;
  const int kp = k * p.bwp + o;
  const long long step_elems = (long long)p.B * W;
  const int steps = p.T;
  const long long arow = row0 + n;
  const bool arow_ok = arow < p.B;
  const IO* xr = (const IO*)p.x + (arow_ok ? arow : 0) * W + k * p.bw + 8 * q;
  Frag fa[NKS], fx[NKS];
  const IO* wa = (const IO*)p.wg + ((long long)(0 * p.nb + k) * p.bwp + o) * p.bwp + 8 * q;
  const IO* wx = (const IO*)p.wg + ((long long)(1 * p.nb + k) * p.bwp + o) * p.bwp + 8 * q;
#pragma unroll
  for (int ks = 0; ks < NKS; ++ks) {
    fa[ks] = *reinterpret_cast<const Frag*>(wa + 32 * ks);
    fx[ks] = *reinterpret_cast<const Frag*>(wx + 32 * ks);
  }
  long long at[4], rowc[4];
  bool ok[4];
  float h[4];
#pragma unroll
  for (int v = 0; v < 4; ++v) {
    const long long row = row0 + 4 * q + v;
    ok[v] = row < p.B;
    rowc[v] = ok[v] ? row : 0;                             // a row past the end reads row 0; nothing of it is stored
    at[v] = rowc[v] * W + ch;
    h[v] = p.h_prev[at[v]];
  }
  const float bias_a = p.bias[kp], bias_x = p.bias[p.Wp + kp], sp = p.sp[kp];
  // Operands of a step: requested kAhead steps ahead, into as many register sets that take turns -- a step takes
  // under a microsecond, less than a load that comes from memory.  Per token at B256 W1024 (gate blocks of 128
  // channels): 1.13 us one step ahead, 0.84 / 0.77 / 0.71 / 0.67 / 0.71 us at 2 / 3 / 4 / 6 / 8; wider blocks have
  // larger sets and take fewer.
  constexpr int kAhead = NKS <= 4 ? 6 : NKS <= 8 ? 4 : 2;
  struct In { Frag xa[NKS]; IO xv[4]; unsigned char fl[4]; };
  In in[kAhead];
  // Loads and stores of the loop are made on every path (clamped addresses, stores dropped through their offset):
  // the wait for a step's operands can then leave the younger loads and stores in flight; with conditional ones
  // the compiler had to wait for everything, the stores just issued included, every step.
  const unsigned char* flag_src = p.flags ? p.flags : (const unsigned char*)p.x;   // no flags: some readable byte
  const long long flag_step = p.flags ? p.B : 0;
  long long flag_row[4];
#pragma unroll
  for (int v = 0; v < 4; ++v) flag_row[v] = p.flags ? rowc[v] : 0;
  auto issue = [&](In& s, int t) {
    const long long tt = t < steps ? t : 0;                // a step past the end re-reads step 0
    const long long base = tt * step_elems;
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) s.xa[ks] = *reinterpret_cast<const Frag*>(xr + base + 32 * ks);
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      s.xv[v] = ((const IO*)p.x)[base + at[v]];
      s.fl[v] = flag_src[tt * flag_step + flag_row[v]];
    }
  };
  auto step = [&](In& s, int t) {
    f32x4v ua = {bias_a, bias_a, bias_a, bias_a}, ux = {bias_x, bias_x, bias_x, bias_x};
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
      ua = __builtin_amdgcn_mfma_f32_16x16x32_bf16(s.xa[ks], fa[ks], ua, 0, 0, 0);
      ux = __builtin_amdgcn_mfma_f32_16x16x32_bf16(s.xa[ks], fx[ks], ux, 0, 0, 0);
    }
    float xcur[4];
    unsigned fcur[4];
#pragma unroll
    for (int v = 0; v < 4; ++v) { xcur[v] = (float)s.xv[v]; fcur[v] = p.flags ? (unsigned)s.fl[v] : 0u; }
    issue(s, t + kAhead);
    const rsrc_t ry = make_rsrc((IO*)p.y + (long long)t * step_elems, (unsigned)step_elems * 2u);
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const GateOut go = gate_forward<Precise<IO>::value, true>(ua[v], ux[v], xcur[v], sp, fcur[v]);
      h[v] = fmaf(go.a, h[v], go.z);
      BufIo<IO>::store((IO)h[v], ry, ok[v] ? (unsigned)at[v] * 2u : kOutOfRange, 0u);
    }
  };
#pragma unroll
  for (int j = 0; j < kAhead; ++j) issue(in[j], j);
  for (int t = 0; t < steps; t += kAhead) {
#pragma unroll
    for (int j = 0; j < kAhead; ++j)
      if (t + j < steps) step(in[j], t + j);
  }
#pragma unroll
  for (int v = 0; v < 4; ++v) if (ok[v]) p.h_state[at[v]] = h[v];
}

// K consecutive decode steps in one launch (teacher-forced inputs x[K, B, W]): the state stays in
// registers across the steps, the gate weights are loaded once, and the next step's x tile is requested
// while the current step is computed.  Same arithmetic as step_kernel, step by step.
template <typename IO, int NKG>
__global__ __launch_bounds__(kThreads) void steps_kernel(FusedArgs p) {
  constexpr int MT = 1, TR = 32, EL = 16;
  typedef Io<IO> Tr;
  typedef typename Tr::Frag Frag;
  constexpr int KC = NKG > 0 ? NKG * Tr::KG : Tr::KCMAX;
  constexpr int LDSROW = KC + Tr::HW;
  __shared__ __attribute__((aligned(16))) IO lds[TR * LDSROW];

  const WaveId w = wave_identity(p, blockIdx.x);
  const int hf = w.hf, tid = threadIdx.x;
  const IO* wg = (const IO*)p.wg;
  const IO* w_a_row = wg + ((long long)(0 * p.nb + w.k) * p.bwp + (w.slab_ok ? w.o : 0)) * p.bwp + hf * Tr::HW;
  const IO* w_x_row = wg + ((long long)(1 * p.nb + w.k) * p.bwp + (w.slab_ok ? w.o : 0)) * p.bwp + hf * Tr::HW;
  const float bias_a = p.bias[w.kp], bias_x = p.bias[p.Wp + w.kp];
  const float sp = w.ch_ok ? p.sp[w.kp] : 0.f;
  const long long W = p.W;
  const long long row0 = (long long)w.wg_in_unit * TR;
  const long long step_elems = (long long)p.B * W;
  const int steps = p.T;

  float h[EL];
#pragma unroll
  for (int e = 0; e < EL; ++e) {
    const long long row = row0 + hf * EL + e;
    h[e] = (w.ch_ok && row < p.B) ? p.h_prev[row * W + w.ch] : 0.f;
  }
  HeldWeights<IO, NKG> hw;
  hw.load(w_a_row, w_x_row);
  constexpr int VPR = KC / Tr::HW;
  constexpr int NVX = NKG > 0 ? (TR * VPR + kThreads - 1) / kThreads : 1;
  Frag pre[NVX];
  auto issue = [&](int k) {
    if constexpr (NKG > 0) {
#pragma unroll
      for (int i = 0; i < NVX; ++i) {
        const int idx = tid + i * kThreads, row = idx / VPR, cv = idx - row * VPR;
        pre[i] = Tr::zero();
        if (idx < TR * VPR && k < steps)
          pre[i] = load_x_frag<IO>(p, (const IO*)p.x + (long long)k * step_elems, row0 + row, p.B, w.k, cv * Tr::HW);
      }
    }
  };
  issue(0);
  for (int k = 0; k < steps; ++k) {
    unsigned fls[EL];
#pragma unroll
    for (int e = 0; e < EL; ++e) {
      const long long row = row0 + hf * EL + e;
      fls[e] = (p.flags && w.ch_ok && row < p.B) ? (unsigned)p.flags[(long long)k * p.B + row] : 0u;
    }
    f32x16 ua[MT], ux[MT];
    float xv[EL];
    if constexpr (NKG > 0) {
#pragma unroll
      for (int i = 0; i < NVX; ++i) {
        const int idx = tid + i * kThreads, row = idx / VPR, cv = idx - row * VPR;
        if (idx < TR * VPR) *reinterpret_cast<Frag*>(lds + row * LDSROW + cv * Tr::HW) = pre[i];
      }
      __syncthreads();
      issue(k + 1);
      if (w.slab_ok) gate_mfma_held<IO, MT, NKG>(lds, hw, 0, w.slab, w.r, hf, bias_a, bias_x, ua[0], ux[0], xv);
      __syncthreads();                                   // the tile is overwritten at the top of the next step
    } else {
      gate_tile_generic<IO, MT>(p, (const IO*)p.x + (long long)k * step_elems, row0, p.B, w.k, w.slab, w.slab_ok,
                                w_a_row, w_x_row, bias_a, bias_x, lds, ua, ux, xv);
    }
    if (w.ch_ok) {
      IO* y = (IO*)p.y + (long long)k * step_elems;
#pragma unroll
      for (int e = 0; e < EL; ++e) {
        const long long row = row0 + hf * EL + e;
        if (row < p.B) {
          GateOut go = gate_forward<Precise<IO>::value, true>(ua[0][e], ux[0][e], xv[e], sp, fls[e]);
          h[e] = fmaf(go.a, h[e], go.z);
          y[row * W + w.ch] = (IO)h[e];
        }
      }
    }
  }
  if (w.ch_ok) {
#pragma unroll
    for (int e = 0; e < EL; ++e) {
      const long long row = row0 + hf * EL + e;
      if (row < p.B) p.h_state[row * W + w.ch] = h[e];
    }
  }
}


}  // namespace rglru

using namespace rglru;

extern "C" {

static int step_impl(const void* x, const void* prep, const float* h_in, float* h, const uint8_t* flags,
                     const void* gate_v, int64_t gate_stride, void* y, int64_t B, int64_t W, int64_t nb, int dtype,
                     void* stream) {
  int rc = check_geometry("step", W, nb, dtype);
  if (rc) return rc;
  if (B <= 0) return fail(RGLRU_E_ARG, "step: B must be positive (got %lld)", (long long)B);
  if (!x || !prep || !h || !h_in || !y) return fail(RGLRU_E_ARG, "step: null pointer");
  if (B * W >= (1ll << 40)) return fail(RGLRU_E_UNSUPPORTED, "step: tensor too large");
  Geometry g = make_geometry(W, nb);
  FusedArgs a;
  memset(&a, 0, sizeof(a));
  fill_common(a, g, prep, dtype);
  if (gate_stride == 0) gate_stride = W;
  if (gate_v && gate_stride < W) return fail(RGLRU_E_ARG, "step: row stride %lld of the gate input is smaller than the width %lld", (long long)gate_stride, (long long)W);
  if (flags == RGLRU_FLAGS_FIRST_RESET) return fail(RGLRU_E_ARG, "step: RGLRU_FLAGS_FIRST_RESET is for whole sequences; pass one flag byte per row");
  a.x = x; a.flags = flags; a.y = y; a.h_state = h; a.h_prev = h_in; a.gate_v = gate_v; a.ld_gate = gate_stride;
  a.B = (int)B; a.T = 1;
  a.aligned = is_aligned(x, W, g.bw, elem_size(dtype));
  long long row_tiles = (B + 31) / 32;
  dim3 grid((unsigned)(row_tiles * g.units));
  hipStream_t s = (hipStream_t)stream;
  const int nks = step16_groups(g, dtype, a.aligned);
  {
    KernelTimer timer(2, s);
    if (nks > 0) {
      // 16 sequences x 16 channels per wave, four waves per workgroup
      if (B > 16ll * 65535 || W >= 65536) return fail(RGLRU_E_UNSUPPORTED, "step: more than 1048560 rows or 65535 channels");
      a.bw_magic = (unsigned)(((1ull << 32) + (unsigned long long)g.bw - 1) / (unsigned long long)g.bw);
      dim3 grid16((unsigned)((W / 16 + kWaves - 1) / kWaves), (unsigned)((B + 15) / 16));
      switch (nks) {
#define RGLRU_STEP16_CASE(N) case N: hipLaunchKernelGGL((step16_kernel<N>), grid16, dim3(kThreads), 0, s, a); break
        RGLRU_STEP16_CASE(1); RGLRU_STEP16_CASE(2); RGLRU_STEP16_CASE(3); RGLRU_STEP16_CASE(4); RGLRU_STEP16_CASE(5);
        RGLRU_STEP16_CASE(6); RGLRU_STEP16_CASE(7); RGLRU_STEP16_CASE(8); RGLRU_STEP16_CASE(9); RGLRU_STEP16_CASE(10);
        RGLRU_STEP16_CASE(11); default: RGLRU_STEP16_CASE(12);
#undef RGLRU_STEP16_CASE
      }
    } else {
      RGLRU_DISPATCH(step_kernel, grid, s, a, dtype, 0);
    }
  }
  return check_launch("step");
}

int rglru_hip_step(const void* x, const void* prep, float* h, const uint8_t* flags, void* y,
                   int64_t B, int64_t W, int64_t nb, int dtype, void* stream) {
  return step_impl(x, prep, h, h, flags, nullptr, 0, y, B, W, nb, dtype, stream);
}

int rglru_hip_step_gated(const void* x, const void* prep, const float* h_in, float* h_out, const uint8_t* flags,
                         const void* v, int64_t v_stride, void* out, int64_t B, int64_t W, int64_t nb, int dtype,
                         void* stream) {
  return step_impl(x, prep, h_in, h_out, flags, v, v_stride, out, B, W, nb, dtype, stream);
}

int rglru_hip_steps(const void* x, const void* prep, float* h, const uint8_t* flags, void* y,
                    int64_t K, int64_t B, int64_t W, int64_t nb, int dtype, void* stream) {
  int rc = check_geometry("steps", W, nb, dtype);
  if (rc) return rc;
  if (B <= 0 || K <= 0) return fail(RGLRU_E_ARG, "steps: K and B must be positive (got %lld, %lld)", (long long)K, (long long)B);
  if (!x || !prep || !h || !y) return fail(RGLRU_E_ARG, "steps: null pointer");
  if (flags == RGLRU_FLAGS_FIRST_RESET) return fail(RGLRU_E_ARG, "steps: RGLRU_FLAGS_FIRST_RESET is for whole sequences; pass one flag byte per step and row");
  if (K * B * W >= (1ll << 40) || K >= (1ll << 31) || B * W >= (1ll << 31)) return fail(RGLRU_E_UNSUPPORTED, "steps: tensor too large");
  Geometry g = make_geometry(W, nb);
  FusedArgs a;
  memset(&a, 0, sizeof(a));
  fill_common(a, g, prep, dtype);
  a.x = x; a.flags = flags; a.y = y; a.h_state = h; a.h_prev = h;
  a.B = (int)B; a.T = (int)K;
  a.aligned = is_aligned(x, W, g.bw, elem_size(dtype));
  long long row_tiles = (B + 31) / 32;
  dim3 grid((unsigned)(row_tiles * g.units));
  hipStream_t s = (hipStream_t)stream;
  const int nks = step16_groups(g, dtype, a.aligned);
  {
    KernelTimer timer(2, s);
    if (nks > 0) {
      const long long waves = ((B + 15) / 16) * (W / 16);
      dim3 grid16((unsigned)((waves + kWaves - 1) / kWaves));
      switch (nks) {
#define RGLRU_STEPS16_CASE(N) case N: hipLaunchKernelGGL((steps16_kernel<N>), grid16, dim3(kThreads), 0, s, a); break
        RGLRU_STEPS16_CASE(1); RGLRU_STEPS16_CASE(2); RGLRU_STEPS16_CASE(3); RGLRU_STEPS16_CASE(4); RGLRU_STEPS16_CASE(5);
        RGLRU_STEPS16_CASE(6); RGLRU_STEPS16_CASE(7); RGLRU_STEPS16_CASE(8); RGLRU_STEPS16_CASE(9); RGLRU_STEPS16_CASE(10);
        RGLRU_STEPS16_CASE(11); default: RGLRU_STEPS16_CASE(12);
#undef RGLRU_STEPS16_CASE
      }
    } else {
      RGLRU_DISPATCH(steps_kernel, grid, s, a, dtype, 0);
    }
  }
  return check_launch("steps");
}


}  // extern "C"
