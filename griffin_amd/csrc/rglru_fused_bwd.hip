// Fused RG-LRU backward for gfx950: the portable kernel, the reverse-scan / gradient kernel pairs of the
// register-held and the wide gate blocks, the fixed-order sums of the parameter gradients, and their
// entry points.  The forward kernels and the conventions shared with them are in rglru_fused.hip / .h.

#include "rglru_fused.h"

namespace rglru {

// ------------------------------------------------------------------------------------------
// Backward (gate recomputation + reverse scan).  Chunks of 32 tokens, walked from the last to the
// first.  Emits the direct input gradient, the gradients at both gate pre-activations and
// per-workgroup partial sums for the bias and Lambda gradients.
// ------------------------------------------------------------------------------------------
template <typename IO, int NKG>
__global__ __launch_bounds__(kThreads, (NKG == 0 ? 2 : 1)) void bwd_kernel(FusedArgs p) {
  constexpr int MT = 1, TR = 32, EL = 16;
  typedef Io<IO> Tr;
  typedef typename Tr::Frag Frag;
  constexpr int KC = NKG > 0 ? NKG * Tr::KG : Tr::KCMAX;
  constexpr int LDSROW = KC + Tr::HW;
  __shared__ __attribute__((aligned(16))) IO lds[TR * LDSROW];
  __shared__ unsigned s_ticket;

  const WaveId w = wave_identity(p, blockIdx.x);
  const int hf = w.hf, tid = threadIdx.x;
  const IO* wg = (const IO*)p.wg;
  const IO* w_a_row = wg + ((long long)(0 * p.nb + w.k) * p.bwp + (w.slab_ok ? w.o : 0)) * p.bwp + hf * Tr::HW;
  const IO* w_x_row = wg + ((long long)(1 * p.nb + w.k) * p.bwp + (w.slab_ok ? w.o : 0)) * p.bwp + hf * Tr::HW;
  HeldWeights<IO, NKG> hw;
  hw.load(w_a_row, w_x_row);
  const float nba = -kLog2e * p.bias[w.kp], nbx = -kLog2e * p.bias[p.Wp + w.kp];   // biases as the sigmoids take them
  const float sp = w.ch_ok ? p.sp[w.kp] : 0.f;
  const float cs = w.ch_ok ? p.cs[w.kp] : 0.f;
  const IO* x = (const IO*)p.x;
  const IO* dy = (const IO*)p.dy;
  IO* dx = (IO*)p.dx; IO* dua = (IO*)p.du_a; IO* dux = (IO*)p.du_x;
  const long long W = p.W;
  float sum_ba = 0.f, sum_bx = 0.f, sum_l = 0.f;
  const Queue q = make_queue(p, w.unit, w.wg_in_unit, p.nC);

  for (;;) {
    if (tid == 0) s_ticket = atomicAdd(q.counter, 1u);
    __syncthreads();
    const long long tk = s_ticket;
    if (tk >= q.tiles) break;
    const int cr = (int)(tk / q.n_b), b = q.first_b + (int)(tk - (long long)cr * q.n_b) * p.queues;
    const int c = p.nC - 1 - cr;
    const int t0 = c * TR;

    f32x16 ua[MT], ux[MT];
    float xv[EL];
    if constexpr (NKG > 0) {
      constexpr int VPR = KC / Tr::HW;
      for (int idx = tid; idx < TR * VPR; idx += kThreads) {
        const int row = idx / VPR, cv = idx - row * VPR;
        Frag v = load_x_frag<IO>(p, x + (long long)b * p.T * W, (long long)t0 + row, p.T, w.k, cv * Tr::HW);
        *reinterpret_cast<Frag*>(lds + row * LDSROW + cv * Tr::HW) = v;
      }
      __syncthreads();
      if (w.slab_ok) gate_mfma_held<IO, MT, NKG>(lds, hw, 0, w.slab, w.r, hf, 0.0f, 0.0f, ua[0], ux[0], xv);
      __syncthreads();
    } else {
      gate_tile_generic<IO, MT>(p, x + (long long)b * p.T * W, t0, p.T, w.k, w.slab, w.slab_ok, w_a_row, w_x_row,
                                0.0f, 0.0f, lds, ua, ux, xv);
    }
    if (!w.slab_ok) continue;

    const long long trow = (long long)b * p.T + t0 + hf * EL;
    // kept per local step: both gates, the decay, the input scale and dy; z = g i x is recomputed
    // where it is needed (two workgroups per compute unit need the registers)
    float r[EL], gi[EL], a[EL], g[EL], gy[EL];
    unsigned flbits = 0u;                                // two flag bits per local step
#pragma unroll
    for (int e = 0; e < EL; ++e) {
      const bool in = t0 + hf * EL + e < p.T;
      const unsigned fl = token_flag(p, trow + e, in) | ((p.first_reset && t0 + hf * EL + e == 0) ? RGLRU_FLAG_RESET : 0u);
      flbits |= fl << (2 * e);
      GateOut go = gate_forward<Precise<IO>::value, true>(ua[0][e], ux[0][e], xv[e], sp, fl, nba, nbx);
      r[e] = go.r; gi[e] = go.i; a[e] = go.a; g[e] = go.g;
      gy[e] = (in && w.ch_ok) ? (float)dy[(trow + e) * W + w.ch] : 0.f;
    }
    // forward recomputation of h_{t-1} from the checkpoint in front of the lane's 16 tokens
    float A = 1.f;
#pragma unroll
    for (int e = 0; e < EL; ++e) A *= a[e];
    const float A_o = xhalf(A, hf);
    const float A_lo = hf ? A_o : A;
    const float A_hi = hf ? A : A_o;
    float h_start = 0.f;
    if (w.ch_ok) {
      if (c == 0 && hf == 0) h_start = p.h0 ? p.h0[(long long)b * W + w.ch] : 0.f;
      else h_start = p.ckpt[((long long)b * p.ckpt_nC + (2 * c - 1 + hf)) * W + w.ch];
    }
    float h = h_start;
    float hp[EL];
#pragma unroll
    for (int e = 0; e < EL; ++e) { hp[e] = h; h = fmaf(a[e], h, g[e] * gi[e] * xv[e]); }

    // reverse affine map of this lane's run and of the chunk
    float carry = 0.f;
#pragma unroll
    for (int e = EL - 1; e >= 0; --e) { float d = gy[e] + carry; carry = a[e] * d; }
    const float D = carry, D_o = xhalf(D, hf);
    const float D_lo = hf ? D_o : D, D_hi = hf ? D : D_o;
    const float A_t = A_lo * A_hi, D_t = fmaf(A_lo, D_hi, D_lo);

    CarryChain chain;
    const long long seq = (long long)b * p.nC * W + w.ch;
    chain.rec = p.rec_a + seq; chain.stride = W;

    float d_in;
    if (c == p.nC - 1) {
      d_in = (w.ch_ok && p.dh_last) ? p.dh_last[(long long)b * W + w.ch] : 0.f;
    } else {
      if (w.ch_ok && hf == 0) carry_publish(chain, c, A_t, D_t, false);
      d_in = carry_lookback(chain, c, +1, p.nC, 0.f, w.ch_ok, p.limit, p.fail);
    }
    const float d_out = fmaf(A_t, d_in, D_t);
    if (w.ch_ok && hf == 0) carry_publish(chain, c, 0.f, d_out, true);
    if (c == 0 && p.dh0 && w.ch_ok && hf == 0) p.dh0[(long long)b * W + w.ch] = d_out;

    carry = hf ? d_in : fmaf(A_hi, d_in, D_hi);
#pragma unroll
    for (int e = EL - 1; e >= 0; --e) {
      const float d = gy[e] + carry;
      carry = a[e] * d;
      const unsigned fl = (flbits >> (2 * e)) & 3u;
      const bool rst = fl & 1u, ina = fl & 2u;
      const float xe = xv[e];
      // z = g * i * x
      float dg = d * gi[e] * xe;
      float di = d * g[e] * xe;
      float dxd = d * g[e] * gi[e];
      // g = sqrt(g2) with the bounded derivative; a = exp(l), g2 = 1 - exp(2l)
      float dg2 = dg * __builtin_amdgcn_rsqf(fmaxf(4.0f * (g[e] * g[e]), 1e-6f));
      float dl = fmaf(d * hp[e], a[e], -2.0f * (a[e] * a[e]) * dg2);
      if (rst) dl = 0.f;
      float dr = dl * cs;
      float va = dr * r[e] * (1.0f - r[e]);
      float vx = di * gi[e] * (1.0f - gi[e]);
      if (ina) { dl = 0.f; va = 0.f; vx = 0.f; dxd = 0.f; }
      sum_l = fmaf(dl, r[e], sum_l);
      sum_ba += va; sum_bx += vx;
      if (w.ch_ok && (t0 + hf * EL + e < p.T)) {
        const long long at = (trow + e) * W + w.ch;
        dx[at] = (IO)dxd; dua[at] = (IO)va; dux[at] = (IO)vx;
      }
    }
  }
  // per-workgroup partial sums (every slot is written, so the buffer needs no clearing)
  if (w.slab_ok) {
    sum_ba += xhalf(sum_ba, hf); sum_bx += xhalf(sum_bx, hf); sum_l += xhalf(sum_l, hf);
    if (hf == 0) {
      float* part = p.partial + (long long)w.wg_in_unit * 3 * p.Wp + w.k * p.bwp + w.o;
      part[0] = sum_ba; part[p.Wp] = sum_bx; part[2 * p.Wp] = sum_l;
    }
  }
}

// ------------------------------------------------------------------------------------------
// Fast backward, part 1 (16-bit storage, register-held weights): gate recomputation + both scans.
// Same mathematics as bwd_kernel, but every global access is a 16-byte vector: x and dy tiles are
// staged through LDS (prefetched one tile ahead), and the three outputs -- the direct input
// gradient and the interleaved pair (du_a, du_x) per channel -- are transposed through per-wave LDS
// areas.  `du2` is [B, T, nb, 2 * bw] with element 2 * o + gate, the layout the second part wants.
// ------------------------------------------------------------------------------------------
template <int ROWS> struct PairStage {                  // ROWS x 32 channels x 2 values of 16 bits
  static constexpr int kRowBytes = 128;
  static constexpr int kBytes = ROWS * kRowBytes + 256;
  static RGLRU_DEVICE unsigned row_offset(int row) { return (unsigned)row * kRowBytes + (row >= ROWS / 2 ? 128u : 0u); }
};

template <typename IO, int NKG, bool MASKED>
__global__ __launch_bounds__(kThreads, (NKG > 8 ? 1 : 2)) void bwd_scan_kernel(FusedArgs p) {
  constexpr int MT = 1, TR = 32, EL = 16;
  typedef Io<IO> Tr;
  typedef typename Tr::Frag Frag;
  // NKG < 0: the caller supplies the gate pre-activations (see fwd_kernel) and gets the gradients at
  // them back as two halves per block, [nb][B*T][du_a (bw) | du_x (bw)], the operand layout of the
  // two GEMMs it runs afterwards; no weights are read here.
  // NKG > 8: a block wider than four slabs, shared by `groups` workgroups as in fwd_kernel: the x
  // tile spans the block, the dy tile only the workgroup's own 128 channels.
  constexpr bool GIVEN = NKG < 0;
  constexpr bool WIDE = NKG > 8;
  constexpr int KC = (GIVEN ? 8 : NKG) * Tr::KG;         // block width (held weights)
  constexpr int TW = WIDE ? KC : kPackedWidth;           // tile width (narrow blocks are packed)
  constexpr int LDSROW = TW + Tr::HW;
  constexpr int DYROW = kPackedWidth + Tr::HW;
  static_assert(sizeof(IO) == 2 && NKG != 0, "fast backward is for 16-bit storage");
  __shared__ __attribute__((aligned(16))) IO lds_x[TR * LDSROW];
  __shared__ __attribute__((aligned(16))) IO lds_dy[TR * DYROW];
  __shared__ __attribute__((aligned(16))) IO lds_pre[GIVEN ? 2 * TR * LDSROW : Tr::HW];
  __shared__ __attribute__((aligned(16))) unsigned char stage_dx_all[kWaves * WaveStage<TR>::kBytes];
  __shared__ __attribute__((aligned(16))) unsigned char stage_du_all[kWaves * (GIVEN ? 2 * WaveStage<TR>::kBytes : PairStage<TR>::kBytes)];
  __shared__ unsigned s_ticket[2];
  // With 128- and 64-channel blocks the weight registers (64, 32) push the kernel into spilling; the
  // input gate's weights then live in LDS instead (each wave's 32 rows, read as B fragments per tile).
  constexpr bool XLDS = (NKG == 8 || NKG == 4);
  constexpr int WROW = KC + Tr::HW;
  __shared__ __attribute__((aligned(16))) IO lds_wx[XLDS ? 32 * kWaves * WROW : Tr::HW];

  const WaveId w = wave_identity(p, blockIdx.x);
  if (w.wg_in_unit >= p.wg_per_unit) return;             // only with xcd_map: the grid's last round is not full
  const int hf = w.hf, tid = threadIdx.x;
  unsigned char* stage_dx = stage_dx_all + w.wave * WaveStage<TR>::kBytes;
  unsigned char* stage_du = stage_du_all + w.wave * (GIVEN ? 2 * WaveStage<TR>::kBytes : PairStage<TR>::kBytes);
  const IO* wg = (const IO*)p.wg;
  const int o_safe = w.slab_ok ? w.o : 0;
  const IO* w_a_row = wg + ((long long)(0 * p.nb + w.k) * p.bwp + o_safe) * p.bwp + hf * Tr::HW;
  const IO* w_x_row = wg + ((long long)(1 * p.nb + w.k) * p.bwp + o_safe) * p.bwp + hf * Tr::HW;
  HeldWeights<IO, NKG> hw;
  if constexpr (XLDS) {
#pragma unroll
    for (int kg = 0; kg < NKG; ++kg) hw.a[kg] = *reinterpret_cast<const Frag*>(w_a_row + kg * Tr::KG);
    // each wave copies the 32 rows of W_x of its own slab (the waves of a packed unit belong to different blocks)
    const IO* src = wg + ((long long)(1 * p.nb + w.k) * p.bwp + (w.slab_ok ? w.slab * 32 : 0)) * p.bwp;
    for (int idx = w.lane; idx < 32 * (KC / Tr::HW); idx += 64) {
      const int row = idx / (KC / Tr::HW), v = idx - row * (KC / Tr::HW);
      *reinterpret_cast<Frag*>(lds_wx + (w.wave * 32 + row) * WROW + v * Tr::HW) = *reinterpret_cast<const Frag*>(src + (long long)row * p.bwp + v * Tr::HW);
    }
    __syncthreads();
  } else if constexpr (!GIVEN) {
    hw.load(w_a_row, w_x_row);
  }
  const float nba = -kLog2e * p.bias[w.kp], nbx = -kLog2e * p.bias[p.Wp + w.kp];   // biases as the sigmoids take them
  const float sp = p.sp[w.kp], cs = p.cs[w.kp];
  const IO* x = (const IO*)p.x;
  const IO* dy = (const IO*)p.dy;
  const long long W = p.W;
  const unsigned row_bytes = (unsigned)p.W * 2u;
  float sum_ba = 0.f, sum_bx = 0.f, sum_l = 0.f;
  const Queue q = make_queue(p, w.unit, w.wg_in_unit, p.nC);

  constexpr int VPR = TW / Tr::HW;
  constexpr int NV = (TR * VPR + kThreads - 1) / kThreads;
  constexpr int VPR_DY = kPackedWidth / Tr::HW;
  constexpr int NV_DY = (TR * VPR_DY + kThreads - 1) / kThreads;
  Frag pre_x[NV], pre_dy[NV_DY], pre_ua[GIVEN ? NV : 1], pre_ux[GIVEN ? NV : 1];
  unsigned pre_off[NV], dy_off[NV_DY], u_off[GIVEN ? NV : 1];
  // GIVEN: the tiles hold the 128 channels of this workgroup's four slabs
  const int group_col = (GIVEN || WIDE) ? (w.unit % p.groups) * kPackedWidth : 0;
  const int x_col = GIVEN ? w.k * p.bw + group_col : w.tile_col;
  const int dy_col = WIDE ? w.k * p.bw + group_col : x_col;
  const int own_col = WIDE ? group_col : 0;              // the dy tile's first column inside the x tile
  const unsigned u_row_bytes = 4u * (unsigned)p.bw;      // a row of `pre` and of du: two halves of bw 16-bit values
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int idx = tid + i * kThreads;
    const int row = idx / VPR, cv = idx - row * VPR;
    pre_off[i] = (idx < TR * VPR) ? (unsigned)row * row_bytes + (unsigned)(x_col + cv * Tr::HW) * 2u : kOutOfRange;
    if constexpr (GIVEN)
      u_off[i] = (idx < TR * VPR) ? (unsigned)row * u_row_bytes + (unsigned)(group_col + cv * Tr::HW) * 2u : kOutOfRange;
  }
#pragma unroll
  for (int i = 0; i < NV_DY; ++i) {
    const int idx = tid + i * kThreads;
    const int row = idx / VPR_DY, cv = idx - row * VPR_DY;
    // a wide block's last group may reach past the block: those columns belong to a wave without a slab
    const bool in = idx < TR * VPR_DY && (!WIDE || own_col + cv * Tr::HW < p.bw);
    dy_off[i] = in ? (unsigned)row * row_bytes + (unsigned)(dy_col + cv * Tr::HW) * 2u : kOutOfRange;
  }
  auto decode = [&](unsigned tk, int& c, int& b) {
    const unsigned cr = tk / (unsigned)q.n_b;
    c = p.nC - 1 - (int)cr;
    b = q.first_b + (int)(tk - cr * (unsigned)q.n_b) * p.queues;
  };
  auto issue = [&](unsigned tk) {
    // a ticket past the end keeps valid addresses (tile 0) but an empty extent: nothing is fetched
    const bool live = (long long)tk < q.tiles;
    int c, b;
    decode(live ? tk : 0u, c, b);
    const int rows = !live ? 0 : ((p.T - c * TR) < TR ? (p.T - c * TR) : TR);
    const long long first = ((long long)b * p.T + (long long)c * TR) * W;
    const rsrc_t rx = make_rsrc(x + first, (unsigned)rows * row_bytes);
    const rsrc_t rdy = make_rsrc(dy + first, (unsigned)rows * row_bytes);
#pragma unroll
    for (int i = 0; i < NV; ++i) pre_x[i] = buf_load_frag<Frag>(rx, pre_off[i]);
#pragma unroll
    for (int i = 0; i < NV_DY; ++i) pre_dy[i] = buf_load_frag<Frag>(rdy, dy_off[i]);
    if constexpr (GIVEN) {
      const IO* ubase = (const IO*)p.pre + ((long long)w.k * p.rows_total + (long long)b * p.T + (long long)c * TR) * (2 * p.bw);
      const rsrc_t ru = make_rsrc(ubase, (unsigned)rows * u_row_bytes);
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        pre_ua[i] = buf_load_frag<Frag>(ru, u_off[i]);
        pre_ux[i] = buf_load_frag<Frag>(ru, u_off[i] == kOutOfRange ? kOutOfRange : u_off[i] + 2u * (unsigned)p.bw);
      }
    }
  };

  // A pass of the loop ends with six 16-byte stores behind the loads of the next tile.  The wait for those loads at
  // the top of the loop counts operations in issue order and must hold on every path into the loop, so the paths
  // that store nothing (the first pass, a wave without a slab) issue six stores that their offset drops: the wait
  // then leaves six operations in flight instead of draining the stores of the tile just finished.
  auto six_dropped_stores = [&]() {
    const rsrc_t nowhere = make_rsrc(p.dx, 0u);
    const i32x4 nothing = {0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < 6; ++i) buf_store_b128(nothing, nowhere, kOutOfRange - 16u * (unsigned)i);   // distinct, or they are merged
  };
  if (tid == 0) s_ticket[0] = atomicAdd(q.counter, 1u);
  __syncthreads();
  unsigned tk = s_ticket[0];
  int par = 0;
  issue(tk);
  six_dropped_stores();
  while ((long long)tk < q.tiles) {
    int c, b;
    decode(tk, c, b);
    const int t0 = c * TR;
    const long long trow = (long long)b * p.T + t0 + hf * EL;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int idx = tid + i * kThreads;
      const int row = idx / VPR, cv = idx - row * VPR;
      if (idx < TR * VPR) {
        *reinterpret_cast<Frag*>(lds_x + row * LDSROW + cv * Tr::HW) = pre_x[i];
        if constexpr (GIVEN) {
          *reinterpret_cast<Frag*>(lds_pre + row * LDSROW + cv * Tr::HW) = pre_ua[i];
          *reinterpret_cast<Frag*>(lds_pre + (TR + row) * LDSROW + cv * Tr::HW) = pre_ux[i];
        }
      }
    }
#pragma unroll
    for (int i = 0; i < NV_DY; ++i) {
      const int idx = tid + i * kThreads;
      const int row = idx / VPR_DY, cv = idx - row * VPR_DY;
      if (idx < TR * VPR_DY) *reinterpret_cast<Frag*>(lds_dy + row * DYROW + cv * Tr::HW) = pre_dy[i];
    }
    // the next ticket, the token flags (two bits per local step) and the state at the start of the chunk (forward
    // checkpoint) are requested once the tile is in LDS: in front of it their latency would sit in the wait above
    // (one atomic instruction for the workgroup, live in its first lane only: atomicAdd would combine the lanes'
    // operations first and wait for the result on the spot)
    const unsigned next_raw = (unsigned)__builtin_amdgcn_raw_ptr_buffer_atomic_add_i32(1, make_rsrc(q.counter, 4u), tid == 0 ? 0u : kOutOfRange, 0, 0);
    unsigned flbits = 0u;
    if constexpr (MASKED) flbits = flag_run(p, trow, t0 + hf * EL);
    float h_start = 0.f;                                 // state in front of this lane's 16 tokens
    if (c == 0 && hf == 0) { if (p.h0) h_start = p.h0[(long long)b * W + w.ch]; }
    else h_start = p.ckpt[((long long)b * p.ckpt_nC + (2 * c - 1 + hf)) * W + w.ch];
    __syncthreads();
    f32x16 ua, ux;
    float xv[EL], gy[EL];
    if (w.slab_ok) {
      if constexpr (GIVEN) {
        const int col = w.wave * 32 + w.r;
#pragma unroll
        for (int e = 0; e < EL; ++e) {
          const int at = (hf * EL + e) * LDSROW + col;
          xv[e] = (float)lds_x[at];
          gy[e] = (float)lds_dy[(hf * EL + e) * DYROW + col];
          ua[e] = (float)lds_pre[at];
          ux[e] = (float)lds_pre[TR * LDSROW + at];
        }
      } else if constexpr (XLDS) {
#pragma unroll
        for (int v = 0; v < 16; ++v) { ua[v] = 0.0f; ux[v] = 0.0f; }     // the biases enter inside the sigmoids
        const int kb = NKG >= 8 ? 0 : w.kb;
        const IO* xrow = lds_x + tile_row<MT>(0, w.r) * LDSROW + kb + hf * Tr::HW;
        const IO* brow = lds_wx + (w.wave * 32 + w.r) * WROW + hf * Tr::HW;
#pragma unroll
        for (int kg = 0; kg < NKG; ++kg) {
          const Frag xa = *reinterpret_cast<const Frag*>(xrow + kg * Tr::KG);
          Tr::mma(ua, xa, hw.a[kg]);
          Tr::mma(ux, xa, *reinterpret_cast<const Frag*>(brow + kg * Tr::KG));
        }
#pragma unroll
        for (int e = 0; e < EL; ++e) xv[e] = (float)lds_x[(hf * EL + e) * LDSROW + kb + w.slab * 32 + w.r];
      } else {
        gate_mfma_held<IO, MT, NKG, TW>(lds_x, hw, 0, w.slab, w.r, hf, 0.0f, 0.0f, ua, ux, xv, w.kb);
      }
      if constexpr (!GIVEN) {
#pragma unroll
        for (int e = 0; e < EL; ++e) gy[e] = (float)lds_dy[(hf * EL + e) * DYROW + (NKG >= 8 ? 0 : w.kb) + w.slab * 32 - own_col + w.r];
      }
    }
    if (tid == 0) s_ticket[par ^ 1] = next_raw;
    __syncthreads();
    par ^= 1;
    const unsigned tk_next = s_ticket[par];
    if (!w.slab_ok) {                                    // a wave without a slab only helps with the loads
      issue(tk_next);
      six_dropped_stores();
      tk = tk_next;
      continue;
    }

    // Gate recomputation in two steps.  The chunk's reverse map needs only the decay a_t (and dy),
    // so the recurrence gate comes first and the map is published before the rest of the gate math:
    // the neighbours see it that much earlier.  z is not kept (g * i * x is recomputed where needed).
    float r[EL], gi[EL], a[EL], g[EL];
    float A = 1.f;
#pragma unroll
    for (int e = 0; e < EL; ++e) {
      const float re = sigmoid_fast(ua[e], nba);
      float l2 = re * sp;
      if constexpr (MASKED) l2 = masked_log2_decay_run(l2, flbits, e);
      const float ae = __builtin_amdgcn_exp2f(l2);
      r[e] = re; a[e] = ae;
      A *= ae;
    }
    const float A_o = xhalf(A, hf);
    const float A_lo = hf ? A_o : A;
    const float A_hi = hf ? A : A_o;
    // reverse affine map of this lane's run and of the chunk
    float carry = 0.f;
#pragma unroll
    for (int e = EL - 1; e >= 0; --e) { float d = gy[e] + carry; carry = a[e] * d; }
    const float D = carry, D_o = xhalf(D, hf);
    const float D_lo = hf ? D_o : D, D_hi = hf ? D : D_o;
    const float A_t = A_lo * A_hi, D_t = fmaf(A_lo, D_hi, D_lo);

    CarryChain chain;
    const long long seq = (long long)b * p.nC * W + w.ch;
    chain.rec = p.rec_a + seq; chain.stride = W;
    const bool last_chunk = c == p.nC - 1;
    if (!last_chunk && hf == 0) carry_publish(chain, c, A_t, D_t, false);

    // input gate and g = sqrt(1 - a^2)
#pragma unroll
    for (int e = 0; e < EL; ++e) {
      const float ie = sigmoid_fast(ux[e], nbx);
      float l2 = r[e] * sp;
      if constexpr (MASKED) l2 = masked_log2_decay_run(l2, flbits, e);     // gives g = 1 / g = 0
      const float ge = __builtin_amdgcn_sqrtf(one_minus_a2<false>(l2, a[e]));
      gi[e] = ie; g[e] = ge;
    }
    float d_in = (last_chunk && p.dh_last) ? p.dh_last[(long long)b * W + w.ch] : 0.f;
    if (!last_chunk) d_in = carry_lookback(chain, c, +1, p.nC, 0.f, true, p.limit, p.fail);
    // the next tile's loads go out behind the look-back: loads return in issue order, so requested in front of it
    // they would put their latency into every round trip of the walk
    issue(tk_next);
    const float d_out = fmaf(A_t, d_in, D_t);
    if (hf == 0) carry_publish(chain, c, 0.f, d_out, true);
    if (hf == 0 && c == 0 && p.dh0) p.dh0[(long long)b * W + w.ch] = d_out;

    // delta_t in place of dy_t (reverse), then one forward pass that carries h_{t-1} along
    carry = hf ? d_in : fmaf(A_hi, d_in, D_hi);
#pragma unroll
    for (int e = EL - 1; e >= 0; --e) { const float d = gy[e] + carry; gy[e] = d; carry = a[e] * d; }
    float h = h_start;                                   // the forward pass left a checkpoint every 16 tokens
    unsigned char* my_dx = stage_dx + WaveStage<TR>::row_offset(hf * EL) + w.r * 2;
    unsigned char* my_du = GIVEN ? stage_du + WaveStage<TR>::row_offset(hf * EL) + w.r * 2
                                 : stage_du + PairStage<TR>::row_offset(hf * EL) + w.r * 4;
#pragma unroll
    for (int e = 0; e < EL; ++e) {
      // With z = g i x, a = exp(l), g = sqrt(1 - a^2) (bounded derivative 1 / (2 max(g, 5e-4))):
      //   dz = delta,  dx_direct = delta g i,  di = delta g x,  dl = delta a (h_{t-1} - 2 a i x / (2 g_b))
      const float d = gy[e];
      const float xe = xv[e];
      // the factors below do not depend on delta; tying them to it keeps the compiler from computing
      // all of them before the look-back, where they would only occupy registers
      float ge = g[e], ie = gi[e], re = r[e];
      asm volatile("" : "+v"(ge), "+v"(ie), "+v"(re) : "v"(d));
      const float c1 = ge * ie;
      const float dxd = d * c1;
      const float ze = c1 * xe;
      // 2 q with q = i x / sqrt(max(4 g^2, 1e-6)): the factors 4 and 2 cancel exactly (powers of two)
      const float q2 = (ie * xe) * __builtin_amdgcn_rsqf(fmaxf(ge * ge, 0.25f * 1e-6f));
      float dl = (a[e] * d) * fmaf(-a[e], q2, h);
      // A reset token has a = 2^-126, which already switches dl off; a padded one has g = 0, which
      // zeroes dxd, vx and z, but its bounded-sqrt term would leak into dl.
      if constexpr (MASKED) { if ((flbits >> (2 * e)) & 2u) dl = 0.f; }
      const float va = dl * (cs * fmaf(-re, re, re));
      const float vx = (d * ze) * (1.0f - ie);
      h = fmaf(a[e], h, ze);
      sum_l = fmaf(dl, re, sum_l);
      sum_ba += va; sum_bx += vx;
      *reinterpret_cast<IO*>(my_dx + e * WaveStage<TR>::kRowBytes) = (IO)dxd;
      if constexpr (GIVEN) {
        *reinterpret_cast<IO*>(my_du + e * WaveStage<TR>::kRowBytes) = (IO)va;
        *reinterpret_cast<IO*>(my_du + WaveStage<TR>::kBytes + e * WaveStage<TR>::kRowBytes) = (IO)vx;
      } else {
        typedef IO io2 __attribute__((ext_vector_type(2)));
        io2 pair; pair[0] = (IO)va; pair[1] = (IO)vx;
        *reinterpret_cast<io2*>(my_du + e * PairStage<TR>::kRowBytes) = pair;
      }
    }
    wave_lds_fence();
    {
      const int rows = (p.T - t0) < TR ? (p.T - t0) : TR;
      const rsrc_t rdx = make_rsrc((const IO*)p.dx + ((long long)b * p.T + t0) * W, (unsigned)rows * row_bytes);
      stage_flush<TR>(stage_dx, rdx, row_bytes, (unsigned)(w.k * p.bw + w.slab * 32) * 2u, w.lane);
      if constexpr (GIVEN) {
        IO* dbase = (IO*)p.du_a + ((long long)w.k * p.rows_total + (long long)b * p.T + t0) * (2 * p.bw);
        const rsrc_t rdu = make_rsrc(dbase, (unsigned)rows * u_row_bytes);
        stage_flush<TR>(stage_du, rdu, u_row_bytes, (unsigned)(w.slab * 32) * 2u, w.lane);
        stage_flush<TR>(stage_du + WaveStage<TR>::kBytes, rdu, u_row_bytes, (unsigned)(p.bw + w.slab * 32) * 2u, w.lane);
      } else {
      const unsigned du_row_bytes = 2u * row_bytes;
      const rsrc_t rdu = make_rsrc((const IO*)p.du_a + ((long long)b * p.T + t0) * 2 * W, (unsigned)rows * du_row_bytes);
      const unsigned du_col = (unsigned)(w.k * 2 * p.bw + w.slab * 64) * 2u;
#pragma unroll
      for (int i = 0; i < TR / 8; ++i) {
        const int row = 8 * i + (w.lane >> 3);
        const unsigned seg = (unsigned)(w.lane & 7) * 16u;
        i32x4 v = *reinterpret_cast<const i32x4*>(stage_du + PairStage<TR>::row_offset(row) + seg);
        buf_store_b128(v, rdu, (unsigned)row * du_row_bytes + du_col + seg);
      }
      }
    }
    wave_lds_fence();
    tk = tk_next;
  }
  // per-workgroup partial sums (every slot is written, so the buffer needs no clearing)
  sum_ba += xhalf(sum_ba, hf); sum_bx += xhalf(sum_bx, hf); sum_l += xhalf(sum_l, hf);
  if (hf == 0 && w.slab_ok) {
    float* part = p.partial + (long long)w.wg_in_unit * 3 * p.Wp + w.k * p.bwp + w.o;
    part[0] = sum_ba; part[p.Wp] = sum_bx; part[2 * p.Wp] = sum_l;
  }
}

// ------------------------------------------------------------------------------------------
// Fast backward in two kernels that split the work along its one sequential dependency.
//
//   bwd_delta_kernel   the reverse scan  delta_t = dy_t + a_{t+1} delta_{t+1}  (and dh0 = a_0 delta_0).
//                      It recomputes only the decay a_t (the recurrence gate: half of the gate
//                      products, one sigmoid, one exp2 per element), runs the chunked scan with the
//                      carry protocol in the reverse direction and writes delta in the storage type.
//   bwd_grad_kernel    everything else, which has no dependency between tokens once delta is known:
//                      both gates again, the gradient at every element, and the two block-diagonal
//                      GEMMs (input gradient and weight gradients) straight from registers and LDS,
//                      so the gradients at the gate pre-activations never leave the chip.  The state
//                      in front of a token, h_{t-1}, is the forward output y_{t-1} as stored.
//
// The scan kernel is light (few registers, many waves per SIMD hide the look-back); the heavy
// kernel has no chains, no tickets and no carries, so its tiles are known in advance and can be
// prefetched, and its weight-gradient accumulators are shared by the eight waves of a workgroup.
// ------------------------------------------------------------------------------------------
#ifndef RGLRU_DELTA_DEPTH
#define RGLRU_DELTA_DEPTH 2
#endif
constexpr int kDeltaDepth = RGLRU_DELTA_DEPTH;         // records a walk of the reverse scan requests per round trip

#ifndef RGLRU_DELTA_OCC
#define RGLRU_DELTA_OCC 2
#endif
template <typename IO, int NKG, bool MASKED, int MT>
__global__ __launch_bounds__(kThreads, (MT == 1 ? 4 : RGLRU_DELTA_OCC)) void bwd_delta_kernel(FusedArgs p) {
  constexpr int TR = 32 * MT, EL = 16 * MT;
  typedef Io<IO> Tr;
  typedef typename Tr::Frag Frag;
  constexpr int TW = kPackedWidth;                       // tile width (narrow blocks are packed)
  constexpr int LDSROW = TW + Tr::HW;
  static_assert(sizeof(IO) == 2 && NKG > 0, "fast backward is for 16-bit storage and register-held weights");
  __shared__ __attribute__((aligned(16))) IO lds_x[TR * LDSROW];
  __shared__ __attribute__((aligned(16))) IO lds_dy[TR * LDSROW];
  __shared__ __attribute__((aligned(16))) unsigned char stage_all[kWaves * WaveStage<TR>::kBytes];
  __shared__ unsigned s_ticket[2];

  const WaveId w = wave_identity(p, blockIdx.x);
  const int hf = w.hf, tid = threadIdx.x;
  unsigned char* stage = stage_all + w.wave * WaveStage<TR>::kBytes;
  const IO* wg = (const IO*)p.wg;
  const IO* w_a_row = wg + ((long long)(0 * p.nb + w.k) * p.bwp + (w.slab_ok ? w.o : 0)) * p.bwp + hf * Tr::HW;
  Frag wa[NKG];
#pragma unroll
  for (int kg = 0; kg < NKG; ++kg) wa[kg] = *reinterpret_cast<const Frag*>(w_a_row + kg * Tr::KG);
  const float nba = -kLog2e * p.bias[w.kp];
  const float sp = p.sp[w.kp];
  const IO* x = (const IO*)p.x;
  const IO* dy = (const IO*)p.dy;
  const long long W = p.W;
  const unsigned row_bytes = (unsigned)p.W * 2u;
  const int nCk = (p.T + TR - 1) / TR;                   // chunks of this kernel's tile length
  const Queue q = make_queue(p, w.unit, w.wg_in_unit, nCk);
  const int kb = NKG == 8 ? 0 : w.kb;

  constexpr int VPR = TW / Tr::HW;
  constexpr int NV = (TR * VPR + kThreads - 1) / kThreads;
  Frag pre_x[NV], pre_dy[NV];
  unsigned pre_off[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int idx = tid + i * kThreads;
    const int row = idx / VPR, cv = idx - row * VPR;
    pre_off[i] = (idx < TR * VPR) ? (unsigned)row * row_bytes + (unsigned)(w.tile_col + cv * Tr::HW) * 2u : kOutOfRange;
  }
  auto decode = [&](unsigned tk, int& c, int& b) {
    const unsigned cr = tk / (unsigned)q.n_b;
    c = nCk - 1 - (int)cr;
    b = q.first_b + (int)(tk - cr * (unsigned)q.n_b) * p.queues;
  };
  auto issue = [&](unsigned tk) {
    // a ticket past the end keeps valid addresses (tile 0) but an empty extent: nothing is fetched
    const bool live = (long long)tk < q.tiles;
    int c, b;
    decode(live ? tk : 0u, c, b);
    const int rows = !live ? 0 : ((p.T - c * TR) < TR ? (p.T - c * TR) : TR);
    const long long first = ((long long)b * p.T + (long long)c * TR) * W;
    const rsrc_t rx = make_rsrc(x + first, (unsigned)rows * row_bytes);
    const rsrc_t rdy = make_rsrc(dy + first, (unsigned)rows * row_bytes);
#pragma unroll
    for (int i = 0; i < NV; ++i) { pre_x[i] = buf_load_frag<Frag>(rx, pre_off[i]); pre_dy[i] = buf_load_frag<Frag>(rdy, pre_off[i]); }
  };

  if (tid == 0) s_ticket[0] = atomicAdd(q.counter, 1u);
  __syncthreads();
  unsigned tk = s_ticket[0];
  int par = 0;
  issue(tk);
  while ((long long)tk < q.tiles) {
    int c, b;
    decode(tk, c, b);
    const int t0 = c * TR;
    const long long trow = (long long)b * p.T + t0 + hf * EL;
    unsigned next_raw = 0;
    if (tid == 0) next_raw = atomicAdd(q.counter, 1u);
    unsigned flbits[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) flbits[mt] = MASKED ? flag_run(p, trow + 16 * mt, t0 + hf * EL + 16 * mt) : 0u;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int idx = tid + i * kThreads;
      const int row = idx / VPR, cv = idx - row * VPR;
      if (idx < TR * VPR) {
        *reinterpret_cast<Frag*>(lds_x + row * LDSROW + cv * Tr::HW) = pre_x[i];
        *reinterpret_cast<Frag*>(lds_dy + row * LDSROW + cv * Tr::HW) = pre_dy[i];
      }
    }
    __syncthreads();
    float a[EL], gy[EL];
    if (w.slab_ok) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        f32x16 ua;
#pragma unroll
        for (int v = 0; v < 16; ++v) ua[v] = 0.0f;          // the bias enters inside the sigmoid
        const IO* xrow = lds_x + tile_row<MT>(mt, w.r) * LDSROW + kb + hf * Tr::HW;
#pragma unroll
        for (int kg = 0; kg < NKG; ++kg) Tr::mma(ua, *reinterpret_cast<const Frag*>(xrow + kg * Tr::KG), wa[kg]);
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          float l2 = sigmoid_fast(ua[v], nba) * sp;
          if constexpr (MASKED) l2 = masked_log2_decay_run(l2, flbits[mt], v);
          else if (mt == 0 && v == 0) l2 = (p.first_reset && c == 0 && hf == 0) ? kResetLog2 : l2;
          a[16 * mt + v] = __builtin_amdgcn_exp2f(l2);
          gy[16 * mt + v] = (float)lds_dy[(hf * EL + 16 * mt + v) * LDSROW + kb + w.slab * 32 + w.r];
        }
      }
    }
    if (tid == 0) s_ticket[par ^ 1] = next_raw;
    __syncthreads();
    par ^= 1;
    const unsigned tk_next = s_ticket[par];
    issue(tk_next);
    if (!w.slab_ok) {                                    // a wave without a slab only helps with the loads
      tk = tk_next;
      continue;
    }
    // reverse affine map of this lane's run and of the chunk: carry_out = A carry_in + D
    float A = 1.f, carry = 0.f;
#pragma unroll
    for (int e = EL - 1; e >= 0; --e) { const float d = gy[e] + carry; carry = a[e] * d; A *= a[e]; }
    const float D = carry;
    const float A_o = xhalf(A, hf), D_o = xhalf(D, hf);
    const float A_lo = hf ? A_o : A, A_hi = hf ? A : A_o;
    const float D_lo = hf ? D_o : D, D_hi = hf ? D : D_o;
    const float A_t = A_lo * A_hi, D_t = fmaf(A_lo, D_hi, D_lo);

    CarryChain chain;
    chain.rec = p.rec_a + (long long)b * p.nC * W + w.ch; chain.stride = W;
    const bool last_chunk = c == nCk - 1;
    if (!last_chunk && hf == 0) carry_publish(chain, c, A_t, D_t, false);
    float d_in = (last_chunk && p.dh_last) ? p.dh_last[(long long)b * W + w.ch] : 0.f;
    if (!last_chunk) d_in = carry_lookback<kDeltaDepth>(chain, c, +1, nCk, 0.f, true, p.limit, p.fail);
    const float d_out = fmaf(A_t, d_in, D_t);
    if (hf == 0) carry_publish(chain, c, 0.f, d_out, true);
    if (hf == 0 && c == 0 && p.dh0) p.dh0[(long long)b * W + w.ch] = d_out;

    // delta of every token, through the wave's staging area, as 16-byte row segments
    carry = hf ? d_in : fmaf(A_hi, d_in, D_hi);
    unsigned char* my = stage + WaveStage<TR>::row_offset(hf * EL) + w.r * 2;
#pragma unroll
    for (int e = EL - 1; e >= 0; --e) {
      const float d = gy[e] + carry;
      carry = a[e] * d;
      *reinterpret_cast<IO*>(my + e * WaveStage<TR>::kRowBytes) = (IO)d;
    }
    wave_lds_fence();
    {
      const int rows = (p.T - t0) < TR ? (p.T - t0) : TR;
      const rsrc_t rd = make_rsrc((const IO*)p.du_a + ((long long)b * p.T + t0) * W, (unsigned)rows * row_bytes);
      stage_flush<TR>(stage, rd, row_bytes, (unsigned)(w.k * p.bw + w.slab * 32) * 2u, w.lane);
    }
    wave_lds_fence();
    tk = tk_next;
  }
}

// The reverse scan with one workgroup per chain, the counterpart of fwd_chain_kernel: sixteen waves take the
// chain's 32-token tiles round robin from the last tile to the first, the recurrence gate's rows of the slab
// sit in LDS, and the carry goes from tile c + 1 to tile c through LDS.  A wave stages its own x tile (the
// block's K range) and its own 32 channels of dy; delta leaves through the x tile's area.
template <typename IO, int NKG, bool MASKED>
__global__ __launch_bounds__(kChainWaves * 64, 1) void bwd_delta_chain_kernel(FusedArgs p) {
  typedef Io<IO> Tr;
  typedef typename Tr::Frag Frag;
  static_assert(sizeof(IO) == 2 && (NKG == 8 || NKG == 4 || NKG == 2), "16-bit storage, gate blocks of 128, 64 or 32 channels");
  constexpr int TR = 32;
  constexpr int KC = NKG * Tr::KG;
  constexpr int S = KC / 32;
  constexpr int LDSROW = KC + Tr::HW;
  constexpr int VPR = KC / Tr::HW;
  constexpr int NV = TR * VPR / 64;
  constexpr int DYROW = 32 + Tr::HW;                       // the wave's 32 channels of dy, padded
  static_assert(TR * LDSROW * (int)sizeof(IO) >= WaveStage<TR>::kBytes, "the staging area lies over the x tile");
  __shared__ __attribute__((aligned(16))) IO lds_all[kChainWaves][TR * LDSROW];
  __shared__ __attribute__((aligned(16))) IO lds_w[32 * LDSROW];                    // [output channel][K], recurrence gate
  __shared__ __attribute__((aligned(8))) unsigned long long carry[kChainWaves][32];

  const int tid = threadIdx.x, lane = tid & 63, r = lane & 31, hf = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int sl = slot % S, u = (slot / S) * 8 + xcd;
  const bool chain_ok = u < p.B * p.nb;
  const int b = chain_ok ? u / p.nb : 0, k = chain_ok ? u - b * p.nb : 0;
  for (int i = tid; i < kChainWaves * 32; i += kChainWaves * 64) (&carry[0][0])[i] = 0ull;
  {
    const IO* wg = (const IO*)p.wg;
    for (int i = tid; i < 32 * VPR; i += kChainWaves * 64) {
      const int o = i / VPR, cv = i % VPR;
      *reinterpret_cast<Frag*>(lds_w + o * LDSROW + cv * Tr::HW) =
          *reinterpret_cast<const Frag*>(wg + ((long long)(0 * p.nb + k) * p.bwp + sl * 32 + o) * p.bwp + cv * Tr::HW);
    }
  }
  __syncthreads();
  if (!chain_ok) return;
  const int col0 = k * KC;
  const int ch = col0 + sl * 32 + r;
  const long long W = p.W;
  IO* lds = lds_all[wave];
  IO* lds_dy = lds;                                        // dy takes the x tile's place once the gate products have read it
  unsigned char* stage = reinterpret_cast<unsigned char*>(lds);
  const float nba = -kLog2e * p.bias[ch];
  const float sp = p.sp[ch];
  const int nC = (p.T + TR - 1) / TR;
  const unsigned row_bytes = (unsigned)p.W * 2u;
  const long long limit = p.limit < 0 ? -p.limit : p.limit;

  Frag pre[NV], pre_dy[2];
  unsigned pre_off[NV], dy_off[2];
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int idx = lane + 64 * i, row = idx / VPR, cv = idx - row * VPR;
    pre_off[i] = (unsigned)row * row_bytes + (unsigned)(col0 + cv * Tr::HW) * 2u;
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {                            // 32 rows x four 16-byte vectors
    const int idx = lane + 64 * i, row = idx >> 2, cv = idx & 3;
    dy_off[i] = (unsigned)row * row_bytes + (unsigned)(col0 + sl * 32 + cv * Tr::HW) * 2u;
  }
  const IO* xb = (const IO*)p.x + (long long)b * p.T * W;
  const IO* dyb = (const IO*)p.dy + (long long)b * p.T * W;
  auto issue = [&](int c) {                                // a tile in front of the first: empty extent, nothing is fetched
    const int rows = c < 0 ? 0 : ((p.T - c * TR) < TR ? (p.T - c * TR) : TR);
    const long long first = (long long)(c < 0 ? 0 : c) * TR * W;
    const rsrc_t rx = make_rsrc(xb + first, (unsigned)rows * row_bytes);
    const rsrc_t rdy = make_rsrc(dyb + first, (unsigned)rows * row_bytes);
#pragma unroll
    for (int i = 0; i < NV; ++i) pre[i] = buf_load_frag<Frag>(rx, pre_off[i]);
#pragma unroll
    for (int i = 0; i < 2; ++i) pre_dy[i] = buf_load_frag<Frag>(rdy, dy_off[i]);
  };
  const rsrc_t rh0 = make_rsrc(p.dh0, p.dh0 ? (unsigned)p.B * (unsigned)W * 4u : 0u);
  const int next_wave = (wave + kChainWaves - 1) % kChainWaves;    // the wave of tile c + 1
  bool gave_up = false;
  // carry into the chain's last tile (used by its wave only): no memory operation inside the loop is conditional
  const float d_first = p.dh_last ? p.dh_last[(long long)b * W + ch] : 0.f;
  issue(nC - 1 - wave);
  {
    // the stores the loop's back edge has in flight behind the prefetched tiles (dh0, two delta segments),
    // dropped through their offsets, in front of its entry (see fwd_chain_kernel)
    BufIo<float>::store(0.f, rh0, kOutOfRange, 0u);
    const i32x4 nothing = {0, 0, 0, 0};
    buf_store_b128(nothing, rh0, kOutOfRange);
    buf_store_b128(nothing, rh0, kOutOfRange + 16u);
  }
  for (int c = nC - 1 - wave; c >= 0; c -= kChainWaves) {
    const int t0 = c * TR;
    unsigned flbits = 0u;
    if constexpr (MASKED) flbits = flag_run(p, (long long)b * p.T + t0 + hf * 16, t0 + hf * 16);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int idx = lane + 64 * i, row = idx / VPR, cv = idx - row * VPR;
      *reinterpret_cast<Frag*>(lds + row * LDSROW + cv * Tr::HW) = pre[i];
    }
    wave_lds_fence();
    f32x16 ua;
#pragma unroll
    for (int v = 0; v < 16; ++v) ua[v] = 0.0f;             // the bias enters inside the sigmoid
    {
      const IO* xrow = lds + tile_row<1>(0, r) * LDSROW + hf * Tr::HW;
      const IO* wrow = lds_w + r * LDSROW + hf * Tr::HW;
      Frag xa[NKG];
#pragma unroll
      for (int kg = 0; kg < NKG; ++kg) xa[kg] = *reinterpret_cast<const Frag*>(xrow + kg * Tr::KG);
      wave_lds_fence();                                    // the x tile is in registers: dy may take its place
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int idx = lane + 64 * i, row = idx >> 2, cv = idx & 3;
        *reinterpret_cast<Frag*>(lds_dy + row * DYROW + cv * Tr::HW) = pre_dy[i];
      }
#pragma unroll
      for (int kg = 0; kg < NKG; ++kg) Tr::mma(ua, xa[kg], *reinterpret_cast<const Frag*>(wrow + kg * Tr::KG));
    }
    wave_lds_fence();
    issue(c - kChainWaves);
    float a[16], gy[16];
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      float l2 = sigmoid_fast(ua[v], nba) * sp;
      if constexpr (MASKED) l2 = masked_log2_decay_run(l2, flbits, v);
      else if (v == 0) l2 = (p.first_reset && c == 0 && hf == 0) ? kResetLog2 : l2;
      a[v] = __builtin_amdgcn_exp2f(l2);
      gy[v] = (float)lds_dy[(hf * 16 + v) * DYROW + r];
    }
    // reverse affine map of this lane's run and of the tile: carry_out = A carry_in + D
    float A = 1.f, run = 0.f;
#pragma unroll
    for (int e = 15; e >= 0; --e) { const float d = gy[e] + run; run = a[e] * d; A *= a[e]; }
    const float D = run;
    const float A_o = xhalf(A, hf), D_o = xhalf(D, hf);
    const float A_lo = hf ? A_o : A, A_hi = hf ? A : A_o;
    const float D_lo = hf ? D_o : D, D_hi = hf ? D : D_o;
    const float A_t = A_lo * A_hi, D_t = fmaf(A_lo, D_hi, D_lo);
    // the carry behind the tile: dh_last, or what the wave of tile c + 1 has left in LDS (entry tag = c + 2)
    float d_in = d_first;
    if (c != nC - 1) {
      long long polls = 0;
      bool ok;
      for (;;) {
        const unsigned long long e = __hip_atomic_load(&carry[next_wave][r], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        ok = (unsigned)e == (unsigned)(c + 2);
        d_in = __uint_as_float((unsigned)(e >> 32));
        if (__all(ok) || ++polls > limit) break;
        __builtin_amdgcn_s_sleep(1);
      }
      gave_up |= !__all(ok);
      if (!ok) d_in = __builtin_nanf("");
    }
    const float d_out = fmaf(A_t, d_in, D_t);
    if (hf == 0) __hip_atomic_store(&carry[wave][r], ((unsigned long long)__float_as_uint(d_out) << 32) | (unsigned long long)(unsigned)(c + 1),
                                    __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    BufIo<float>::store(d_out, rh0, (hf == 0 && c == 0) ? ((unsigned)b * (unsigned)W + (unsigned)ch) * 4u : kOutOfRange, 0u);

    // delta of every token, through the x tile's area, as 16-byte row segments
    run = hf ? d_in : fmaf(A_hi, d_in, D_hi);
    wave_lds_fence();                                      // dy has been read: its area becomes the staging area
    unsigned char* my = stage + WaveStage<TR>::row_offset(hf * 16) + r * 2;
#pragma unroll
    for (int e = 15; e >= 0; --e) {
      const float d = gy[e] + run;
      run = a[e] * d;
      *reinterpret_cast<IO*>(my + e * WaveStage<TR>::kRowBytes) = (IO)d;
    }
    wave_lds_fence();
    {
      const int rows = (p.T - t0) < TR ? (p.T - t0) : TR;
      const rsrc_t rd = make_rsrc((const IO*)p.du_a + ((long long)b * p.T + t0) * W, (unsigned)rows * row_bytes);
      stage_flush<TR>(stage, rd, row_bytes, (unsigned)(col0 + sl * 32) * 2u, lane);
    }
    wave_lds_fence();
  }
  if (gave_up && lane == 0) atomicOr(p.fail, 1u);
}

constexpr int kGradWaves = 8;                            // waves per workgroup of the gradient kernel
constexpr int kGradThreads = 64 * kGradWaves;

// One workgroup = one unit (a 128-channel gate block, or two / four narrower ones), eight waves in two
// roles, one wave of each role per SIMD.  A tile is 32 tokens of one sequence.
//   element waves (0-3, one per 32-channel slab): gate products on the matrix unit with the weights in
//     registers, then the gate math and the gradient at every element of the tile.  With the row
//     permutation of tile_row() a lane's accumulator registers are 16 consecutive tokens of one
//     channel, which is exactly the fragment layout of the weight-gradient product
//     dW[j][o] = sum_t x[t][j] du[t][o] (contraction over tokens): the x values and the du values of a
//     lane ARE its A and B fragments, no transposition needed.  They go to LDS together with the
//     token-major du tile and the direct part of the input gradient.  The lane's x, delta and h
//     values reach that layout through the matrix unit as well (tile times identity).
//   product waves (4-7, one per slab): for the tile the element waves finished one iteration earlier,
//     dx[t][j] = direct + sum_kappa du[t][kappa] w2t[j][kappa] for the slab's input channels j, and the
//     weight gradients of the slab's output channels against all input channels of the block, both
//     gates, accumulated in registers for the whole launch.  They also move the x tiles into LDS.
// The element waves are bound by the vector unit, the product waves by the matrix unit and LDS, so
// each SIMD overlaps the two; neither role needs more than 256 registers (weights in one, weight
// gradient accumulators in the other).  Exchange buffers and the x tile are double-buffered: one
// barrier per tile.
template <typename IO, int NKG, bool MASKED>
__global__ __launch_bounds__(kGradThreads, 1) void bwd_grad_kernel(FusedArgs p) {
  typedef Io<IO> Tr;
  typedef typename Tr::Frag Frag;
  static_assert(sizeof(IO) == 2 && NKG > 0, "16-bit storage only");
  constexpr int TR = 32;
  constexpr int KC = NKG * Tr::KG;                       // block width
  constexpr int S = KC / 32;                             // slabs per block
  constexpr int BPU = 4 / S;                             // blocks per unit
  constexpr int TW = kPackedWidth;                       // unit width
  constexpr int NKG2 = 2 * NKG;                          // K groups of the input-gradient product (2 * KC kappa)
  constexpr int ROW = TW + Tr::HW, ROW_DU = 2 * TW + Tr::HW;
  __shared__ __attribute__((aligned(16))) IO lds_x[3][TR * ROW];        // x tiles of three consecutive iterations
  __shared__ __attribute__((aligned(16))) IO lds_du[2][TR * ROW_DU];    // [token][2 * unit channel + gate]
  __shared__ __attribute__((aligned(16))) float lds_dxd[2][4][16][64];  // direct input gradient [slab][register][lane]
  __shared__ __attribute__((aligned(16))) Frag lds_xt[2][4][2][64];     // x fragments [slab][K group][lane]
  __shared__ __attribute__((aligned(16))) Frag lds_dub[2][4][2][2][64]; // du fragments [slab][gate][K group][lane]
  __shared__ __attribute__((aligned(16))) unsigned char stage_all[4 * WaveStage<TR>::kBytes];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 31, hf = lane >> 5;
  const int slab = wave & 3;
  const bool element_role = wave < 4;
  const int units = (p.nb + BPU - 1) / BPU;
  const int unit = blockIdx.x % units, wg_in_unit = blockIdx.x / units, n_wg = gridDim.x / units;
  const int blk = slab / S, sl = slab - blk * S;           // the wave's block inside the unit, its slab inside the block
  const bool slab_ok = unit * BPU + blk < p.nb;
  const int k = slab_ok ? unit * BPU + blk : p.nb - 1;
  const int uo = slab * 32 + r;                            // channel inside the unit
  const int unit_col = unit * TW;                          // first channel of the unit
  const int ch = slab_ok ? unit_col + uo : 0;
  const int kb = blk * KC;
  unsigned char* stage = stage_all + slab * WaveStage<TR>::kBytes;
  const long long W = p.W;
  const unsigned row_bytes = (unsigned)p.W * 2u;
  const int nC = (p.T + TR - 1) / TR;
  const int n_tiles = p.B * nC;                            // tiles of the unit; the workgroup takes wg_in_unit, + n_wg, ...

  // Position of a tile, advanced by n_wg tiles at a time without divisions.
  struct Place { int tile, b, c; };
  const int step_b = n_wg / nC, step_c = n_wg - step_b * nC;
  auto advance = [&](Place& q) {
    q.tile += n_wg; q.b += step_b; q.c += step_c;
    if (q.c >= nC) { q.c -= nC; q.b += 1; }
  };
  Place first;
  first.tile = wg_in_unit; first.b = wg_in_unit / nC; first.c = wg_in_unit - first.b * nC;

  if (element_role) {
    // ------------------------------------------------------------------ element waves
    HeldWeights<IO, NKG> hw;
    {
      const IO* wg = (const IO*)p.wg;
      const int o = sl * 32 + r;
      hw.load(wg + ((long long)(0 * p.nb + k) * p.bwp + o) * p.bwp + hf * Tr::HW,
              wg + ((long long)(1 * p.nb + k) * p.bwp + o) * p.bwp + hf * Tr::HW);
    }
    const float nba = -kLog2e * p.bias[ch], nbx = -kLog2e * p.bias[p.Wp + ch];
    const float sp = p.sp[ch], cs = p.cs[ch];
    float sum_ba = 0.f, sum_bx = 0.f, sum_l = 0.f;
    // The lane's x, delta and h_{t-1} values (16 consecutive tokens of its channel) come from the matrix
    // unit: a 32 x 32 tile times the identity returns the tile in accumulator layout, which is that
    // layout.  delta and y (shifted by one token) are loaded from memory directly as A fragments (row =
    // token tile_row(r), 8 channels of the wave's slab each), so they never pass through LDS.
    Frag ident[2];
#pragma unroll
    for (int q = 0; q < 2; ++q)
#pragma unroll
      for (int i = 0; i < Tr::HW; ++i) ident[q][i] = (IO)((16 * q + 8 * hf + i == r) ? 1.0f : 0.0f);
    Frag pre_d[2], pre_h[2];
    const int my_row = tile_row<1>(0, r);
    auto issue = [&](const Place& q) {
      const bool live = q.tile < n_tiles;
      const int b = live ? q.b : 0, c = live ? q.c : 0;
      const int t0 = c * TR;
      const int rows = !live ? 0 : ((p.T - t0) < TR ? (p.T - t0) : TR);
      const rsrc_t rd = make_rsrc((const IO*)p.du_a + ((long long)b * p.T + t0) * W, (unsigned)rows * row_bytes);
      // the state in front of token t is the output row t - 1; tile row i wants y row t0 - 1 + i.  The
      // row in front of the sequence's first token does not exist (h0 takes its place further down).
      const int shift = c == 0 ? 1 : 0;
      const int y_first = t0 - 1 + shift;
      const int y_rows = !live ? 0 : (t0 + rows - 1 - y_first);
      const rsrc_t rh = make_rsrc((const IO*)p.y + ((long long)b * p.T + y_first) * W, (unsigned)(y_rows > 0 ? y_rows : 0) * row_bytes);
#pragma unroll
      for (int q2 = 0; q2 < 2; ++q2) {
        const unsigned col = (unsigned)(unit_col + slab * 32 + q2 * Tr::KG + hf * Tr::HW) * 2u;
        pre_d[q2] = buf_load_frag<Frag>(rd, (unsigned)my_row * row_bytes + col);
        pre_h[q2] = buf_load_frag<Frag>(rh, my_row >= shift ? (unsigned)(my_row - shift) * row_bytes + col : kOutOfRange);
      }
    };
    // gate products of one tile: issued one iteration before their results are used, so the matrix
    // unit works on the next tile while the vector unit works on the current one
    auto gate_products = [&](const IO* tile_x, f32x16& ua, f32x16& ux) {
#pragma unroll
      for (int v = 0; v < 16; ++v) { ua[v] = 0.0f; ux[v] = 0.0f; }       // the biases enter inside the sigmoids
      const IO* xrow = tile_x + my_row * ROW + kb + hf * Tr::HW;
#pragma unroll
      for (int kg = 0; kg < NKG; ++kg) {
        const Frag xa = *reinterpret_cast<const Frag*>(xrow + kg * Tr::KG);
        Tr::mma(ua, xa, hw.a[kg]);
        Tr::mma(ux, xa, hw.x[kg]);
      }
    };
    Place at = first;
    issue(at);
    __syncthreads();                                     // x tiles 0 and 1 are in LDS
    f32x16 ua, ux;
    gate_products(lds_x[0], ua, ux);
    int xb = 0;                                          // x buffer of the current tile
    for (int it = 0; at.tile < n_tiles + n_wg; ++it) {
      const int cur = it & 1;
      const int xn = xb == 2 ? 0 : xb + 1;
      if (at.tile < n_tiles && slab_ok) {
        const int b = at.b, c = at.c;
        const int t0 = c * TR;
        unsigned flbits = 0u;
        if constexpr (MASKED) flbits = flag_run(p, (long long)b * p.T + t0 + hf * 16, t0 + hf * 16);
        float h_first = 0.f;                             // h0 of the sequence, for the lane that owns token 0
        if (c == 0 && hf == 0 && p.h0) h_first = p.h0[(long long)b * W + ch];

        const IO* tile_x = lds_x[xb];
        f32x16 xc, dc, hc, ua_next, ux_next;
#pragma unroll
        for (int v = 0; v < 16; ++v) { xc[v] = 0.0f; dc[v] = 0.0f; hc[v] = 0.0f; }
        const IO* xrow = tile_x + my_row * ROW + hf * Tr::HW;
#pragma unroll
        for (int q2 = 0; q2 < 2; ++q2) {
          Tr::mma(dc, pre_d[q2], ident[q2]);
          Tr::mma(hc, pre_h[q2], ident[q2]);
          Tr::mma(xc, *reinterpret_cast<const Frag*>(xrow + slab * 32 + q2 * Tr::KG), ident[q2]);
        }
        gate_products(lds_x[xn], ua_next, ux_next);
        Place nxt = at;
        advance(nxt);
        issue(nxt);
        if (c == 0 && hf == 0) hc[0] = h_first;

        IO* du_tile = lds_du[cur];
#pragma unroll
        for (int q = 0; q < 2; ++q) {
        Frag fx_t, fa, fx;                                 // x, du_a, du_x of the lane's tokens of K group q
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const int v = 8 * q + i;
          const int tok = hf * 16 + v;
          const float xe = xc[v];
          const float d = dc[v];
          const float hp = hc[v];
          const float re = sigmoid_fast(ua[v], nba), ie = sigmoid_fast(ux[v], nbx);
          float l2 = re * sp;
          if constexpr (MASKED) l2 = masked_log2_decay_run(l2, flbits, v);
          else if (v == 0) l2 = (p.first_reset && c == 0 && hf == 0) ? kResetLog2 : l2;
          const float ae = __builtin_amdgcn_exp2f(l2);
          const float g2 = one_minus_a2<false>(l2, ae);
          const float ge = __builtin_amdgcn_sqrtf(g2);
          // With z = g i x, a = exp(l), g = sqrt(1 - a^2) (bounded derivative 1 / sqrt(max(4 g^2, 1e-6))):
          //   dx_direct = delta g i,  di = delta g x,  dl = delta a (h_{t-1} - a i x / sqrt(max(g^2, 2.5e-7)))
          const float c1 = ge * ie;
          const float dxd = d * c1;
          const float ze = c1 * xe;
          const float q2 = (ie * xe) * __builtin_amdgcn_rsqf(fmaxf(g2, 0.25f * 1e-6f));
          float dl = (ae * d) * fmaf(-ae, q2, hp);
          // A reset token has a = 2^-126, which already switches dl off; a padded one has g = 0, which
          // zeroes dxd, vx and z, but its bounded-sqrt term would leak into dl.
          if constexpr (MASKED) { if ((flbits >> (2 * v)) & 2u) dl = 0.f; }
          const float va = dl * (cs * fmaf(-re, re, re));
          const float vx = (d * ze) * (1.0f - ie);
          sum_l = fmaf(dl, re, sum_l);
          sum_ba += va; sum_bx += vx;
          typedef IO io2 __attribute__((ext_vector_type(2)));
          io2 pair; pair[0] = (IO)va; pair[1] = (IO)vx;
          *reinterpret_cast<io2*>(du_tile + tok * ROW_DU + 2 * uo) = pair;
          lds_dxd[cur][slab][v][lane] = dxd;
          fx_t[i] = (IO)xe; fa[i] = pair[0]; fx[i] = pair[1];
        }
        lds_xt[cur][slab][q][lane] = fx_t;
        lds_dub[cur][slab][0][q][lane] = fa;
        lds_dub[cur][slab][1][q][lane] = fx;
        }
        ua = ua_next; ux = ux_next;
      }
      xb = xn;
      advance(at);
      __syncthreads();
    }
    if (slab_ok) {
      // per-workgroup partial of the bias and Lambda gradients
      sum_ba += xhalf(sum_ba, hf); sum_bx += xhalf(sum_bx, hf); sum_l += xhalf(sum_l, hf);
      if (hf == 0) {
        float* ps = p.partial + (long long)wg_in_unit * 3 * p.Wp + ch;
        ps[0] = sum_ba; ps[p.Wp] = sum_bx; ps[2 * p.Wp] = sum_l;
      }
    }
  } else {
    // ------------------------------------------------------------------ product waves
    // this wave's rows of w2t, B operand of the input-gradient product; lane (n = j, hf) holds
    // kappa = 16 kg + 8 hf + i
    Frag w2[NKG2];
    {
      const IO* row = (const IO*)p.w2t + ((long long)k * p.bwp + sl * 32 + r) * (2 * p.bwp) + hf * Tr::HW;
#pragma unroll
      for (int kg = 0; kg < NKG2; ++kg) w2[kg] = *reinterpret_cast<const Frag*>(row + kg * Tr::KG);
    }
    f32x16 dw[2][S];                                     // [gate][input slab js of the block]: rows = own output channels, columns = j
#pragma unroll
    for (int g = 0; g < 2; ++g)
#pragma unroll
      for (int js = 0; js < S; ++js)
#pragma unroll
        for (int v = 0; v < 16; ++v) dw[g][js][v] = 0.f;
    // x tiles: 32 rows x 16 vectors, two per thread of the four product waves
    const int gid = tid - 4 * 64;
    Frag pre_x[2];
    auto issue = [&](const Place& q) {
      const bool live = q.tile < n_tiles;
      const int b = live ? q.b : 0, c = live ? q.c : 0;
      const int t0 = c * TR;
      const int rows = !live ? 0 : ((p.T - t0) < TR ? (p.T - t0) : TR);
      const rsrc_t rx = make_rsrc((const IO*)p.x + ((long long)b * p.T + t0) * W, (unsigned)rows * row_bytes);
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int idx = gid + 256 * i, row = idx >> 4, cv = idx & 15;
        pre_x[i] = buf_load_frag<Frag>(rx, (unsigned)row * row_bytes + (unsigned)(unit_col + cv * Tr::HW) * 2u);
      }
    };
    auto store_x = [&](int buf) {
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int idx = gid + 256 * i, row = idx >> 4, cv = idx & 15;
        *reinterpret_cast<Frag*>(lds_x[buf] + row * ROW + cv * Tr::HW) = pre_x[i];
      }
    };
    // the x tile of iteration it + 2 goes to LDS in iteration it
    Place ahead = first;
    issue(ahead);
    store_x(0);
    advance(ahead);
    issue(ahead);
    store_x(1);
    advance(ahead);
    issue(ahead);
    __syncthreads();                                     // x tiles 0 and 1 are in LDS
    Place at = first, done = first;                      // `done`: the tile the element waves finished last
    int xw = 2;                                          // x buffer written in this iteration
    for (int it = 0; at.tile < n_tiles + n_wg; ++it) {
      const int prev = (it & 1) ^ 1;
      store_x(xw);
      xw = xw == 2 ? 0 : xw + 1;
      advance(ahead);
      issue(ahead);
      if (it > 0 && slab_ok) {
        const int b = done.b, c = done.c;
        const int t0 = c * TR;
        // weight gradients: the fragments the element waves left in LDS
#pragma unroll
        for (int q = 0; q < 2; ++q) {
          // all fragments of a K group first, so that their LDS latencies overlap
          const Frag ba = lds_dub[prev][slab][0][q][lane], bx = lds_dub[prev][slab][1][q][lane];
          Frag xt[S];
#pragma unroll
          for (int js = 0; js < S; ++js) xt[js] = lds_xt[prev][blk * S + js][q][lane];
#pragma unroll
          for (int js = 0; js < S; ++js) {
            Tr::mma(dw[0][js], ba, xt[js]);
            Tr::mma(dw[1][js], bx, xt[js]);
          }
        }
        // input gradient of this slab's channels: direct part + du . w2t^T.  The A fragments are
        // requested four at a time so that their LDS latency overlaps (one fragment per product would
        // expose it sixteen times).
        f32x16 acc;
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[v] = lds_dxd[prev][slab][v][lane];
        const IO* a_row_du = lds_du[prev] + tile_row<1>(0, r) * ROW_DU + 2 * kb + hf * Tr::HW;
        constexpr int kBatch = NKG2 < 4 ? NKG2 : 4;
#pragma unroll
        for (int kg0 = 0; kg0 < NKG2; kg0 += kBatch) {
          Frag af[kBatch];
#pragma unroll
          for (int j = 0; j < kBatch; ++j) af[j] = *reinterpret_cast<const Frag*>(a_row_du + (kg0 + j) * Tr::KG);
#pragma unroll
          for (int j = 0; j < kBatch; ++j) Tr::mma(acc, af[j], w2[kg0 + j]);
        }
        unsigned char* my = stage + WaveStage<TR>::row_offset(hf * 16) + r * 2;
#pragma unroll
        for (int v = 0; v < 16; ++v) *reinterpret_cast<IO*>(my + v * WaveStage<TR>::kRowBytes) = (IO)acc[v];
        wave_lds_fence();
        const int rows = (p.T - t0) < TR ? (p.T - t0) : TR;
        const rsrc_t rdx = make_rsrc((const IO*)p.dx + ((long long)b * p.T + t0) * W, (unsigned)rows * row_bytes);
        stage_flush<TR>(stage, rdx, row_bytes, (unsigned)(unit_col + slab * 32) * 2u, lane);
        wave_lds_fence();
      }
      done = at;
      advance(at);
      __syncthreads();
    }
    if (slab_ok) {
      // per-workgroup partial of the weight gradients, laid out like the gradients themselves: [wg][k][gate][o][j].
      // Register v of an accumulator is row o = 8 (v / 4) + 4 hf + v % 4 of the wave's slab, the lane's r its column j.
      // 16-bit partials cross the wave's staging area and leave as 16-byte row segments.
#pragma unroll
      for (int g = 0; g < 2; ++g) {
        const long long first = ((((long long)wg_in_unit * p.nb + k) * 2 + g) * p.bwp + sl * 32) * p.bwp;
        if (p.dw_bf16) {
          const rsrc_t rp = make_rsrc((__bf16*)p.dw_partial + first, 32u * (unsigned)p.bwp * 2u);
#pragma unroll
          for (int js = 0; js < S; ++js) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
              const int o = 8 * (v >> 2) + 4 * hf + (v & 3);
              *reinterpret_cast<IO*>(stage + WaveStage<TR>::row_offset(o) + r * 2) = (IO)dw[g][js][v];
            }
            wave_lds_fence();
            stage_flush<TR>(stage, rp, (unsigned)p.bwp * 2u, (unsigned)(js * 32) * 2u, lane);
            wave_lds_fence();
          }
        } else {
          float* part = p.dw_partial + first;
#pragma unroll
          for (int js = 0; js < S; ++js)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
              const int o = 8 * (v >> 2) + 4 * hf + (v & 3);
              part[(long long)o * p.bwp + js * 32 + r] = dw[g][js][v];
            }
        }
      }
    }
  }
}

// ------------------------------------------------------------------------------------------
// Backward of blocks wider than 128 channels, second part: the two block-diagonal GEMMs of the gate
// gradients on the pairs du2[n][k][2 o + gate] that bwd_scan_kernel left in memory,
//     dx[n, j]   += sum_kappa du2[n, kappa] * w2t[j, kappa]          (kappa = 2 * o + gate)
//     dW[gate][j][o] = sum_n x[n, j] * du2[n, 2 o + gate]
// over the flattened token axis n = b * T + t, 32 tokens per tile.  A unit is a group of two
// 32-column slabs j of one gate block; its eight waves are (slab, quarter): a wave owns every fourth
// 32-wide kappa tile, and for those it keeps its slab's w2t fragments (B operand of the first GEMM,
// which it contracts over its own kappa only: the four quarters' partial tiles are added through LDS)
// and its slab's 32 x 32 accumulators of the second GEMM in registers for the whole launch.  The
// second GEMM contracts over tokens, i.e. over the ROWS of the du2 and x tiles as they lie in LDS:
// both operands come from transposing LDS reads (lds_transposed_frag), nothing is transposed by hand.
// Where LDS has room for two tiles (blocks of up to 320 channels) the next tile is written while this
// one is multiplied and a tile costs one barrier; the wider blocks keep one tile and two barriers.
// ------------------------------------------------------------------------------------------
template <int NKG> struct GateGradWideLds {
  static constexpr int TR = 32, K2 = 2 * NKG * 16, JW = 64;
  // du2 rows: K2 * 2 bytes is a multiple of 128, + 64 bytes makes the stride 64 or 192 modulo the 256 bytes of the
  // banks, so the four rows a transposing read touches (64 bytes of each) fall on different banks
  static constexpr int ROW_DU = K2 + 32, ROW_X = JW + 8;
  static constexpr int kDuBytes = TR * ROW_DU * 2, kXBytes = TR * ROW_X * 2, kRedBytes = 2 * 3 * 4 * 64 * 16;
  static constexpr int kStageBytes = 2 * WaveStage<TR>::kBytes;
  static constexpr bool kDouble = 2 * (kDuBytes + 2 * kXBytes + kRedBytes) + kStageBytes <= 160 * 1024;
  static constexpr int kBuffers = kDouble ? 2 : 1;
};

template <typename IO, int NKG>
__global__ __launch_bounds__(kGradThreads, 1) void gate_grad_wide_kernel(FusedArgs p) {
  typedef Io<IO> Tr;
  typedef typename Tr::Frag Frag;
  typedef GateGradWideLds<NKG> Lds;
  static_assert(sizeof(IO) == 2 && NKG > 8, "16-bit storage, blocks wider than 128 channels");
  constexpr int TR = Lds::TR;
  constexpr int KC = NKG * Tr::KG;                       // block width
  constexpr int K2 = Lds::K2;                            // kappa per block
  constexpr int S = KC / 32;                             // slabs in the block
  constexpr int JG = (S + 1) / 2;                        // units per block (two slabs each)
  constexpr int NKT = K2 / 32;                           // kappa tiles
  constexpr int NI = (NKT + 3) / 4;                      // ... per wave
  constexpr int JW = Lds::JW;                            // columns of the unit's x / dx tiles
  constexpr int ROW_DU = Lds::ROW_DU, ROW_X = Lds::ROW_X;
  constexpr bool DB = Lds::kDouble;
  constexpr int NB = Lds::kBuffers;
  __shared__ __attribute__((aligned(16))) IO lds_du[NB][TR * ROW_DU];
  __shared__ __attribute__((aligned(16))) IO lds_x[NB][TR * ROW_X];
  __shared__ __attribute__((aligned(16))) IO lds_dx[NB][TR * ROW_X];
  __shared__ __attribute__((aligned(16))) f32x4 lds_red[NB][2][4][3][64];  // [slab][receiving quarter][sender][lane]: four accumulator registers a vector
  __shared__ __attribute__((aligned(16))) unsigned char stage_all[Lds::kStageBytes];

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), r = lane & 31, hf = lane >> 5;
  const int sl = wave & 1, q = wave >> 1;
  // The JG units of a block that walk the same tiles read the same du2 rows.  Workgroups go to the eight XCDs
  // round-robin by index, each XCD has its own L2: index = xcd + 8 * slot puts the JG members of a
  // (block, tile sequence) pair into consecutive slots of ONE XCD, so that du2 comes from memory once.
  const int n_wg = p.wg_per_unit;
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int pair = xcd + 8 * (slot / JG), jg = slot % JG;
  const int k = pair % p.nb, wg_in_unit = pair / p.nb;
  if (wg_in_unit >= n_wg) return;                          // the grid is rounded up to whole rounds of eight pairs
  const int slab = jg * 2 + sl;
  const bool slab_ok = slab < S;
  const int j0 = (slab_ok ? slab : 0) * 32;                // the wave's first column inside the block
  unsigned char* stage = stage_all + sl * WaveStage<TR>::kBytes;
  const long long rows_total = (long long)p.B * p.T;
  const long long n_tiles = (rows_total + TR - 1) / TR;
  const unsigned row_bytes = (unsigned)p.W * 2u;

  // this wave's w2t fragments: row j0 + r, kappa tiles q, q + 4, ...; lane (j, hf) holds kappa = 32 kt + 16 g + 8 hf + i
  Frag w2[NI][2];
  {
    const IO* row = (const IO*)p.w2t + ((long long)k * p.bwp + j0 + r) * (2 * p.bwp) + hf * Tr::HW;
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
      for (int g = 0; g < 2; ++g) {
        const int kt = q + 4 * i;
        w2[i][g] = (slab_ok && kt < NKT) ? *reinterpret_cast<const Frag*>(row + kt * 32 + g * Tr::KG) : Tr::zero();
      }
  }
  f32x16 dw[NI];
#pragma unroll
  for (int i = 0; i < NI; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) dw[i][v] = 0.f;

  // cooperative tile loads: du2 (TR x K2 of block k), x and the direct part of dx (TR x 64 of the unit)
  constexpr int VPR_DU = K2 / Tr::HW, VPR_X = JW / Tr::HW;
  constexpr int NV_DU = (TR * VPR_DU + kGradThreads - 1) / kGradThreads;
  static_assert(TR * VPR_X <= kGradThreads, "one x vector per thread");
  const int unit_col = k * p.bw + jg * JW;                 // first channel of the unit
  struct Pre { Frag du[NV_DU]; Frag x, dx; };
  Pre preA, preB;                                          // register sets of the tiles one and two passes ahead
  unsigned du_off[NV_DU], x_off;
#pragma unroll
  for (int i = 0; i < NV_DU; ++i) {
    const int idx = tid + i * kGradThreads;
    const int row = idx / VPR_DU, cv = idx - row * VPR_DU;
    du_off[i] = idx < TR * VPR_DU ? (unsigned)row * 2u * row_bytes + (unsigned)(2 * k * p.bw + cv * Tr::HW) * 2u : kOutOfRange;
  }
  {
    const int row = tid / VPR_X, cv = tid - row * VPR_X;
    x_off = (tid < TR * VPR_X && jg * JW + cv * Tr::HW < KC) ? (unsigned)row * row_bytes + (unsigned)(unit_col + cv * Tr::HW) * 2u : kOutOfRange;
  }
  auto issue = [&](Pre& s, long long tile) {
    // a tile past the end keeps valid addresses but an empty extent: nothing is fetched
    const bool live = tile < n_tiles;
    const long long row0 = live ? tile * TR : 0;
    const int rows = !live ? 0 : (int)((rows_total - row0) < TR ? (rows_total - row0) : TR);
    const rsrc_t rdu = make_rsrc((const IO*)p.du_a + row0 * 2 * p.W, (unsigned)rows * 2u * row_bytes);
    const rsrc_t rx = make_rsrc((const IO*)p.x + row0 * p.W, (unsigned)rows * row_bytes);
    const rsrc_t rdx = make_rsrc((const IO*)p.dx + row0 * p.W, (unsigned)rows * row_bytes);
#pragma unroll
    for (int i = 0; i < NV_DU; ++i) s.du[i] = buf_load_frag<Frag>(rdu, du_off[i]);
    s.x = buf_load_frag<Frag>(rx, x_off);
    s.dx = buf_load_frag<Frag>(rdx, x_off);
  };
  // the tile in the registers above goes to LDS buffer b
  auto deposit = [&](const Pre& s, int b) {
#pragma unroll
    for (int i = 0; i < NV_DU; ++i) {
      const int idx = tid + i * kGradThreads;
      const int row = idx / VPR_DU, cv = idx - row * VPR_DU;
      if (idx < TR * VPR_DU) *reinterpret_cast<Frag*>(lds_du[b] + row * ROW_DU + cv * Tr::HW) = s.du[i];
    }
    if (tid < TR * VPR_X) {
      const int row = tid / VPR_X, cv = tid - row * VPR_X;
      *reinterpret_cast<Frag*>(lds_x[b] + row * ROW_X + cv * Tr::HW) = s.x;
      *reinterpret_cast<Frag*>(lds_dx[b] + row * ROW_X + cv * Tr::HW) = s.dx;
    }
  };

  // The tiles are requested two passes ahead, into two register sets that alternate (one pass of 2 us does not
  // cover a load that misses L2: 378 -> 345 us at B1 T32768 W2560).  Every pass ends with one store behind the loads
  // it issued; stores that their offset drops put the passes in front of the loop into the same state, so the wait
  // for a set's loads leaves the younger set's loads and the stores in flight on every path into the loop (the
  // counter is in issue order; without this the compiler must wait for everything, the store of the tile just
  // finished included).
  long long tile = wg_in_unit;
  const i32x4 nothing = {0, 0, 0, 0};
  const rsrc_t nowhere = make_rsrc(p.dx, 0u);
  // (352 and 384 channels: six accumulator tiles a wave, no room for the second set -- one pass ahead.)
  constexpr bool TWO = NI <= 5;
  constexpr int AHEAD = (DB ? 2 : 1) + (TWO ? 1 : 0);      // passes between a tile's request and its multiplication
  issue(preA, tile);
  if (DB) {
    deposit(preA, 0);
    if (TWO) {
      issue(preB, tile + n_wg);
      buf_store_b128(nothing, nowhere, kOutOfRange);
      issue(preA, tile + 2 * n_wg);
    } else {
      issue(preA, tile + n_wg);
    }
    buf_store_b128(nothing, nowhere, kOutOfRange - 16u);
    __syncthreads();
  } else {
    buf_store_b128(nothing, nowhere, kOutOfRange);
    if (TWO) {
      issue(preB, tile + n_wg);
      buf_store_b128(nothing, nowhere, kOutOfRange - 16u);
    }
  }
  int buf = 0;
  auto pass = [&](Pre& s) {
    if (DB) {
      // the buffer of the tile before this one: every wave has passed the barrier that ended its reads
      deposit(s, buf ^ 1);
      issue(s, tile + AHEAD * n_wg);
    } else {
      deposit(s, 0);
      issue(s, tile + AHEAD * n_wg);
      __syncthreads();
    }
    const long long row0 = tile * TR;
    const IO* du_tile = lds_du[buf];
    const IO* a_row_du = du_tile + tile_row<1>(0, r) * ROW_DU + hf * Tr::HW;
    // first GEMM over this wave's share of kappa.  The four quarters' partial tiles are added through LDS, each
    // quarter finishing four of a lane's sixteen tokens: registers 4 v4 .. 4 v4 + 3 go to quarter v4.  (A slab past
    // the block's end multiplies zeros; its stores are dropped through their offset, so that every wave issues the
    // same memory operations and the wait for the next tile's loads does not have to cover the stores.)
    float direct[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) direct[e] = (float)lds_dx[buf][(hf * 16 + 4 * q + e) * ROW_X + sl * 32 + r];
    f32x16 acc;
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[v] = 0.f;
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int kt = q + 4 * i;
      if (kt < NKT) {
        Tr::mma(acc, *reinterpret_cast<const Frag*>(a_row_du + (2 * kt) * Tr::KG), w2[i][0]);
        Tr::mma(acc, *reinterpret_cast<const Frag*>(a_row_du + (2 * kt + 1) * Tr::KG), w2[i][1]);
      }
    }
    f32x4 mine = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int v4 = 0; v4 < 4; ++v4) {
      const f32x4 part = {acc[4 * v4], acc[4 * v4 + 1], acc[4 * v4 + 2], acc[4 * v4 + 3]};
      if (v4 == q) mine = part;
      else lds_red[buf][sl][v4][q < v4 ? q : q - 1][lane] = part;
    }
    // second GEMM: dW2T[j, kappa] += sum over the tile's tokens, this wave's kappa tiles; tokens 0..15, then 16..31
    {
      const Frag xt0 = lds_transposed_frag(lds_x[buf], ROW_X, 0, sl * 32, lane);
      const Frag xt1 = lds_transposed_frag(lds_x[buf], ROW_X, 16, sl * 32, lane);
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        const int kt = q + 4 * i;
        if (kt < NKT) {
          Tr::mma(dw[i], xt0, lds_transposed_frag(du_tile, ROW_DU, 0, kt * 32, lane));
          Tr::mma(dw[i], xt1, lds_transposed_frag(du_tile, ROW_DU, 16, kt * 32, lane));
        }
      }
    }
    __syncthreads();
    {
      const f32x4 p0 = lds_red[buf][sl][q][0][lane], p1 = lds_red[buf][sl][q][1][lane], p2 = lds_red[buf][sl][q][2][lane];
      unsigned char* my = stage + WaveStage<TR>::row_offset(hf * 16 + 4 * q) + r * 2;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float sum = (direct[e] + mine[e]) + (p0[e] + (p1[e] + p2[e]));
        *reinterpret_cast<IO*>(my + e * WaveStage<TR>::kRowBytes) = (IO)sum;
      }
      wave_lds_fence();
      // the wave's eight rows (tokens 4 q .. + 3 and 16 + 4 q .. + 3) as 16-byte segments, one per lane of the lower half
      const int rows = (int)((rows_total - row0) < TR ? (rows_total - row0) : TR);
      const rsrc_t rdx = make_rsrc((const IO*)p.dx + row0 * p.W, (unsigned)rows * row_bytes);
      const int frow = ((lane >> 4) & 1) * 16 + 4 * q + ((lane >> 2) & 3);
      const unsigned seg = (unsigned)(lane & 3) * 16u;
      const i32x4 v = *reinterpret_cast<const i32x4*>(stage + WaveStage<TR>::row_offset(frow) + seg);
      buf_store_b128(v, rdx, (lane < 32 && slab_ok) ? (unsigned)frow * row_bytes + (unsigned)(k * p.bw + j0) * 2u + seg : kOutOfRange);
      wave_lds_fence();
    }
    if (DB) buf ^= 1;
    tile += n_wg;
  };
  for (;;) {
    if (tile >= n_tiles) break;
    pass(TWO && DB ? preB : preA);
    if (tile >= n_tiles) break;
    pass(TWO && !DB ? preB : preA);
  }
  // per-workgroup partial of the weight gradients, laid out like the gradients themselves: [wg][k][gate][o][j];
  // a lane's registers 4 v4 .. 4 v4 + 3 are four consecutive input channels j of its (gate, o)
  if (slab_ok) {
    float* part = p.dw_partial + ((long long)wg_in_unit * p.nb + k) * 2 * p.bwp * p.bwp;
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int kt = q + 4 * i;
      if (kt < NKT) {
        const int kappa = kt * 32 + r, o = kappa >> 1, gate = kappa & 1;
#pragma unroll
        for (int v4 = 0; v4 < 4; ++v4) {
          const int j = j0 + 8 * v4 + 4 * hf;
          const f32x4 four = {dw[i][4 * v4], dw[i][4 * v4 + 1], dw[i][4 * v4 + 2], dw[i][4 * v4 + 3]};
          *reinterpret_cast<f32x4*>(part + ((long long)gate * p.bwp + o) * p.bwp + j) = four;
        }
      }
    }
  }
}

// Last launch of a backward pass: sums the per-workgroup partial results and writes the parameter
// gradients in the caller's type.  Workgroups [0, vec_blocks) own 16 channels each of db_a, db_x and
// dLambda; the rest (backward paths with their own weight-gradient GEMM) own 2048 elements each of the two weight
// gradients, dW_gate[k][o][j] = sum over workgroups of the partials [wg][k][gate][o][j].
struct FinishArgs {
  const float* partial; const float* dsp; void* db_a; void* db_x; void* dlambda;
  const float* dw_partial; void* dw_a; void* dw_x;
  int W, nb, bw, bwp, Wp, wg_per_unit, n_wg, vec_blocks, grad_dtype, dw_bf16;
  int dw_vec;                                              // unpadded blocks of a multiple of 8 channels, 16-byte aligned gradients
};

__global__ __launch_bounds__(256) void finish_kernel(FinishArgs p) {
  __shared__ float part_sum[3][16][16];
  if ((int)blockIdx.x >= p.vec_blocks) {
    // eight consecutive input channels j of one (block, gate, output channel o) per thread: the partials are laid
    // out like the gradients, so this is a streaming sum in a fixed order with 16-byte accesses (dw_vec: the
    // block width equals the padded width)
    const long long per_gate = (long long)p.bw * p.bw;
    if (!p.dw_vec) {
      // any width, any alignment: eight elements of the unpadded gradients per thread, one at a time
      const long long total = (long long)p.nb * 2 * per_gate;
      const long long first = ((long long)(blockIdx.x - p.vec_blocks) * blockDim.x + threadIdx.x) * 8;
      const long long stride = (long long)p.nb * 2 * p.bwp * p.bwp;
      for (long long i = first; i < first + 8 && i < total; ++i) {
        const int j = (int)(i % p.bw), o = (int)((i / p.bw) % p.bw);
        const int gate = (int)((i / per_gate) % 2);
        const long long k = i / (2 * per_gate);
        const float* src = p.dw_partial + (((k * 2 + gate) * p.bwp + o) * p.bwp + j);
        float sum = 0.f;
        for (int g = 0; g < p.n_wg; ++g) sum += src[(long long)g * stride];
        store_vec(gate ? p.dw_x : p.dw_a, (k * p.bw + o) * p.bw + j, sum, p.grad_dtype);
      }
      return;
    }
    const long long total8 = (long long)p.nb * 2 * per_gate / 8;
    const long long i8 = (long long)(blockIdx.x - p.vec_blocks) * blockDim.x + threadIdx.x;
    if (i8 >= total8) return;
    const long long i = i8 * 8;
    const int gate = (int)((i / per_gate) % 2);
    const long long k = i / (2 * per_gate);
    const long long stride = (long long)p.nb * 2 * per_gate;
    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = 0.f;
    if (p.dw_bf16) {
      const __bf16* src16 = (const __bf16*)p.dw_partial + i;
      int g = 0;
      for (; g + 7 < p.n_wg; g += 8) {                       // eight loads in flight per thread
        bf16x8 v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = *reinterpret_cast<const bf16x8*>(src16 + (long long)(g + u) * stride);
#pragma unroll
        for (int u = 0; u < 8; ++u)
#pragma unroll
          for (int e = 0; e < 8; ++e) acc[e] += (float)v[u][e];
      }
      for (; g < p.n_wg; ++g) {
        const bf16x8 v = *reinterpret_cast<const bf16x8*>(src16 + (long long)g * stride);
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] += (float)v[e];
      }
    } else {
      const float* src = p.dw_partial + i;
      int g = 0;
      for (; g + 3 < p.n_wg; g += 4) {
        f32x4 v[4][2];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          v[u][0] = *reinterpret_cast<const f32x4*>(src + (long long)(g + u) * stride);
          v[u][1] = *reinterpret_cast<const f32x4*>(src + (long long)(g + u) * stride + 4);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
          for (int e = 0; e < 8; ++e) acc[e] += v[u][e >> 2][e & 3];
      }
      for (; g < p.n_wg; ++g) {
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] += src[(long long)g * stride + e];
      }
    }
    void* dst = gate ? p.dw_x : p.dw_a;
    const long long at = k * per_gate + (i % per_gate);      // element (k, o, j) of one gate's gradient
    if (p.grad_dtype == RGLRU_BF16) {
      bf16x8 out;
#pragma unroll
      for (int e = 0; e < 8; ++e) out[e] = (__bf16)acc[e];
      *reinterpret_cast<bf16x8*>((__bf16*)dst + at) = out;
    } else {
      const f32x4 lo = {acc[0], acc[1], acc[2], acc[3]}, hi = {acc[4], acc[5], acc[6], acc[7]};
      *reinterpret_cast<f32x4*>((float*)dst + at) = lo;
      *reinterpret_cast<f32x4*>((float*)dst + at + 4) = hi;
    }
    return;
  }
  // 16 channels per workgroup; sixteen threads per channel each sum a share of the per-workgroup
  // partials (independent loads), combined through LDS in a fixed order
  const int cl = threadIdx.x & 15, share = threadIdx.x >> 4;
  const int ch = blockIdx.x * 16 + cl;
  float sa = 0.f, sx = 0.f, sl = 0.f;
  int kp = 0;
  if (ch < p.W) {
    const int k = ch / p.bw, o = ch - k * p.bw;
    kp = k * p.bwp + o;
#pragma unroll 4
    for (int g = share; g < p.wg_per_unit; g += 16) {
      const float* part = p.partial + (long long)g * 3 * p.Wp + kp;
      sa += part[0]; sx += part[p.Wp]; sl += part[2 * p.Wp];
    }
  }
  part_sum[0][share][cl] = sa; part_sum[1][share][cl] = sx; part_sum[2][share][cl] = sl;
  __syncthreads();
  if (share == 0 && ch < p.W) {
    sa = 0.f; sx = 0.f; sl = 0.f;
#pragma unroll
    for (int q = 0; q < 16; ++q) { sa += part_sum[0][q][cl]; sx += part_sum[1][q][cl]; sl += part_sum[2][q][cl]; }
    store_vec(p.db_a, ch, sa, p.grad_dtype);
    store_vec(p.db_x, ch, sx, p.grad_dtype);
    store_vec(p.dlambda, ch, sl * p.dsp[kp], p.grad_dtype);
  }
}


}  // namespace rglru

using namespace rglru;

extern "C" {

static int check_grad_dtype(const char* who, int grad_dtype);

// Tail of the backward entry points whose scan kernel leaves the gradients at the gate pre-activations in
// memory: the two gate-gradient GEMMs (dx += du W; weight-gradient partials), then the fixed-order sums.
static int gate_gemms_and_finish(const FusedArgs& a, const Geometry& g, const void* prep, int dtype, int grad_dtype,
                                 const void* x, const void* du_a, const void* du_x, long long du_ld, long long du_blk,
                                 void* dx, char* scratch, int64_t B, int64_t T,
                                 void* dw_a, void* dw_x, void* db_a, void* db_x, void* dlambda, hipStream_t s) {
  const ScratchLayout SL = make_scratch_layout(B, T, g, kScratchPlain);
  const int splits = gate_dw_splits(B * T, g);
  float* dw_partial = (float*)(scratch + SL.dw_partial);
  int rc = launch_gate_gemms(x, du_a, du_x, du_ld, du_blk, a.w2t, dx, dw_partial, B * T, g, dtype, splits, s);
  if (rc) return rc;
  FinishArgs r;
  memset(&r, 0, sizeof(r));
  r.partial = a.partial; r.dsp = finish_dsp(g, prep, dtype); r.db_a = db_a; r.db_x = db_x; r.dlambda = dlambda;
  r.dw_partial = dw_partial; r.dw_a = dw_a; r.dw_x = dw_x;
  r.W = (int)g.W; r.nb = (int)g.nb; r.bw = (int)g.bw; r.bwp = (int)g.bwp; r.Wp = (int)g.Wp; r.wg_per_unit = a.wg_per_unit;
  r.n_wg = splits; r.vec_blocks = (int)((g.W + 15) / 16); r.grad_dtype = grad_dtype;
  r.dw_vec = (g.bw == g.bwp && (uintptr_t)dw_a % 16 == 0 && (uintptr_t)dw_x % 16 == 0) ? 1 : 0;
  const long long total = g.nb * g.bw * 2 * g.bw;
  hipLaunchKernelGGL(finish_kernel, dim3((unsigned)(r.vec_blocks + (total / 8 + 255) / 256)), dim3(256), 0, s, r);
  return check_launch("bwd finish");
}


int rglru_hip_bwd_pre(const void* x, void* pre, const void* prep, const float* h0,
                      const uint8_t* flags, const void* dy, const float* dh_last, void* ws, void* scratch,
                      void* dx, void* du, void* dw_a, void* dw_x, void* db_a, void* db_x, void* dlambda, float* dh0,
                      int64_t B, int64_t T, int64_t W, int64_t nb, int dtype, int grad_dtype, void* stream) {
  int rc = check_geometry("bwd_pre", W, nb, dtype);
  if (rc) return rc;
  rc = check_grad_dtype("bwd_pre", grad_dtype);
  if (rc) return rc;
  if (!rglru_hip_pre_path(W, nb, dtype)) return fail(RGLRU_E_UNSUPPORTED, "bwd_pre: needs bf16 storage and gate blocks of a multiple of 32 channels");
  if (B <= 0 || T <= 0) return fail(RGLRU_E_ARG, "bwd_pre: B and T must be positive (got %lld, %lld)", (long long)B, (long long)T);
  if (!x || !pre || !prep || !dy || !ws || !scratch || !dx || !du || !dw_a || !dw_x || !db_a || !db_x || !dlambda)
    return fail(RGLRU_E_ARG, "bwd_pre: null pointer");
  rc = check_extents("bwd_pre", B, T, W);
  if (rc) return rc;
  Geometry g = make_geometry(W, nb);
  if (!is_aligned(x, W, g.bw, 2) || !is_aligned(dy, W, g.bw, 2) || !is_aligned(dx, W, g.bw, 2) ||
      (uintptr_t)pre % 16 || (uintptr_t)du % 16)
    return fail(RGLRU_E_UNSUPPORTED, "bwd_pre: x, pre, dy, dx and du must be 16-byte aligned");
  WorkLayout L = make_work_layout(B, T, g);
  hipStream_t s = (hipStream_t)stream;
  char* wb = (char*)ws;
  FusedArgs a;
  memset(&a, 0, sizeof(a));
  fill_common(a, g, prep, dtype);
  if (flags == RGLRU_FLAGS_FIRST_RESET) { flags = nullptr; a.first_reset = 1; }
  a.x = x; a.pre = pre; a.rows_total = B * T; a.h0 = h0; a.flags = flags; a.dy = dy; a.dh_last = dh_last;
  a.flags_vec = (T % 16 == 0) && ((uintptr_t)flags % 16 == 0);
  a.dx = dx; a.du_a = du; a.dh0 = dh0;
  a.ckpt = (float*)(wb + L.ckpt); a.rec_a = (rec_t*)(wb + L.b_rec_a);
  a.ticket = (unsigned*)(wb + L.b_ticket); a.fail = (unsigned*)(wb + L.fail);
  a.partial = (float*)((char*)scratch + make_scratch_layout(B, T, g, kScratchPlain).partial);
  a.B = (int)B; a.T = (int)T; a.nC = (int)((T + kChunk - 1) / kChunk); a.ckpt_nC = 2 * (int)L.nC;
  a.aligned = 1;
  a.wg_per_unit = pick_wg_per_unit(a.units, B * (long long)a.nC, 2, L.max_wg);
  a.queues = pick_queues(B, a.wg_per_unit);
  const bool masked = (flags != nullptr) || a.first_reset || (T % kChunk != 0);
  dim3 grid((unsigned)(a.wg_per_unit * a.units));
  rc = launch_clear(wb, L.b_begin, L.b_end, s);          // records and tickets of this pass
  if (rc) return rc;
  rc = launch_gate_pre_gemm(x, a.wg, pre, B * T, g, s);  // the gate projections again
  if (rc) return rc;
  {
    KernelTimer timer(1, s);
    if (masked) hipLaunchKernelGGL((bwd_scan_kernel<__bf16, -1, true>), grid, dim3(kThreads), 0, s, a);
    else hipLaunchKernelGGL((bwd_scan_kernel<__bf16, -1, false>), grid, dim3(kThreads), 0, s, a);
  }
  rc = check_launch("bwd_pre scan");
  if (rc) return rc;
  // du is [nb][B T][du_a (bw) | du_x (bw)]
  return gate_gemms_and_finish(a, g, prep, dtype, grad_dtype, x, du, (const __bf16*)du + g.bw, 2 * g.bw, B * T * 2 * g.bw,
                               dx, (char*)scratch, B, T, dw_a, dw_x, db_a, db_x, dlambda, s);
}

static int check_grad_dtype(const char* who, int grad_dtype) {
  if (grad_dtype != RGLRU_F32 && grad_dtype != RGLRU_BF16) return fail(RGLRU_E_ARG, "%s: unknown gradient dtype %d", who, grad_dtype);
  return RGLRU_OK;
}

int rglru_hip_bwd(const void* x, const void* prep, const float* h0,
                  const uint8_t* flags, const void* dy, const float* dh_last, void* ws, void* scratch,
                  void* dx, void* du_a, void* du_x, void* dw_a, void* dw_x, void* db_a, void* db_x, void* dlambda,
                  float* dh0, int64_t B, int64_t T, int64_t W, int64_t nb, int dtype, int grad_dtype,
                  void* stream) {
  int rc = check_geometry("bwd", W, nb, dtype);
  if (rc) return rc;
  rc = check_grad_dtype("bwd", grad_dtype);
  if (rc) return rc;
  if (B <= 0 || T <= 0) return fail(RGLRU_E_ARG, "bwd: B and T must be positive (got %lld, %lld)", (long long)B, (long long)T);
  if (!x || !prep || !dy || !ws || !scratch || !dx || !du_a || !du_x || !dw_a || !dw_x || !db_a || !db_x || !dlambda)
    return fail(RGLRU_E_ARG, "bwd: null pointer");
  rc = check_extents("bwd", B, T, W);
  if (rc) return rc;
  Geometry g = make_geometry(W, nb);
  WorkLayout L = make_work_layout(B, T, g);
  hipStream_t s = (hipStream_t)stream;
  char* wb = (char*)ws;
  FusedArgs a;
  memset(&a, 0, sizeof(a));
  fill_common(a, g, prep, dtype);
  if (flags == RGLRU_FLAGS_FIRST_RESET) { flags = nullptr; a.first_reset = 1; }
  a.x = x; a.h0 = h0; a.flags = flags; a.dy = dy; a.dh_last = dh_last;
  a.flags_vec = (T % 16 == 0) && ((uintptr_t)flags % 16 == 0);
  a.dx = dx; a.du_a = du_a; a.du_x = du_x; a.dh0 = dh0;
  a.ckpt = (float*)(wb + L.ckpt); a.rec_a = (rec_t*)(wb + L.b_rec_a);
  a.ticket = (unsigned*)(wb + L.b_ticket); a.fail = (unsigned*)(wb + L.fail);
  a.partial = (float*)((char*)scratch + make_scratch_layout(B, T, g, kScratchPlain).partial);
  a.B = (int)B; a.T = (int)T; a.nC = (int)((T + kChunk - 1) / kChunk); a.ckpt_nC = 2 * (int)L.nC; a.nCf = (int)L.nCf;
  a.aligned = is_aligned(x, W, g.bw, elem_size(dtype));
  a.wg_per_unit = pick_wg_per_unit(a.units, B * (long long)a.nC, 2, L.max_wg);
  a.queues = pick_queues(B, a.wg_per_unit);
  dim3 grid((unsigned)(a.wg_per_unit * a.units));
  rc = launch_clear(wb, L.b_begin, L.b_end, s);          // records and tickets of this pass
  if (rc) return rc;
  {
    KernelTimer timer(1, s);
    RGLRU_DISPATCH(bwd_kernel, grid, s, a, dtype, held_groups(g, dtype, a.aligned));
  }
  rc = check_launch("bwd");
  if (rc) return rc;
  return gate_gemms_and_finish(a, g, prep, dtype, grad_dtype, x, du_a, du_x, W, g.bw, dx, (char*)scratch, B, T,
                               dw_a, dw_x, db_a, db_x, dlambda, s);
}

int rglru_hip_fast_path(int64_t W, int64_t nb, int dtype) {
  if (dtype != RGLRU_BF16 || W <= 0 || nb <= 0 || W % nb) return 0;
  const int64_t bw = W / nb;
  return (bw == 32 || bw == 64 || bw == 128) ? 1 : 0;
}

// tokens per tile of the reverse-scan kernel: 32 * kDeltaMT
#ifndef RGLRU_DELTA_MT
#define RGLRU_DELTA_MT 2
#endif
constexpr int kDeltaMT = RGLRU_DELTA_MT;

int rglru_hip_bwd_full(const void* x, const void* y, const void* prep, const float* h0,
                       const uint8_t* flags, const void* dy, const float* dh_last, void* ws, void* scratch,
                       void* dx, void* dw_a, void* dw_x, void* db_a, void* db_x, void* dlambda,
                       float* dh0, int64_t B, int64_t T, int64_t W, int64_t nb, int dtype, int grad_dtype,
                       void* stream) {
  int rc = check_geometry("bwd_full", W, nb, dtype);
  if (rc) return rc;
  rc = check_grad_dtype("bwd_full", grad_dtype);
  if (rc) return rc;
  if (!rglru_hip_fast_path(W, nb, dtype))
    return fail(RGLRU_E_UNSUPPORTED, "bwd_full: needs 16-bit storage and gate blocks of 32, 64 or 128 channels");
  if (B <= 0 || T <= 0) return fail(RGLRU_E_ARG, "bwd_full: B and T must be positive (got %lld, %lld)", (long long)B, (long long)T);
  if (!x || !y || !prep || !dy || !ws || !scratch || !dx || !dw_a || !dw_x || !db_a || !db_x || !dlambda)
    return fail(RGLRU_E_ARG, "bwd_full: null pointer");
  rc = check_extents("bwd_full", B, T, W);
  if (rc) return rc;
  Geometry g = make_geometry(W, nb);
  if (!is_aligned(x, W, g.bw, 2) || !is_aligned(y, W, g.bw, 2) || !is_aligned(dy, W, g.bw, 2) || !is_aligned(dx, W, g.bw, 2))
    return fail(RGLRU_E_UNSUPPORTED, "bwd_full: x, y, dy and dx must be 16-byte aligned");
  if ((uintptr_t)dw_a % 16 || (uintptr_t)dw_x % 16 || (uintptr_t)scratch % 16)
    return fail(RGLRU_E_UNSUPPORTED, "bwd_full: dw_a, dw_x and scratch must be 16-byte aligned");
  WorkLayout L = make_work_layout(B, T, g);
  hipStream_t s = (hipStream_t)stream;
  char* wb = (char*)ws;
  FusedArgs a;
  memset(&a, 0, sizeof(a));
  fill_common(a, g, prep, dtype);
  if (flags == RGLRU_FLAGS_FIRST_RESET) { flags = nullptr; a.first_reset = 1; }
  a.x = x; a.y = const_cast<void*>(y); a.h0 = h0; a.flags = flags; a.dy = dy; a.dh_last = dh_last;
  a.flags_vec = (T % 16 == 0) && ((uintptr_t)flags % 16 == 0);
  const ScratchLayout SL = make_scratch_layout(B, T, g, kScratchFast);
  char* sb = (char*)scratch;
  a.dx = dx; a.du_a = sb + SL.delta; a.dh0 = dh0;
  a.ckpt = (float*)(wb + L.ckpt); a.rec_a = (rec_t*)(wb + L.b_rec_a);
  a.ticket = (unsigned*)(wb + L.b_ticket); a.fail = (unsigned*)(wb + L.fail);
  a.partial = (float*)(sb + SL.partial); a.dw_partial = (float*)(sb + SL.dw_partial);
  a.B = (int)B; a.T = (int)T; a.nC = (int)((T + kChunk - 1) / kChunk); a.ckpt_nC = 2 * (int)L.nC;
  a.aligned = 1;
  const int nkg = held_groups(g, dtype, 1);
  pack_units(a, g, nkg);
#ifndef RGLRU_DW_BF16
#define RGLRU_DW_BF16 1
#endif
  // 16-bit weight gradients asked for: the per-workgroup sums (fp32 in registers over a workgroup's share of
  // the tokens) cross memory as bf16 too, which halves what the finish kernel reads back
  a.dw_bf16 = (RGLRU_DW_BF16 && grad_dtype == RGLRU_BF16) ? 1 : 0;
  // reverse scan: delta[B, T, W] (and dh0)
  const long long chunks = (T + 32 * kDeltaMT - 1) / (32 * kDeltaMT);
  a.wg_per_unit = pick_wg_per_unit(a.units, B * chunks, kDeltaMT == 1 ? 4 : RGLRU_DELTA_OCC, L.max_wg);
  a.queues = pick_queues(B, a.wg_per_unit);
  const bool masked = (flags != nullptr) || (T % (32 * kDeltaMT) != 0);
  dim3 grid((unsigned)(a.wg_per_unit * a.units));
  const bool chain_scan = fwd_chain_pays(B, T, W);
  if (chain_scan) {
    // enough chains to give every compute unit one of its own (see fwd_impl)
    const dim3 cgrid((unsigned)(8 * ((B * nb + 7) / 8) * (g.bw / 32)));
    const bool cmasked = (flags != nullptr) || (T % 32 != 0);
    KernelTimer timer(1, s);
#define RGLRU_LAUNCH_DELTA_CHAIN(N)                                                                                  \
    if (cmasked) hipLaunchKernelGGL((bwd_delta_chain_kernel<__bf16, N, true>), cgrid, dim3(kChainWaves * 64), 0, s, a); \
    else hipLaunchKernelGGL((bwd_delta_chain_kernel<__bf16, N, false>), cgrid, dim3(kChainWaves * 64), 0, s, a)
    if (nkg == 8) { RGLRU_LAUNCH_DELTA_CHAIN(8); } else if (nkg == 4) { RGLRU_LAUNCH_DELTA_CHAIN(4); } else { RGLRU_LAUNCH_DELTA_CHAIN(2); }
#undef RGLRU_LAUNCH_DELTA_CHAIN
  } else {
    rc = launch_clear(wb, L.b_begin, L.b_end, s);        // records and tickets of this pass
    if (rc) return rc;
    KernelTimer timer(1, s);
#define RGLRU_LAUNCH_DELTA(N)                                                                                        \
    if (masked) hipLaunchKernelGGL((bwd_delta_kernel<__bf16, N, true, kDeltaMT>), grid, dim3(kThreads), 0, s, a);      \
    else hipLaunchKernelGGL((bwd_delta_kernel<__bf16, N, false, kDeltaMT>), grid, dim3(kThreads), 0, s, a)
    if (nkg == 8) { RGLRU_LAUNCH_DELTA(8); } else if (nkg == 4) { RGLRU_LAUNCH_DELTA(4); } else { RGLRU_LAUNCH_DELTA(2); }
#undef RGLRU_LAUNCH_DELTA
  }
  rc = check_launch("bwd_full scan");
  if (rc) return rc;
  // gradients: one workgroup per compute unit, the same units
  int n_wg = num_compute_units() / a.units; if (n_wg < 1) n_wg = 1; if (n_wg > kGemmWgPerUnit) n_wg = kGemmWgPerUnit;
  const long long grad_tiles = B * ((T + 31) / 32);
  if (n_wg > grad_tiles) n_wg = (int)grad_tiles;
  const bool masked_grad = (flags != nullptr) || (T % 32 != 0);
  dim3 grid2((unsigned)(n_wg * a.units));
  {
    KernelTimer timer(3, s);
#define RGLRU_LAUNCH_GRAD(N)                                                                                          \
    if (masked_grad) hipLaunchKernelGGL((bwd_grad_kernel<__bf16, N, true>), grid2, dim3(kGradThreads), 0, s, a);         \
    else hipLaunchKernelGGL((bwd_grad_kernel<__bf16, N, false>), grid2, dim3(kGradThreads), 0, s, a)
    if (nkg == 8) { RGLRU_LAUNCH_GRAD(8); } else if (nkg == 4) { RGLRU_LAUNCH_GRAD(4); } else { RGLRU_LAUNCH_GRAD(2); }
#undef RGLRU_LAUNCH_GRAD
  }
  rc = check_launch("bwd_full gradients");
  if (rc) return rc;
  FinishArgs r;
  memset(&r, 0, sizeof(r));
  r.partial = a.partial; r.dsp = finish_dsp(g, prep, dtype); r.db_a = db_a; r.db_x = db_x; r.dlambda = dlambda;
  r.dw_partial = a.dw_partial; r.dw_a = dw_a; r.dw_x = dw_x;
  r.W = (int)W; r.nb = (int)nb; r.bw = (int)g.bw; r.bwp = (int)g.bwp; r.Wp = (int)g.Wp; r.wg_per_unit = n_wg;
  r.n_wg = n_wg; r.vec_blocks = (int)((W + 15) / 16); r.grad_dtype = grad_dtype; r.dw_bf16 = a.dw_bf16; r.dw_vec = 1;
  const long long total = nb * g.bw * 2 * g.bw;
  hipLaunchKernelGGL(finish_kernel, dim3((unsigned)(r.vec_blocks + (total / 8 + 255) / 256)), dim3(256), 0, s, r);
  return check_launch("bwd_full finish");
}

int rglru_hip_wide_path(int64_t W, int64_t nb, int dtype) {
  if (W <= 0 || nb <= 0 || W % nb) return 0;
  return wide_groups(make_geometry(W, nb), dtype, 1) != 0 ? 1 : 0;
}

int rglru_hip_backward_path(int64_t B, int64_t T, int64_t W, int64_t nb, int dtype, int aligned) {
  if (B <= 0 || T <= 0 || W <= 0 || nb <= 0 || W % nb || (dtype != RGLRU_F32 && dtype != RGLRU_BF16)) return -1;
  if (aligned && rglru_hip_fast_path(W, nb, dtype)) return fwd_chain_pays(B, T, W) ? RGLRU_PATH_FAST_CHAIN : RGLRU_PATH_FAST_TILED;
  if (aligned && rglru_hip_wide_path(W, nb, dtype)) return RGLRU_PATH_WIDE;
  if (aligned && rglru_hip_pre_path(W, nb, dtype)) return RGLRU_PATH_PRE;
  return RGLRU_PATH_PORTABLE;
}

int rglru_hip_bwd_wide(const void* x, const void* prep, const float* h0,
                       const uint8_t* flags, const void* dy, const float* dh_last, void* ws, void* scratch,
                       void* dx, void* dw_a, void* dw_x, void* db_a, void* db_x, void* dlambda,
                       float* dh0, int64_t B, int64_t T, int64_t W, int64_t nb, int dtype, int grad_dtype,
                       void* stream) {
  int rc = check_geometry("bwd_wide", W, nb, dtype);
  if (rc) return rc;
  rc = check_grad_dtype("bwd_wide", grad_dtype);
  if (rc) return rc;
  if (!rglru_hip_wide_path(W, nb, dtype))
    return fail(RGLRU_E_UNSUPPORTED, "bwd_wide: needs 16-bit storage and gate blocks of 160 to 384 channels in steps of 32");
  if (B <= 0 || T <= 0) return fail(RGLRU_E_ARG, "bwd_wide: B and T must be positive (got %lld, %lld)", (long long)B, (long long)T);
  if (!x || !prep || !dy || !ws || !scratch || !dx || !dw_a || !dw_x || !db_a || !db_x || !dlambda)
    return fail(RGLRU_E_ARG, "bwd_wide: null pointer");
  rc = check_extents("bwd_wide", B, T, W);
  if (rc) return rc;
  Geometry g = make_geometry(W, nb);
  if (!is_aligned(x, W, g.bw, 2) || !is_aligned(dy, W, g.bw, 2) || !is_aligned(dx, W, g.bw, 2))
    return fail(RGLRU_E_UNSUPPORTED, "bwd_wide: x, dy and dx must be 16-byte aligned");
  if ((uintptr_t)dw_a % 16 || (uintptr_t)dw_x % 16 || (uintptr_t)scratch % 16)
    return fail(RGLRU_E_UNSUPPORTED, "bwd_wide: dw_a, dw_x and scratch must be 16-byte aligned");
  WorkLayout L = make_work_layout(B, T, g);
  hipStream_t s = (hipStream_t)stream;
  char* wb = (char*)ws;
  FusedArgs a;
  memset(&a, 0, sizeof(a));
  fill_common(a, g, prep, dtype);
  if (flags == RGLRU_FLAGS_FIRST_RESET) { flags = nullptr; a.first_reset = 1; }
  a.x = x; a.h0 = h0; a.flags = flags; a.dy = dy; a.dh_last = dh_last;
  a.flags_vec = (T % 16 == 0) && ((uintptr_t)flags % 16 == 0);
  const ScratchLayout SL = make_scratch_layout(B, T, g, kScratchWide);
  char* sb = (char*)scratch;
  a.dx = dx; a.du_a = sb + SL.delta; a.dh0 = dh0;
  a.ckpt = (float*)(wb + L.ckpt); a.rec_a = (rec_t*)(wb + L.b_rec_a);
  a.ticket = (unsigned*)(wb + L.b_ticket); a.fail = (unsigned*)(wb + L.fail);
  a.partial = (float*)(sb + SL.partial); a.dw_partial = (float*)(sb + SL.dw_partial);
  a.B = (int)B; a.T = (int)T; a.nC = (int)((T + kChunk - 1) / kChunk); a.ckpt_nC = 2 * (int)L.nC; a.nCf = (int)L.nCf;
  a.aligned = 1;
  const int nkg = wide_groups(g, dtype, 1);
  // reverse scan and gate math: direct part of dx, du2, per-workgroup bias and Lambda sums
  a.wg_per_unit = pick_wg_per_unit(a.units, B * (long long)a.nC, 1, L.max_wg);
  a.queues = pick_queues(B, a.wg_per_unit);
  const bool masked = (flags != nullptr) || a.first_reset || (T % kChunk != 0);
  a.xcd_map = 1;
  dim3 grid((unsigned)(8 * (((long long)nb * a.wg_per_unit + 7) / 8) * a.groups));
  rc = launch_clear(wb, L.b_begin, L.b_end, s);          // records and tickets of this pass
  if (rc) return rc;
  {
    KernelTimer timer(1, s);
#define RGLRU_LAUNCH_WIDE_SCAN(N)                                                                                    \
    case N:                                                                                                          \
      if (masked) hipLaunchKernelGGL((bwd_scan_kernel<__bf16, N, true>), grid, dim3(kThreads), 0, s, a);              \
      else hipLaunchKernelGGL((bwd_scan_kernel<__bf16, N, false>), grid, dim3(kThreads), 0, s, a);                     \
      break
    switch (nkg) {
      RGLRU_LAUNCH_WIDE_SCAN(10); RGLRU_LAUNCH_WIDE_SCAN(12); RGLRU_LAUNCH_WIDE_SCAN(14); RGLRU_LAUNCH_WIDE_SCAN(16);
      RGLRU_LAUNCH_WIDE_SCAN(18); RGLRU_LAUNCH_WIDE_SCAN(20); RGLRU_LAUNCH_WIDE_SCAN(22); RGLRU_LAUNCH_WIDE_SCAN(24);
      default: return fail(RGLRU_E_UNSUPPORTED, "bwd_wide: no kernel for blocks of %lld channels", (long long)g.bw);
    }
#undef RGLRU_LAUNCH_WIDE_SCAN
  }
  rc = check_launch("bwd_wide scan");
  if (rc) return rc;
  // the two gate-gradient GEMMs: units of two slabs, one workgroup per compute unit
  const int grad_units = (int)(nb * ((g.S + 1) / 2));
  int n_wg = num_compute_units() / grad_units; if (n_wg < 1) n_wg = 1; if (n_wg > kWideWgPerUnit) n_wg = kWideWgPerUnit;
  const long long grad_tiles = (B * T + 31) / 32;
  if (n_wg > grad_tiles) n_wg = (int)grad_tiles;
  const int scan_wg_per_unit = a.wg_per_unit;
  a.wg_per_unit = n_wg;
  const long long grad_pairs = (long long)nb * n_wg;      // (block, tile sequence) pairs, dealt to the XCDs in rounds of eight
  dim3 grid2((unsigned)(8 * ((grad_pairs + 7) / 8) * ((g.S + 1) / 2)));
  {
    KernelTimer timer(3, s);
    switch (nkg) {
      case 10: hipLaunchKernelGGL((gate_grad_wide_kernel<__bf16, 10>), grid2, dim3(kGradThreads), 0, s, a); break;
      case 12: hipLaunchKernelGGL((gate_grad_wide_kernel<__bf16, 12>), grid2, dim3(kGradThreads), 0, s, a); break;
      case 14: hipLaunchKernelGGL((gate_grad_wide_kernel<__bf16, 14>), grid2, dim3(kGradThreads), 0, s, a); break;
      case 16: hipLaunchKernelGGL((gate_grad_wide_kernel<__bf16, 16>), grid2, dim3(kGradThreads), 0, s, a); break;
      case 18: hipLaunchKernelGGL((gate_grad_wide_kernel<__bf16, 18>), grid2, dim3(kGradThreads), 0, s, a); break;
      case 20: hipLaunchKernelGGL((gate_grad_wide_kernel<__bf16, 20>), grid2, dim3(kGradThreads), 0, s, a); break;
      case 22: hipLaunchKernelGGL((gate_grad_wide_kernel<__bf16, 22>), grid2, dim3(kGradThreads), 0, s, a); break;
      default: hipLaunchKernelGGL((gate_grad_wide_kernel<__bf16, 24>), grid2, dim3(kGradThreads), 0, s, a); break;
    }
  }
  rc = check_launch("bwd_wide gate gradients");
  if (rc) return rc;
  FinishArgs r;
  memset(&r, 0, sizeof(r));
  r.partial = a.partial; r.dsp = finish_dsp(g, prep, dtype); r.db_a = db_a; r.db_x = db_x; r.dlambda = dlambda;
  r.dw_partial = a.dw_partial; r.dw_a = dw_a; r.dw_x = dw_x;
  r.W = (int)W; r.nb = (int)nb; r.bw = (int)g.bw; r.bwp = (int)g.bwp; r.Wp = (int)g.Wp; r.wg_per_unit = scan_wg_per_unit;
  r.n_wg = n_wg; r.vec_blocks = (int)((W + 15) / 16); r.grad_dtype = grad_dtype; r.dw_vec = 1;
  const long long total = nb * g.bw * 2 * g.bw;
  hipLaunchKernelGGL(finish_kernel, dim3((unsigned)(r.vec_blocks + (total / 8 + 255) / 256)), dim3(256), 0, s, r);
  return check_launch("bwd_wide finish");
}


}  // extern "C"
