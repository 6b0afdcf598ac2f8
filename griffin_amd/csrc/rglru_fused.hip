// Fused RG-LRU kernels for gfx950: parameter preparation, forward, backward, decode step.
//
// Work decomposition.  The gates are block diagonal (griffin/griffin.py:129-154), so a tile of
// TR = 32 * MT tokens of one sequence and one gate block depends on nothing but the same tokens
// of that block.  A workgroup of four waves stages that x tile once in LDS; each wave owns one
// 32-channel slab of the block:
//   - the two gate pre-activations of its slab come from MFMA (rows = time, columns = channels,
//     K = the block's input channels), weights kept in registers when the block is <= 128 wide;
//   - the row permutation tile_row() makes every lane own a run of consecutive time steps of one
//     channel, so the gate math (griffin/griffin.py:237-255) and the recurrence
//     h_t = a_t h_{t-1} + z_t (griffin/griffin.py:279-284) run in registers, in time order;
//   - carries between tiles travel through the publish / look-back protocol of rglru_device.h.
// Workgroups are persistent: each is bound to one weight set ("unit" = gate block x group of four
// slabs) and pulls (chunk, sequence) tiles of that unit from a ticket counter, in chain order.

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstring>
#include <type_traits>

#include "rglru_device.h"
#include "rglru_host.h"
#include "rglru_layout.h"

namespace rglru {

// ------------------------------------------------------------------------------------------
// Parameter preparation
// ------------------------------------------------------------------------------------------
struct PrepArgs {
  const void* w_a; const void* w_x; const void* b_a; const void* b_x; const void* lambda;
  void* wg; float* bias; float* sp; float* cs; float* dsp; void* w2t;
  int W, nb, bw, bwp, Wp, vec_dtype;
  int vec_ok;                          // 16-bit weights, unpadded blocks, 16-byte aligned: eight elements per thread
  float c;
  uint4* clear; long long clear_n;     // optional: a workspace region to zero in the same launch
};

// Element i of a vector stored as fp32 or bf16 (RGLRU_F32 / RGLRU_BF16).
RGLRU_DEVICE float load_vec(const void* p, long long i, int dtype) {
  return dtype == RGLRU_BF16 ? (float)((const __bf16*)p)[i] : ((const float*)p)[i];
}
RGLRU_DEVICE void store_vec(void* p, long long i, float v, int dtype) {
  if (dtype == RGLRU_BF16) ((__bf16*)p)[i] = (__bf16)v; else ((float*)p)[i] = v;
}

RGLRU_DEVICE float log_sigmoid(float v) {
  return v >= 0.f ? -log1pf(expf(-v)) : v - log1pf(expf(v));
}

// Per-channel constants of padded channel kp: the two biases, c log sigmoid(Lambda) in natural and
// binary logarithm, and the factor of the Lambda gradient.
RGLRU_DEVICE void prepare_channel(const PrepArgs& p, int kp) {
  const int k = kp / p.bwp, o = kp - k * p.bwp;
  float ba = 0.f, bx = 0.f, sp = 0.f, cs = 0.f, dsp = 0.f;
  if (o < p.bw) {
    const int ch = k * p.bw + o;
    ba = load_vec(p.b_a, ch, p.vec_dtype); bx = load_vec(p.b_x, ch, p.vec_dtype);
    const float lam = load_vec(p.lambda, ch, p.vec_dtype);
    const float ls = log_sigmoid(lam);
    cs = p.c * ls;
    sp = cs * kLog2e;
    dsp = p.c / (1.0f + expf(lam));          // c * d/dLambda log sigmoid(Lambda) = c * sigmoid(-Lambda)
  }
  p.bias[kp] = ba; p.bias[p.Wp + kp] = bx; p.sp[kp] = sp; p.cs[kp] = cs; p.dsp[kp] = dsp;
}

template <typename IO>
__global__ void prepare_kernel(PrepArgs p) {
  const long long per_gate = (long long)p.nb * p.bwp * p.bwp;
  const long long n_w = 2 * per_gate;
  const long long total = 2 * n_w + p.Wp;
  long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x;
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long z = i; z < p.clear_n; z += stride) p.clear[z] = make_uint4(0u, 0u, 0u, 0u);
  if (sizeof(IO) == 2 && p.vec_ok) {
    // 16 bytes per thread: wg is a copy of [w_a ; w_x]; a vector of w2t is four output channels x two gates
    const long long per_gate8 = per_gate / 8, n_w8 = 2 * per_gate8;
    const int row8 = 2 * p.bw / 8;                         // vectors per row j of w2t
    const long long per_block8 = (long long)p.bw * row8;
    const unsigned short* wa = (const unsigned short*)p.w_a;
    const unsigned short* wx = (const unsigned short*)p.w_x;
    for (; i < 2 * n_w8 + p.Wp; i += stride) {
      if (i < n_w8) {
        const int gate = i >= per_gate8;
        ((uint4*)p.wg)[i] = ((const uint4*)(gate ? p.w_x : p.w_a))[i - gate * per_gate8];
      } else if (i < 2 * n_w8) {
        const long long e8 = i - n_w8;
        const int k = (int)(e8 / per_block8);
        const int rem = (int)(e8 - (long long)k * per_block8);
        const int j = rem / row8, c8 = rem - j * row8;
        const long long at = ((long long)k * p.bw + 4 * c8) * p.bw + j;   // W[k][4 c8][j]
        unsigned v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = (unsigned)wa[at + (long long)u * p.bw] | ((unsigned)wx[at + (long long)u * p.bw] << 16);
        ((uint4*)p.w2t)[e8] = make_uint4(v[0], v[1], v[2], v[3]);
      } else {
        prepare_channel(p, (int)(i - 2 * n_w8));
      }
    }
    return;
  }
  for (; i < total; i += stride) {
    if (i < n_w) {
      int gate = (int)(i / per_gate);
      long long rem = i - gate * per_gate;
      int k = (int)(rem / ((long long)p.bwp * p.bwp));
      int oj = (int)(rem - (long long)k * p.bwp * p.bwp);
      int o = oj / p.bwp, j = oj - o * p.bwp;
      float v = 0.f;
      if (o < p.bw && j < p.bw) {
        const IO* src = (const IO*)(gate ? p.w_x : p.w_a);
        v = (float)src[((long long)k * p.bw + o) * p.bw + j];
      }
      ((IO*)p.wg)[i] = (IO)v;
    } else if (i >= n_w + p.Wp) {
      // w2t[k][j][2 * o + gate]
      long long e = i - n_w - p.Wp;
      const long long per_block = 2ll * p.bwp * p.bwp;
      int k = (int)(e / per_block);
      int rem = (int)(e - (long long)k * per_block);
      int j = rem / (2 * p.bwp), kap = rem - j * 2 * p.bwp;
      int o = kap >> 1, gate = kap & 1;
      float v = 0.f;
      if (o < p.bw && j < p.bw) {
        const IO* src = (const IO*)(gate ? p.w_x : p.w_a);
        v = (float)src[((long long)k * p.bw + o) * p.bw + j];
      }
      ((IO*)p.w2t)[e] = (IO)v;
    } else {
      prepare_channel(p, (int)(i - n_w));
    }
  }
}


// ------------------------------------------------------------------------------------------
// Arguments common to the fused kernels
// ------------------------------------------------------------------------------------------
struct FusedArgs {
  // tensors
  const void* x; const void* pre; const void* wg; const float* bias; const float* sp; const float* cs; const void* w2t;
  const float* h0; const uint8_t* flags;
  void* y; float* h_last;                                 // forward
  const void* dy; const float* dh_last;                   // backward in
  void* dx; void* du_a; void* du_x; float* dh0;           // backward out
  float* h_state; const float* h_prev;                    // decode step: state out, state in (may be the same)
  const void* gate_v;                                     // decode step: y = h * gelu_tanh(gate_v) when set
  long long ld_gate;                                      // ... elements between rows of gate_v (>= W)
  // block forward: x = causal depthwise conv of the rows at `x` (taps by lag, carried rows in conv_state),
  // out `gated` = y * gelu_tanh(gate_v); x_out, y and conv_new_state are optional outputs
  const void* conv_state; const void* conv_taps; const void* conv_bias;
  void* x_out; void* conv_new_state; void* gated;
  long long ld_x;                                         // elements between rows of x (>= W)
  int conv_k, conv_vec_dtype;
  // chain forward that also prepares (rglru_hip_prepare_fwd): the caller's parameters, the image to build from
  // them and the workspace region to zero, all in the forward launch
  PrepArgs prep;
  // workspace
  float* ckpt; rec_t* rec_a; unsigned* ticket;
  unsigned* fail; float* partial; float* dw_partial;
  // geometry
  int B, T, W, nb, bw, bwp, S, Wp, groups, units;
  int bpu;                                                // gate blocks per unit (packed narrow blocks), else 1
  long long rows_total;                                   // B * T, the row count of one block of `pre`
  int nC, nCf, ckpt_nC, wg_per_unit, aligned, full_slabs, queues, flags_vec;
  int dw_bf16;                                            // fast backward: per-workgroup weight-gradient sums stored as bf16
  int xcd_map;                                            // wide blocks: the workgroups that share a block's x tiles sit on one XCD
  int first_reset;                                        // token 0 of every sequence carries RGLRU_FLAG_RESET (and flags is null)
  unsigned bw_magic;                                      // decode step: ceil(2^32 / bw), channel / bw as a multiply-high (channel < 2^16)
  long long limit;
};

// Ticket queues.  A unit's (chunk, sequence) tiles are dealt to `queues` counters: queue j owns the
// sequences b = j, j + queues, ...; its tickets enumerate them chunk-major, i.e. in chain order.  A
// workgroup serves queue wg_in_unit % queues.  Spreading the tickets keeps same-address atomics rare.
struct Queue {
  unsigned* counter; int first_b, n_b; long long tiles;
};
RGLRU_DEVICE Queue make_queue(const FusedArgs& p, int unit, int wg_in_unit, int chunks) {
  Queue q;
  const int j = wg_in_unit % p.queues;
  q.counter = p.ticket + unit * kMaxQueues + j;
  q.first_b = j;
  q.n_b = (p.B - j + p.queues - 1) / p.queues;
  q.tiles = (long long)q.n_b * chunks;
  return q;
}

// Identity of the wave inside its unit; shared by the kernels below.
struct WaveId {
  int lane, r, hf, wave, unit, wg_in_unit, k, slab, o, ch, kp;
  int tile_col, kb;          // first channel of the unit's x tile; offset of the wave's block inside it
  bool slab_ok, ch_ok;
};

// Width of the x tile of the kernels with register-held weights.  Blocks of 64 or 32 channels are
// packed two or four to a unit, so the four waves of a workgroup always have a slab each.
constexpr int kPackedWidth = 128;

RGLRU_DEVICE WaveId wave_identity(const FusedArgs& p, int block) {
  WaveId w;
  w.lane = threadIdx.x & 63; w.r = w.lane & 31; w.hf = w.lane >> 5; w.wave = threadIdx.x >> 6;
  w.unit = block % p.units; w.wg_in_unit = block / p.units;
  if (p.xcd_map) {
    // Workgroups go to the eight XCDs round-robin by index and each XCD has its own L2.  The `groups` units
    // of a wide block stage the same x tiles: index = xcd + 8 * slot keeps the members of a (block,
    // workgroup number) pair in consecutive slots of one XCD, so the tile comes from memory once.  The grid
    // is rounded up to whole rounds of eight pairs; a workgroup number past the end means "nothing to do".
    const int xcd = block & 7, slot = block >> 3;
    const int pair = xcd + 8 * (slot / p.groups);
    w.unit = (pair % p.nb) * p.groups + slot % p.groups;
    w.wg_in_unit = pair / p.nb;
  }
  if (p.bpu > 1) {
    // packed: the unit covers bpu consecutive blocks of S slabs each (bpu * S = waves per workgroup)
    const int blk = w.wave / p.S, k = w.unit * p.bpu + blk;
    w.slab = w.wave - blk * p.S;
    w.slab_ok = k < p.nb;
    w.k = w.slab_ok ? k : p.nb - 1;
    w.tile_col = w.unit * p.bpu * p.bw; w.kb = blk * p.bw;
  } else {
    w.k = w.unit / p.groups;
    w.slab = (w.unit % p.groups) * kWaves + w.wave;
    w.slab_ok = w.slab < p.S;
    w.tile_col = w.k * p.bw; w.kb = 0;
  }
  w.o = w.slab * 32 + w.r;
  w.ch_ok = w.slab_ok && w.o < p.bw;
  w.ch = w.k * p.bw + (w.ch_ok ? w.o : 0);
  w.kp = w.k * p.bwp + (w.slab_ok ? w.o : 0);
  return w;
}

// ------------------------------------------------------------------------------------------
// x tile staging.  A tile is TR consecutive rows (tokens, or sequences for the decode step) of one
// gate block, kept in LDS with row stride KS + HW elements.
// ------------------------------------------------------------------------------------------
template <typename IO>
RGLRU_DEVICE typename Io<IO>::Frag load_x_frag(const FusedArgs& p, const IO* xmat, long long grow,
                                               long long rows_total, int k, int col) {
  typedef Io<IO> Tr;
  typename Tr::Frag v = Tr::zero();
  if (grow < rows_total) {
    const IO* src = xmat + grow * (long long)p.W + (long long)k * p.bw + col;
    if (p.aligned && col + Tr::HW <= p.bw) {
      v = *reinterpret_cast<const typename Tr::Frag*>(src);
    } else {
#pragma unroll
      for (int e = 0; e < Tr::HW; ++e) if (col + e < p.bw) v[e] = src[e];
    }
  }
  return v;
}

// Gate pre-activations of one tile, generic variant (any block width, weights streamed from
// memory, K staged through LDS in slices of KCMAX).  On return ua/ux hold W x + b for the wave's
// slab (register v of tile mt <-> local row hf*16*MT + 16*mt + v) and xv the matching x values.
// Every thread of the workgroup must call this (it contains barriers).
template <typename IO, int MT>
RGLRU_DEVICE void gate_tile_generic(const FusedArgs& p, const IO* xmat, long long row0, long long rows_total,
                                    int k, int slab, bool slab_ok, const IO* w_a_row, const IO* w_x_row,
                                    float bias_a, float bias_x, IO* lds,
                                    f32x16 (&ua)[MT], f32x16 (&ux)[MT], float (&xv)[16 * MT]) {
  typedef Io<IO> Tr;
  typedef typename Tr::Frag Frag;
  constexpr int TR = 32 * MT;
  constexpr int KG = Tr::KG, HW = Tr::HW, KCMAX = Tr::KCMAX;
  constexpr int LDSROW = KCMAX + HW;
  const int tid = threadIdx.x, lane = tid & 63, r = lane & 31, hf = lane >> 5;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int v = 0; v < 16; ++v) { ua[mt][v] = bias_a; ux[mt][v] = bias_x; }
#pragma unroll
  for (int e = 0; e < 16 * MT; ++e) xv[e] = 0.f;

  for (int kc0 = 0; kc0 < p.bwp; kc0 += KCMAX) {
    const int kcw = (p.bwp - kc0) < KCMAX ? (p.bwp - kc0) : KCMAX;
    const int vecs = kcw / HW;
    for (int idx = tid; idx < TR * vecs; idx += kThreads) {
      const int row = idx / vecs, cv = idx - row * vecs;
      Frag v = load_x_frag<IO>(p, xmat, row0 + row, rows_total, k, kc0 + cv * HW);
      *reinterpret_cast<Frag*>(lds + row * LDSROW + cv * HW) = v;
    }
    __syncthreads();
    if (slab_ok) {
      for (int kk = 0; kk < kcw; kk += KG) {
        Frag fa = *reinterpret_cast<const Frag*>(w_a_row + kc0 + kk);
        Frag fx = *reinterpret_cast<const Frag*>(w_x_row + kc0 + kk);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          Frag xa = *reinterpret_cast<const Frag*>(lds + tile_row<MT>(mt, r) * LDSROW + kk + hf * HW);
          Tr::mma(ua[mt], xa, fa);
          Tr::mma(ux[mt], xa, fx);
        }
      }
      const int own = slab * 32 - kc0;                    // first column of this wave's slab in the slice
      if (own >= 0 && own < kcw) {
#pragma unroll
        for (int e = 0; e < 16 * MT; ++e) xv[e] = (float)lds[(hf * 16 * MT + e) * LDSROW + own + r];
      }
    }
    __syncthreads();
  }
}

// Register-resident weights: the wave's 32 rows of both gate matrices, NKG K groups each.
template <typename IO, int NKG>
struct HeldWeights {
  typename Io<IO>::Frag a[NKG > 0 ? NKG : 1], x[NKG > 0 ? NKG : 1];
  RGLRU_DEVICE void load(const IO* w_a_row, const IO* w_x_row) {
    if constexpr (NKG > 0) {
#pragma unroll
      for (int kg = 0; kg < NKG; ++kg) {
        a[kg] = *reinterpret_cast<const typename Io<IO>::Frag*>(w_a_row + kg * Io<IO>::KG);
        x[kg] = *reinterpret_cast<const typename Io<IO>::Frag*>(w_x_row + kg * Io<IO>::KG);
      }
    }
  }
};

// MFMA phase for register-held weights, one accumulator tile: the whole block width (NKG * KG
// columns) is in LDS with row stride NKG * KG + HW.  Also returns the 16 x values of the tile in
// accumulator layout.
template <typename IO, int MT, int NKG, int TW = NKG * Io<IO>::KG>
RGLRU_DEVICE void gate_mfma_held(const IO* lds, const HeldWeights<IO, NKG>& hw, int mt, int slab, int r, int hf,
                                 float bias_a, float bias_x, f32x16& ua, f32x16& ux, float (&xv)[16], int kb = 0) {
  typedef Io<IO> Tr;
  typedef typename Tr::Frag Frag;
  constexpr int KG = Tr::KG, HW = Tr::HW;
  constexpr int LDSROW = TW + HW;                          // the tile is TW columns wide; the block starts at kb
#pragma unroll
  for (int v = 0; v < 16; ++v) { ua[v] = bias_a; ux[v] = bias_x; }
  const IO* row = lds + tile_row<MT>(mt, r) * LDSROW + kb + hf * HW;
#pragma unroll
  for (int kg = 0; kg < NKG; ++kg) {
    Frag xa = *reinterpret_cast<const Frag*>(row + kg * KG);
    Tr::mma(ua, xa, hw.a[kg]);
    Tr::mma(ux, xa, hw.x[kg]);
  }
#pragma unroll
  for (int e = 0; e < 16; ++e) xv[e] = (float)lds[(hf * 16 * MT + 16 * mt + e) * LDSROW + kb + slab * 32 + r];
}

RGLRU_DEVICE unsigned token_flag(const FusedArgs& p, long long token_row, bool inside) {
  if (!inside) return RGLRU_FLAG_INACTIVE;
  return p.flags ? (unsigned)p.flags[token_row] & 3u : 0u;   // bits 2-3 belong to the block forward's convolution
}

// Flags of a lane's run of 16 consecutive tokens, two bits per token (token e at bits 2e, 2e + 1);
// tokens past the end of the sequence read as inactive.  When the sequence length is a multiple of
// 16 and the flag array is 16-byte aligned (flags_vec), a run is wholly inside or outside the
// sequence and its flags are one 16-byte load.
RGLRU_DEVICE unsigned pack_flag_bytes(unsigned d) {
  unsigned t = d & 0x03030303u;
  t = (t | (t >> 6)) & 0x000F000Fu;
  return (t | (t >> 12)) & 0xFFu;
}
RGLRU_DEVICE unsigned flag_run(const FusedArgs& p, long long token_row, int t_first) {
  // first_reset: "every sequence starts a document" without a flag array (the run that holds token 0)
  const unsigned first = (p.first_reset && t_first == 0) ? RGLRU_FLAG_RESET : 0u;
  if (p.flags_vec) {
    if (t_first >= p.T) return 0xAAAAAAAAu;
    if (!p.flags) return first;
    const uint4 w = *reinterpret_cast<const uint4*>(p.flags + token_row);
    return pack_flag_bytes(w.x) | (pack_flag_bytes(w.y) << 8) | (pack_flag_bytes(w.z) << 16) | (pack_flag_bytes(w.w) << 24) | first;
  }
  unsigned bits = first;
#pragma unroll
  for (int e = 0; e < 16; ++e) bits |= token_flag(p, token_row + e, t_first + e < p.T) << (2 * e);
  return bits;
}

// ------------------------------------------------------------------------------------------
// Forward
// ------------------------------------------------------------------------------------------
// Gate math of 16 consecutive local steps (first = index of the first one in this lane's run).
// MASKED = false is the common case: no flags, the tile lies inside the sequence.
// reset0 (plain variant only): the run's first token starts a document although there is no flag array.
template <typename IO, bool MASKED>
RGLRU_DEVICE void fwd_gates(unsigned flbits, const f32x16& ua, const f32x16& ux,
                            const float (&xv)[16], float sp, float* a, float* z, float nba = 0.0f, float nbx = 0.0f,
                            bool reset0 = false) {
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    GateOut go;
    if constexpr (MASKED) go = gate_forward_run<Precise<IO>::value>(ua[v], ux[v], xv[v], sp, flbits, v, nba, nbx);
    else if (v == 0) go = gate_forward<Precise<IO>::value, true>(ua[v], ux[v], xv[v], sp, reset0 ? RGLRU_FLAG_RESET : 0u, nba, nbx);
    else go = gate_forward<Precise<IO>::value, false>(ua[v], ux[v], xv[v], sp, 0u, nba, nbx);
    a[v] = go.a; z[v] = go.z;
  }
}

// records a forward walk requests per round trip (see carry_compose)
#ifndef RGLRU_FWD_DEPTH
#define RGLRU_FWD_DEPTH 2
#endif
constexpr int kFwdDepth = RGLRU_FWD_DEPTH;

// One wave's tile of 32 * MT tokens between its two stages: gate outputs in time order, the affine
// maps of the lower lane run and of the whole tile, and where the tile sits.
template <int MT>
struct FwdTile {
  float a[16 * MT], z[16 * MT];
  float A_lo, H_lo, A_t, H_t;
  int b, c;
};

// Descriptor of one sequence's forward carry records.
RGLRU_DEVICE rsrc_t seq_records(const FusedArgs& p, int b) {
  return make_rsrc(p.rec_a + (long long)b * p.nCf * p.W, (unsigned)p.nCf * (unsigned)p.W * 8u);
}

// Stage 1: affine map of the tile from (a, z); publishes it unless the tile starts its chain.
template <int MT, bool MASKED>
RGLRU_DEVICE void fwd_local(const FusedArgs& p, const WaveId& w, FwdTile<MT>& t, bool live = true) {
  constexpr int EL = 16 * MT;
  const int hf = w.hf;
  float A = 1.f, H = 0.f;
#pragma unroll
  for (int e = 0; e < EL; ++e) { H = fmaf(t.a[e], H, t.z[e]); A *= t.a[e]; }
  const float A_o = xhalf(A, hf), H_o = xhalf(H, hf);
  t.A_lo = hf ? A_o : A; t.H_lo = hf ? H_o : H;
  const float A_hi = hf ? A : A_o, H_hi = hf ? H : H_o;
  t.A_t = A_hi * t.A_lo; t.H_t = fmaf(A_hi, t.H_lo, H_hi);
  const bool ch_ok = (MASKED ? w.ch_ok : true) && live;
  // every store of the pipelined loop is issued unconditionally and masked through its offset, so
  // the number of memory operations in flight is the same on every path
  const unsigned voff = (t.c != 0 && ch_ok && hf == 0) ? ((unsigned)t.c * (unsigned)p.W + (unsigned)w.ch) * 8u : kOutOfRange;
  rec_store_buf(seq_records(p, t.b), voff, t.A_t, t.H_t);
}

// Stage 2: carry in, carry out and checkpoint, then the recurrence itself and the stores.
template <typename IO, int MT, bool MASKED, bool STAGED, bool BLOCK = false>
RGLRU_DEVICE void fwd_finalize(const FusedArgs& p, const WaveId& w, const FwdTile<MT>& t, unsigned char* stage,
                               const CarryBatch<kFwdDepth>* first = nullptr, bool live = true,
                               const bf16x8* gate_rows = nullptr) {
  constexpr int EL = 16 * MT, TR = 32 * MT;
  const int hf = w.hf, b = t.b, c = t.c;
  const long long W = p.W;
  const int t0 = c * TR;
  const bool ch_ok = (MASKED ? w.ch_ok : true) && live;     // a dead call stores nothing
  CarryChain chain;
  chain.rec = p.rec_a + (long long)b * p.nCf * W + w.ch; chain.stride = W;

  float h_in = 0.f;
  if (c != 0) {
    h_in = first ? carry_lookback_from<kFwdDepth>(*first, chain, c, -1, -1, 0.f, ch_ok, p.limit, p.fail)
                 : carry_lookback<kFwdDepth>(chain, c, -1, -1, 0.f, ch_ok, p.limit, p.fail);
  } else if (p.h0 && ch_ok) {
    h_in = p.h0[(long long)b * W + w.ch];
  }
  const float h_end = fmaf(t.A_t, h_in, t.H_t);
  const float h_mid = fmaf(t.A_lo, h_in, t.H_lo);
  {
    // carry out, checkpoint(s) and final state: unconditional stores masked through their offsets
    const unsigned uW = (unsigned)W, ch = (unsigned)w.ch;
    const bool lower = ch_ok && hf == 0;
    rec_store_buf(seq_records(p, b), lower ? ((unsigned)c * uW + ch) * 8u : kOutOfRange, 0.f, h_end);
    const rsrc_t rhl = make_rsrc(p.h_last, p.h_last ? (unsigned)p.B * uW * 4u : 0u);
    BufIo<float>::store(h_end, rhl, (lower && c == p.nCf - 1) ? ((unsigned)b * uW + ch) * 4u : kOutOfRange, 0u);
  }

  float h = hf ? h_mid : h_in;
  // checkpoints for the backward pass: the state after every 16 tokens (slot = token / 16); slots past
  // the end of the buffer are dropped by the descriptor
  const rsrc_t rck = make_rsrc(p.ckpt + (long long)b * p.ckpt_nC * W, (unsigned)p.ckpt_nC * (unsigned)W * 4u);
  unsigned ck_off[MT];
#pragma unroll
  for (int g16 = 0; g16 < MT; ++g16)
    ck_off[g16] = ch_ok ? ((unsigned)(c * 2 * MT + hf * MT + g16) * (unsigned)W + (unsigned)w.ch) * 4u : kOutOfRange;
  // y tile through a buffer descriptor: rows past the end of the sequence are dropped
  const int rows = !live ? 0 : ((p.T - t0) < TR ? (p.T - t0) : TR);
  const unsigned row_bytes = (unsigned)p.W * (unsigned)sizeof(IO);
  const rsrc_t ry = make_rsrc((const IO*)p.y + ((long long)b * p.T + t0) * W, (BLOCK && !p.y) ? 0u : (unsigned)rows * row_bytes);
  if constexpr (STAGED) {
    // 16-bit outputs: transpose through the wave's staging area, then 16-byte stores
    unsigned char* my = stage + WaveStage<TR>::row_offset(hf * EL) + w.r * 2;
#pragma unroll
    for (int e = 0; e < EL; ++e) {
      h = fmaf(t.a[e], h, t.z[e]);
      *reinterpret_cast<IO*>(my + e * WaveStage<TR>::kRowBytes) = (IO)h;
      if ((e & 15) == 15) BufIo<float>::store(h, rck, ck_off[e >> 4], 0u);
    }
    wave_lds_fence();
    if constexpr (BLOCK) {
      // output gate at the store: a lane holds the same 8 channels of a row of y and of the gate input
      const rsrc_t rg = make_rsrc((const IO*)p.gated + ((long long)b * p.T + t0) * W, (unsigned)rows * row_bytes);
      const unsigned col_bytes = (unsigned)(w.k * p.bw + w.slab * 32) * 2u;
#pragma unroll
      for (int i = 0; i < TR / 16; ++i) {
        const int row = 16 * i + (w.lane >> 2);
        const unsigned seg = (unsigned)(w.lane & 3) * 16u;
        const i32x4 raw = *reinterpret_cast<const i32x4*>(stage + WaveStage<TR>::row_offset(row) + seg);
        const unsigned off = (unsigned)row * row_bytes + col_bytes + seg;
        buf_store_b128(raw, ry, off);                       // y itself: dropped unless the caller keeps it
        const bf16x8 hv = __builtin_bit_cast(bf16x8, raw);
        bf16x8 out;
#pragma unroll
        for (int e = 0; e < 8; ++e) out[e] = (__bf16)((float)hv[e] * gelu_tanh_parts((float)gate_rows[i][e]).gelu);
        buf_store_b128(__builtin_bit_cast(i32x4, out), rg, off);
      }
    } else {
      stage_flush<TR>(stage, ry, row_bytes, (unsigned)(w.k * p.bw + w.slab * 32) * 2u, w.lane);
    }
    wave_lds_fence();
  } else {
    unsigned voff = ch_ok ? (unsigned)(hf * EL) * row_bytes + (unsigned)w.ch * (unsigned)sizeof(IO) : kOutOfRange;
#pragma unroll
    for (int e = 0; e < EL; ++e) {
      h = fmaf(t.a[e], h, t.z[e]);
      BufIo<IO>::store((IO)h, ry, voff + (unsigned)e * row_bytes, 0u);
      if ((e & 15) == 15) BufIo<float>::store(h, rck, ck_off[e >> 4], 0u);
    }
  }
}

// Forward tile = 32 * kFwdMT tokens; a tile is finished in the iteration that computed it.  64-token
// tiles halve the look-backs, barriers, tickets and records per token (39.6 us against 43.5 us for
// 32-token tiles with two tiles in flight at B8 T2048 W1024, 84 us against 104 us for one sequence of
// 32768 tokens).
constexpr int kFwdMT = 2;
// ... except where a block wider than 128 channels needs the registers: each wave holds 8 NKG registers of
// weights, and with one wave a SIMD nothing covers a tile's latency chain.  Measured per block width at
// B1 T32768 and B4 T2048 (forward, ms; 64-token tiles and one workgroup a compute unit first):
//   160: 0.185 -> 0.147, 192: 0.224 -> 0.161, 224: 0.199 -> 0.176 with 64-token tiles and two workgroups
//   (224: 7 spilled registers); 288: 0.370 -> 0.302, 320: 0.390 -> 0.347 with 32-token tiles and two
//   workgroups (320: 14 spilled registers); 256, 352, 384 are fastest as they were.
constexpr int fwd_mt(int nkg) { return (nkg == 18 || nkg == 20) ? 1 : kFwdMT; }
constexpr int fwd_wide_occ(int nkg) { return (nkg == 16 || nkg > 20) ? 1 : 2; }

// workgroups per compute unit of the forward kernel without weights in registers (NKG < 0); 4 spills
#define RGLRU_GIVEN_OCC 3
// ... and with the weights of 64- or 32-wide blocks (NKG = 4, 2): 150-168 registers, three fit
#ifndef RGLRU_NARROW_OCC
#define RGLRU_NARROW_OCC 3
#endif
// BLOCK: the recurrent block's forward around the scan in the same launch (griffin/griffin.py:474-487 in
// front, :464 and :520 behind).  The rows at p.x are the block's first projection; a lane loads four
// consecutive rows of eight channels plus the three rows in front of them, convolves them (taps by lag
// from LDS, lags masked per token through bits 2-3 of the flag bytes = 3 - min(position, 3)) and puts the
// result where the plain kernel puts x; the store stage multiplies by gelu_tanh of the second projection.
template <typename IO, int NKG, bool MASKED, bool BLOCK = false>
__global__ __launch_bounds__(kThreads, (BLOCK ? 2 : NKG < 0 ? RGLRU_GIVEN_OCC : (NKG == 4 || NKG == 2) ? RGLRU_NARROW_OCC : NKG > 8 ? fwd_wide_occ(NKG) : 2)) void fwd_kernel(FusedArgs p) {
  constexpr int MT = fwd_mt(NKG), TR = 32 * MT, EL = 16 * MT;
  static_assert(!BLOCK || (sizeof(IO) == 2 && (NKG == 8 || NKG == 4 || NKG == 2)), "block forward: 16-bit storage, register-held weights");
  typedef Io<IO> Tr;
  typedef typename Tr::Frag Frag;
  // NKG > 0: gate weights held in registers, pre-activations on MFMA.  Up to NKG = 8 (128 channels) a
  // workgroup covers a whole block (or several narrow ones); a wider block (NKG = bw / 16 > 8) is
  // shared by `groups` workgroups of four 32-channel slabs each, every one of which stages the block's
  // whole x tile and holds its slabs' rows of both matrices (8 NKG registers a lane, one wave a SIMD).
  // NKG < 0: the caller supplies the pre-activations.  NKG == 0: the portable path (any width,
  // alignment and storage type), weights streamed.
  constexpr bool GIVEN = NKG < 0;
  constexpr int KC = NKG > 8 ? NKG * Tr::KG : NKG != 0 ? kPackedWidth : Tr::KCMAX;   // LDS tile width in elements
  constexpr int LDSROW = KC + Tr::HW;
  __shared__ __attribute__((aligned(16))) IO lds[TR * LDSROW];
  __shared__ __attribute__((aligned(16))) IO lds_pre[GIVEN ? 2 * TR * LDSROW : Tr::HW];   // W_a x | W_x x tiles
  __shared__ __attribute__((aligned(16))) unsigned char stage_all[kWaves * WaveStage<TR>::kBytes];
  __shared__ unsigned s_ticket[2];
  __shared__ __attribute__((aligned(16))) float conv_w[BLOCK ? 5 * KC : 4];    // taps of lag 0..3, then the bias

  const WaveId w = wave_identity(p, blockIdx.x);
  if (w.wg_in_unit >= p.wg_per_unit) return;             // only with xcd_map: the grid's last round is not full
  const int hf = w.hf, tid = threadIdx.x;
  unsigned char* stage = stage_all + w.wave * WaveStage<TR>::kBytes;
  if constexpr (BLOCK) {
    // read after the barrier that follows the first ticket
    for (int i = tid; i < 5 * KC; i += kThreads) {
      const int j = i / KC, ch = w.tile_col + (i - j * KC);
      float v = 0.f;
      if (ch < p.W) {
        if (j == 4) { if (p.conv_bias) v = p.conv_vec_dtype == RGLRU_BF16 ? (float)((const __bf16*)p.conv_bias)[ch] : ((const float*)p.conv_bias)[ch]; }
        else if (j < p.conv_k) {
          const long long at = (long long)ch * p.conv_k + (p.conv_k - 1 - j);     // the tap of lag j
          v = p.conv_vec_dtype == RGLRU_BF16 ? (float)((const __bf16*)p.conv_taps)[at] : ((const float*)p.conv_taps)[at];
        }
      }
      conv_w[i] = v;
    }
  }
  const IO* wg = (const IO*)p.wg;
  const IO* w_a_row = wg + ((long long)(0 * p.nb + w.k) * p.bwp + (w.slab_ok ? w.o : 0)) * p.bwp + hf * Tr::HW;
  const IO* w_x_row = wg + ((long long)(1 * p.nb + w.k) * p.bwp + (w.slab_ok ? w.o : 0)) * p.bwp + hf * Tr::HW;
  // the biases enter inside the sigmoids (as -log2(e) * b), the matrix products start from zero
  const float nba = -kLog2e * p.bias[w.kp], nbx = -kLog2e * p.bias[p.Wp + w.kp];
  const float sp = w.ch_ok ? p.sp[w.kp] : 0.f;
  const IO* x = (const IO*)p.x;
  const long long W = p.W;
  const Queue q = make_queue(p, w.unit, w.wg_in_unit, p.nCf);

  if constexpr (NKG != 0) {
    // software-pipelined loop: the next ticket is taken while the current tile's MFMAs run and the
    // next x tile is requested right before the wave starts waiting for its carry
    HeldWeights<IO, NKG> hw;
    hw.load(w_a_row, w_x_row);
    constexpr int VPR = KC / Tr::HW;                     // 16-byte vectors per tile row
    constexpr int NV = (TR * VPR + kThreads - 1) / kThreads;
    Frag pre[NV], pre_a[GIVEN ? NV : 1], pre_x[GIVEN ? NV : 1];
    const unsigned row_bytes = (unsigned)p.W * (unsigned)sizeof(IO);
    // GIVEN: the tiles hold the 128 channels of this workgroup's four slabs, not the block's K range
    const int group_col = GIVEN ? (w.unit % p.groups) * KC : 0;
    const int x_col = GIVEN ? w.k * p.bw + group_col : w.tile_col;
    const unsigned u_row_bytes = 2u * (unsigned)p.bw * (unsigned)sizeof(IO);   // a row of `pre`: W_a x | W_x x of one block
    unsigned pre_off[NV];                                // lane offsets inside a tile (fixed)
    unsigned u_off[GIVEN ? NV : 1];
    // BLOCK: rows 4 rho .. 4 rho + 3 of channel vector bcv; the descriptor starts three rows before the tile
    static_assert(!BLOCK || (NV == 4 && VPR == 16), "block forward: four rows of a 128-channel tile per lane");
    const int rho = tid / VPR, bcv = tid - rho * VPR;
    const unsigned x_row_bytes = BLOCK ? (unsigned)p.ld_x * (unsigned)sizeof(IO) : row_bytes;
    const bool bcol_ok = BLOCK && (x_col + bcv * Tr::HW < p.W);
    const unsigned bcol_bytes = (unsigned)(x_col + bcv * Tr::HW) * (unsigned)sizeof(IO);
    Frag halo[BLOCK ? 3 : 1];
    unsigned conv_fl = 0u;                               // flag bytes of the lane's four rows
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int idx = tid + i * kThreads;
      const int row = idx / VPR, cv = idx - row * VPR;
      if constexpr (BLOCK)
        pre_off[i] = bcol_ok ? (unsigned)(4 * rho + i + 3) * x_row_bytes + bcol_bytes : kOutOfRange;
      else
      pre_off[i] = (idx < TR * VPR) ? (unsigned)row * row_bytes + (unsigned)(x_col + cv * Tr::HW) * (unsigned)sizeof(IO)
                                    : kOutOfRange;
      if constexpr (GIVEN)
        u_off[i] = (idx < TR * VPR) ? (unsigned)row * u_row_bytes + (unsigned)(group_col + cv * Tr::HW) * (unsigned)sizeof(IO)
                                    : kOutOfRange;
    }
    auto issue = [&](long long tk_in) {
      // a ticket past the end keeps valid addresses (tile 0) but an empty extent: nothing is fetched
      const bool live = tk_in < q.tiles;
      const unsigned tk = live ? (unsigned)tk_in : 0u;
      const int c = (int)(tk / (unsigned)q.n_b), b = q.first_b + (int)(tk - (unsigned)c * (unsigned)q.n_b) * p.queues;
      const int rows = !live ? 0 : ((p.T - c * TR) < TR ? (p.T - c * TR) : TR);
      if constexpr (BLOCK) {
        const rsrc_t rx = make_rsrc(x + ((long long)b * p.T + (long long)c * TR - 3) * p.ld_x, rows ? (unsigned)(rows + 3) * x_row_bytes : 0u);
#pragma unroll
        for (int i = 0; i < NV; ++i) pre[i] = buf_load_frag<Frag>(rx, pre_off[i]);
        // the rows in front of a sequence are the carried state (fetched where the tile is consumed) or zero
        const bool front = c == 0 && rho == 0;
#pragma unroll
        for (int h = 0; h < 3; ++h)
          halo[h] = buf_load_frag<Frag>(rx, (front || !bcol_ok) ? kOutOfRange : (unsigned)(4 * rho + h) * x_row_bytes + bcol_bytes);
        if constexpr (MASKED) {
          const rsrc_t rf = make_rsrc(p.flags + (long long)b * p.T + (long long)c * TR, p.flags ? (unsigned)rows : 0u);
          if (p.flags_vec) {
            conv_fl = (unsigned)__builtin_amdgcn_raw_buffer_load_b32(rf, (unsigned)(4 * rho), 0, 0);
          } else {
            conv_fl = 0u;
#pragma unroll
            for (int i = 0; i < 4; ++i) conv_fl |= ((unsigned)__builtin_amdgcn_raw_buffer_load_b8(rf, (unsigned)(4 * rho + i), 0, 0) & 0xffu) << (8 * i);
          }
        }
      } else {
      const rsrc_t rx = make_rsrc(x + ((long long)b * p.T + (long long)c * TR) * W, (unsigned)rows * row_bytes);
#pragma unroll
      for (int i = 0; i < NV; ++i) pre[i] = buf_load_frag<Frag>(rx, pre_off[i]);
      }
      if constexpr (GIVEN) {
        // the x-gate half of a row starts bw elements after the a-gate half
        const IO* ubase = (const IO*)p.pre + ((long long)w.k * p.rows_total + (long long)b * p.T + (long long)c * TR) * (2 * p.bw);
        const rsrc_t ru = make_rsrc(ubase, (unsigned)rows * u_row_bytes);
        const unsigned half = (unsigned)p.bw * (unsigned)sizeof(IO);
#pragma unroll
        for (int i = 0; i < NV; ++i) {
          pre_a[i] = buf_load_frag<Frag>(ru, u_off[i]);
          pre_x[i] = buf_load_frag<Frag>(ru, u_off[i] == kOutOfRange ? kOutOfRange : u_off[i] + half);
        }
      }
    };
    if (tid == 0) s_ticket[0] = atomicAdd(q.counter, 1u);
    __syncthreads();
    long long tk = s_ticket[0];
    int par = 0;
    issue(tk);
    FwdTile<MT> cur;
    cur.b = 0; cur.c = 0;
#pragma unroll
    for (int e = 0; e < EL; ++e) { cur.a[e] = 0.f; cur.z[e] = 0.f; }
    cur.A_lo = cur.H_lo = cur.A_t = cur.H_t = 0.f;
    // every wave has a slab except in the last unit of a block count that does not fill it
    const bool slab_ok = (NKG == 8) ? true : w.slab_ok;
    const rsrc_t rticket = make_rsrc(q.counter, 4u);
    const unsigned rec_stride = (unsigned)W * 8u;
    const unsigned rec_lane = (slab_ok && w.ch_ok) ? (unsigned)w.ch * 8u : kOutOfRange;
    // A dead finalize in front of the loop: the loop is entered with the same memory operations in
    // flight as its back edge has, so the waits at its top are exact instead of worst case.
    bf16x8 gate_rows[BLOCK ? TR / 16 : 1];               // the lane's vectors of the second projection
    if constexpr (BLOCK) {
#pragma unroll
      for (int i = 0; i < TR / 16; ++i) gate_rows[i] = Io<__bf16>::zero();
    }
    fwd_finalize<IO, MT, MASKED, sizeof(IO) == 2, BLOCK>(p, w, cur, stage, nullptr, false, gate_rows);
    while (tk < q.tiles) {
      cur.c = (int)((unsigned)tk / (unsigned)q.n_b);
      cur.b = q.first_b + (int)((unsigned)tk - (unsigned)cur.c * (unsigned)q.n_b) * p.queues;
      const long long trow = (long long)cur.b * p.T + cur.c * TR + hf * EL;
      // token flags of this lane's runs: requested first, so that the gate math waits for nothing younger
      unsigned flbits[MT];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) flbits[mt] = MASKED ? flag_run(p, trow + 16 * mt, cur.c * TR + hf * EL + 16 * mt) : 0u;
      // next ticket: one instruction for the whole workgroup, live only in its first lane
      const unsigned next_raw = (unsigned)__builtin_amdgcn_raw_ptr_buffer_atomic_add_i32(1, rticket, tid == 0 ? 0u : kOutOfRange, 0, 0);
      // records this tile will need: requested now, used after its gate math
      CarryBatch<kFwdDepth> ahead;
      carry_prefetch<kFwdDepth>(make_rsrc(p.rec_a + (long long)cur.b * p.nCf * W, (unsigned)p.nCf * rec_stride), rec_lane,
                       rec_stride, cur.c, -1, -1, ahead);
      if constexpr (BLOCK) {
        const int t0 = cur.c * TR;
        const int rows = (p.T - t0) < TR ? (p.T - t0) : TR;
        Frag um[7] = {halo[0], halo[1], halo[2], pre[0], pre[1], pre[2], pre[3]};      // tokens t0 + 4 rho - 3 .. + 3
        if (cur.c == 0 && p.conv_state && rho == 0 && bcol_ok) {
          // carried rows of the previous call: state row j holds the token K - 1 - j steps back
          const int K1 = p.conv_k - 1;
          const rsrc_t rs = make_rsrc((const IO*)p.conv_state + (long long)cur.b * K1 * W, (unsigned)K1 * row_bytes);
#pragma unroll
          for (int h = 0; h < 3; ++h) {
            const int j = K1 - 3 + h;
            um[h] = buf_load_frag<Frag>(rs, j >= 0 ? (unsigned)j * row_bytes + bcol_bytes : kOutOfRange);
          }
        }
        float tap[4][8], cbias[8];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const f32x4 lo = *reinterpret_cast<const f32x4*>(conv_w + j * KC + bcv * 8);
          const f32x4 hi = *reinterpret_cast<const f32x4*>(conv_w + j * KC + bcv * 8 + 4);
#pragma unroll
          for (int e = 0; e < 4; ++e) { tap[j][e] = lo[e]; tap[j][4 + e] = hi[e]; }
        }
        {
          const f32x4 lo = *reinterpret_cast<const f32x4*>(conv_w + 4 * KC + bcv * 8);
          const f32x4 hi = *reinterpret_cast<const f32x4*>(conv_w + 4 * KC + bcv * 8 + 4);
#pragma unroll
          for (int e = 0; e < 4; ++e) { cbias[e] = lo[e]; cbias[4 + e] = hi[e]; }
        }
        const rsrc_t rxo = make_rsrc((const IO*)p.x_out + ((long long)cur.b * p.T + t0) * W, p.x_out ? (unsigned)rows * row_bytes : 0u);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int hidden = MASKED ? (int)((conv_fl >> (8 * i + 2)) & 3u) : 0;        // lags 4 - hidden .. 3 do not apply
          Frag out;
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            float a = fmaf((float)um[3 + i][e], tap[0][e], cbias[e]);
#pragma unroll
            for (int lag = 1; lag < 4; ++lag) {
              const float with = fmaf((float)um[3 + i - lag][e], tap[lag][e], a);
              a = (MASKED && lag + hidden > 3) ? a : with;
            }
            out[e] = (IO)a;
          }
          *reinterpret_cast<Frag*>(lds + (4 * rho + i) * LDSROW + bcv * Tr::HW) = out;
          buf_store_b128(__builtin_bit_cast(i32x4, out), rxo, bcol_ok ? (unsigned)(4 * rho + i) * row_bytes + bcol_bytes : kOutOfRange);
        }
        if (cur.c == p.nCf - 1 && p.conv_new_state && bcol_ok) {
          // the last K - 1 rows of [carried rows ; input] become the next call's carried rows
          const int K1 = p.conv_k - 1;
          const int last = p.T - 1 - t0;                     // tile row of the sequence's last token
          if (rho == last / 4) {
            const rsrc_t rn = make_rsrc((IO*)p.conv_new_state + (long long)cur.b * K1 * W, (unsigned)K1 * row_bytes);
#pragma unroll
            for (int idx = 0; idx < 7; ++idx) {
              const int srow = (4 * rho - 3 + idx) - (last - K1 + 1);
              buf_store_b128(__builtin_bit_cast(i32x4, um[idx]), rn, (srow >= 0 && srow < K1) ? (unsigned)srow * row_bytes + bcol_bytes : kOutOfRange);
            }
          }
        }
      } else {
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const int idx = tid + i * kThreads;
        const int row = idx / VPR, cv = idx - row * VPR;
        if (idx < TR * VPR) {
          *reinterpret_cast<Frag*>(lds + row * LDSROW + cv * Tr::HW) = pre[i];
          if constexpr (GIVEN) {
            *reinterpret_cast<Frag*>(lds_pre + row * LDSROW + cv * Tr::HW) = pre_a[i];
            *reinterpret_cast<Frag*>(lds_pre + (TR + row) * LDSROW + cv * Tr::HW) = pre_x[i];
          }
        }
      }
      }
      __syncthreads();
      if (slab_ok) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          f32x16 ua, ux;
          float xv[16];
          if constexpr (GIVEN) {
            const int col = w.wave * 32 + w.r;
#pragma unroll
            for (int e = 0; e < 16; ++e) {
              const int at = (hf * 16 * MT + 16 * mt + e) * LDSROW + col;
              xv[e] = (float)lds[at];
              ua[e] = (float)lds_pre[at];
              ux[e] = (float)lds_pre[TR * LDSROW + at];
            }
          } else
          gate_mfma_held<IO, MT, NKG, KC>(lds, hw, mt, w.slab, w.r, hf, 0.0f, 0.0f, ua, ux, xv, NKG >= 8 ? 0 : w.kb);
          fwd_gates<IO, MASKED>(flbits[mt], ua, ux, xv, sp, cur.a + 16 * mt, cur.z + 16 * mt, nba, nbx,
                                p.first_reset && mt == 0 && cur.c == 0 && hf == 0);
        }
      }
      fwd_local<MT, MASKED>(p, w, cur, slab_ok);
      if (tid == 0) s_ticket[par ^ 1] = next_raw;
      __syncthreads();
      par ^= 1;
      const long long tk_next = s_ticket[par];
      if constexpr (BLOCK) {
        // the tile's rows of the second projection, in the layout of the store stage
        const int t0 = cur.c * TR;
        const int rows = (p.T - t0) < TR ? (p.T - t0) : TR;
        const unsigned v_row_bytes = (unsigned)p.ld_gate * (unsigned)sizeof(IO);
        const rsrc_t rv = make_rsrc((const IO*)p.gate_v + ((long long)cur.b * p.T + t0) * p.ld_gate, slab_ok ? (unsigned)rows * v_row_bytes : 0u);
#pragma unroll
        for (int i = 0; i < TR / 16; ++i)
          gate_rows[i] = buf_load_frag<bf16x8>(rv, (unsigned)(16 * i + (w.lane >> 2)) * v_row_bytes +
                                                   (unsigned)(w.k * p.bw + w.slab * 32) * 2u + (unsigned)(w.lane & 3) * 16u);
      }
      issue(tk_next);
      fwd_finalize<IO, MT, MASKED, sizeof(IO) == 2, BLOCK>(p, w, cur, stage, &ahead, slab_ok, gate_rows);
      tk = tk_next;
    }
  } else {
    for (;;) {
      if (tid == 0) s_ticket[0] = atomicAdd(q.counter, 1u);
      __syncthreads();
      const long long tk = s_ticket[0];
      if (tk >= q.tiles) break;
      const int c = (int)(tk / q.n_b), b = q.first_b + (int)(tk - (long long)c * q.n_b) * p.queues;
      f32x16 ua[MT], ux[MT];
      float xv[EL];
      gate_tile_generic<IO, MT>(p, x + (long long)b * p.T * W, (long long)c * TR, p.T, w.k, w.slab, w.slab_ok,
                                w_a_row, w_x_row, 0.0f, 0.0f, lds, ua, ux, xv);
      if (w.slab_ok) {
        const long long trow = (long long)b * p.T + c * TR + hf * EL;
        FwdTile<MT> tile;
        tile.b = b; tile.c = c;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          float xpart[16];
#pragma unroll
          for (int e = 0; e < 16; ++e) xpart[e] = xv[16 * mt + e];
          fwd_gates<IO, true>(flag_run(p, trow + 16 * mt, c * TR + hf * EL + 16 * mt), ua[mt], ux[mt], xpart, sp, tile.a + 16 * mt, tile.z + 16 * mt, nba, nbx);
        }
        fwd_local<MT, true>(p, w, tile);
        // 16-bit outputs go through the wave's staging area when whole 64-byte row segments can be
        // written (aligned rows, blocks made of full slabs); else element by element
        if (sizeof(IO) == 2 && p.aligned && p.full_slabs) fwd_finalize<IO, MT, true, true>(p, w, tile, stage);
        else fwd_finalize<IO, MT, true, false>(p, w, tile, stage);
      }
    }
  }
}

// ------------------------------------------------------------------------------------------
// Forward for shapes with many chains (sequences x 32-channel slabs: about one per compute unit or more).
// A workgroup owns ONE chain for the whole sequence, so nothing is exchanged between workgroups: no tickets,
// no records in memory, no look-back, and the composition order is fixed (results repeat bit for bit).  Its
// sixteen waves take the chain's 32-token tiles round robin (wave j: tiles j, j + 16, ...).  Each wave stages
// its own x tiles (32 rows of the block's K range) in a private LDS area, so the loop has no workgroup
// barrier; the slab's rows of both gate matrices sit in LDS once for all waves, which keeps a wave at 128
// registers (four waves a SIMD); the output tile is transposed through the x tile's area once that is
// consumed.  The state goes from tile to tile through LDS: one 8-byte entry {tile number + 1, state} per
// channel, written by the tile's wave and polled by the wave of the next tile, which is resident by
// construction.  The slabs of a gate block run as workgroups of one XCD (block index = XCD + 8 * slot), so
// the x tile they share is fetched from memory once and served to the others by that XCD's L2.
// Measured at B8 T2048 W1024 (256 chains on 256 compute units): 33 us against 39 us for the tiled kernel
// with look-back; the vector unit is busy 77 % of the waves' lifetime (4.8 cycles per instruction: a
// transcendental takes 8.5, 96 of a tile's 429 are).
// ------------------------------------------------------------------------------------------
constexpr int kChainWaves = 16;

// PREP: the launch also does what prepare_kernel does (the parameter image for the backward kernels, the zeroed
// workspace region) and takes its own weights, biases and decay constants straight from the caller's parameters.
template <typename IO, int NKG, bool MASKED, bool PREP = false>
__global__ __launch_bounds__(kChainWaves * 64, 1) void fwd_chain_kernel(FusedArgs p) {
  typedef Io<IO> Tr;
  typedef typename Tr::Frag Frag;
  static_assert(sizeof(IO) == 2 && (NKG == 8 || NKG == 4 || NKG == 2), "16-bit storage, gate blocks of 128, 64 or 32 channels");
  constexpr int TR = 32;
  constexpr int KC = NKG * Tr::KG;                         // block width = K range of the gate products
  constexpr int S = KC / 32;                               // slabs (chains) per block
  constexpr int LDSROW = KC + Tr::HW;
  constexpr int VPR = KC / Tr::HW;                         // 16-byte vectors per tile row
  constexpr int NV = TR * VPR / 64;                        // vectors per lane and tile
  static_assert(TR * LDSROW * (int)sizeof(IO) >= WaveStage<TR>::kBytes, "the staging area lies over the x tile");
  __shared__ __attribute__((aligned(16))) IO lds_all[kChainWaves][TR * LDSROW];
  __shared__ __attribute__((aligned(16))) IO lds_w[2 * 32 * LDSROW];                // [gate][output channel][K]
  __shared__ __attribute__((aligned(8))) unsigned long long carry[kChainWaves][32];

  const int tid = threadIdx.x, lane = tid & 63, r = lane & 31, hf = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // known to be wave-uniform: what derives from it stays scalar
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int sl = slot % S, u = (slot / S) * 8 + xcd;       // slab of the block; (sequence, block) pair
  const bool chain_ok = u < p.B * p.nb;                    // the grid is rounded up to whole rounds of eight pairs
  const int b = chain_ok ? u / p.nb : 0, k = chain_ok ? u - b * p.nb : 0;
  // Hand-off entries {tile number + 1, state}, all "nothing yet" -- except the last wave's, which tile 0 reads: it
  // starts out as {0, h0}, what a tile in front of the sequence would have left.  Tile 0 then takes its state like
  // every other tile (the initial state kept in a register for it was spilled, and the reload on that path put a
  // wait for all memory operations into every hand-off).
  for (int i = tid; i < kChainWaves * 32; i += kChainWaves * 64) {
    unsigned long long entry = 0ull;
    if (i >= (kChainWaves - 1) * 32 && chain_ok && p.h0)
      entry = (unsigned long long)__float_as_uint(p.h0[(long long)b * p.W + k * KC + sl * 32 + (i - (kChainWaves - 1) * 32)]) << 32;
    (&carry[0][0])[i] = entry;
  }
  // The chain kernels use no carry records and no tickets: all this pass needs from the workspace is a failure word
  // that starts out zero.  Workgroup 0 clears it in its first instructions; a workgroup sets it only after it
  // has walked its whole chain, by which time that store has long landed.
  if (blockIdx.x == 0 && tid == 0) __hip_atomic_store(p.fail, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  {
    for (int i = tid; i < 2 * 32 * VPR; i += kChainWaves * 64) {
      const int gate = i / (32 * VPR), o = (i / VPR) % 32, cv = i % VPR;
      const IO* wg = PREP ? (const IO*)(gate ? p.prep.w_x : p.prep.w_a) + ((long long)k * p.bwp + sl * 32 + o) * p.bwp
                          : (const IO*)p.wg + ((long long)(gate * p.nb + k) * p.bwp + sl * 32 + o) * p.bwp;
      *reinterpret_cast<Frag*>(lds_w + (gate * 32 + o) * LDSROW + cv * Tr::HW) = *reinterpret_cast<const Frag*>(wg + cv * Tr::HW);
    }
  }
  __syncthreads();
  if (!chain_ok) return;
  if constexpr (PREP) {
    if (b == 0) {
      // The first sequence's workgroups write the image of their slab: the rows of both matrices as they are,
      // the transposed and gate-interleaved copy w2t[k][j][2 o + gate] (one 32-bit pair per (j, o)), and the
      // per-channel constants.
      IO* wg_out = (IO*)p.prep.wg;
      for (int i = tid; i < 2 * 32 * VPR; i += kChainWaves * 64) {
        const int gate = i / (32 * VPR), o = (i / VPR) % 32, cv = i % VPR;
        *reinterpret_cast<Frag*>(wg_out + ((long long)(gate * p.nb + k) * p.bwp + sl * 32 + o) * p.bwp + cv * Tr::HW) =
            *reinterpret_cast<const Frag*>(lds_w + (gate * 32 + o) * LDSROW + cv * Tr::HW);
      }
      unsigned* w2t = (unsigned*)p.prep.w2t;
      const unsigned short* lw = (const unsigned short*)lds_w;
      for (int i = tid; i < KC * 32; i += kChainWaves * 64) {
        const int j = i >> 5, o = i & 31;
        const unsigned pair = (unsigned)lw[o * LDSROW + j] | ((unsigned)lw[(32 + o) * LDSROW + j] << 16);
        w2t[((long long)k * p.bwp + j) * p.bwp + sl * 32 + o] = pair;
      }
      if (tid < 32) prepare_channel(p.prep, k * p.bwp + sl * 32 + tid);
    }
  }
  const int col0 = k * KC;                                 // first channel of the block
  const int ch = col0 + sl * 32 + r;                       // the lane's channel
  const long long W = p.W;
  IO* lds = lds_all[wave];
  unsigned char* stage = reinterpret_cast<unsigned char*>(lds);
  float nba, nbx, sp;
  if constexpr (PREP) {                                    // the constants prepare_channel derives, for this lane's channel
    nba = -kLog2e * load_vec(p.prep.b_a, ch, p.prep.vec_dtype);
    nbx = -kLog2e * load_vec(p.prep.b_x, ch, p.prep.vec_dtype);
    sp = p.prep.c * log_sigmoid(load_vec(p.prep.lambda, ch, p.prep.vec_dtype)) * kLog2e;
  } else {
    nba = -kLog2e * p.bias[ch]; nbx = -kLog2e * p.bias[p.Wp + ch];
    sp = p.sp[ch];
  }
  const int nC = (p.T + TR - 1) / TR;
  const unsigned row_bytes = (unsigned)p.W * 2u;
  const long long limit = p.limit < 0 ? -p.limit : p.limit;

  Frag pre[NV];
  unsigned pre_off[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int idx = lane + 64 * i, row = idx / VPR, cv = idx - row * VPR;
    pre_off[i] = (unsigned)row * row_bytes + (unsigned)(col0 + cv * Tr::HW) * 2u;
  }
  const IO* xb = (const IO*)p.x + (long long)b * p.T * W;
  auto issue = [&](int c) {                                // a tile past the end: empty extent, nothing is fetched
    const int rows = c >= nC ? 0 : ((p.T - c * TR) < TR ? (p.T - c * TR) : TR);
    const rsrc_t rx = make_rsrc(xb + (long long)(c < nC ? c : 0) * TR * W, (unsigned)rows * row_bytes);
#pragma unroll
    for (int i = 0; i < NV; ++i) pre[i] = buf_load_frag<Frag>(rx, pre_off[i]);
  };
  const rsrc_t rck = make_rsrc(p.ckpt + (long long)b * p.ckpt_nC * W, (unsigned)p.ckpt_nC * (unsigned)W * 4u);
  const rsrc_t rhl = make_rsrc(p.h_last, p.h_last ? (unsigned)p.B * (unsigned)W * 4u : 0u);
  const int prev_wave = (wave + kChainWaves - 1) % kChainWaves;
  bool gave_up = false;
  issue(wave);
  {
    // The loop's back edge has four stores in flight behind the prefetched tile (final state, checkpoint, two
    // output segments).  The same four, dropped through their offsets, in front of its entry: the wait for the
    // tile at the loop's top can then leave the stores in flight on both paths.
    BufIo<float>::store(0.f, rhl, kOutOfRange, 0u);
    BufIo<float>::store(0.f, rck, kOutOfRange, 0u);
    const i32x4 nothing = {0, 0, 0, 0};
    buf_store_b128(nothing, rck, kOutOfRange);
    buf_store_b128(nothing, rhl, kOutOfRange);
  }
  for (int c = wave; c < nC; c += kChainWaves) {
    const int t0 = c * TR;
    unsigned flbits = 0u;
    if constexpr (MASKED) flbits = flag_run(p, (long long)b * p.T + t0 + hf * 16, t0 + hf * 16);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int idx = lane + 64 * i, row = idx / VPR, cv = idx - row * VPR;
      *reinterpret_cast<Frag*>(lds + row * LDSROW + cv * Tr::HW) = pre[i];
    }
    wave_lds_fence();
    issue(c + kChainWaves);
    f32x16 ua, ux;
    float xv[16], a[16], z[16];
#pragma unroll
    for (int v = 0; v < 16; ++v) { ua[v] = 0.0f; ux[v] = 0.0f; }     // the biases enter inside the sigmoids
    {
      const IO* xrow = lds + tile_row<1>(0, r) * LDSROW + hf * Tr::HW;
      const IO* wrow = lds_w + r * LDSROW + hf * Tr::HW;
#pragma unroll
      for (int kg = 0; kg < NKG; ++kg) {
        const Frag xa = *reinterpret_cast<const Frag*>(xrow + kg * Tr::KG);
        Tr::mma(ua, xa, *reinterpret_cast<const Frag*>(wrow + kg * Tr::KG));
        Tr::mma(ux, xa, *reinterpret_cast<const Frag*>(wrow + 32 * LDSROW + kg * Tr::KG));
      }
#pragma unroll
      for (int e = 0; e < 16; ++e) xv[e] = (float)lds[(hf * 16 + e) * LDSROW + sl * 32 + r];
    }
    fwd_gates<IO, MASKED>(flbits, ua, ux, xv, sp, a, z, nba, nbx, p.first_reset && c == 0 && hf == 0);
    // affine map of the lane's 16 tokens, then of the lower half and of the whole tile
    float A = 1.f, H = 0.f;
#pragma unroll
    for (int e = 0; e < 16; ++e) { H = fmaf(a[e], H, z[e]); A *= a[e]; }
    const float A_o = xhalf(A, hf), H_o = xhalf(H, hf);
    const float A_lo = hf ? A_o : A, H_lo = hf ? H_o : H;
    const float A_hi = hf ? A : A_o, H_hi = hf ? H : H_o;
    const float A_t = A_hi * A_lo, H_t = fmaf(A_hi, H_lo, H_hi);
    // the state in front of the tile: what the wave of the tile before has left in LDS (h0 for tile 0).  A wait
    // that runs out of polls hands on NaN, so the failure shows in the results; every wave still reaches the end.
    float h_in;
    {
      long long polls = 0;
      bool ok;
      for (;;) {
        const unsigned long long e = __hip_atomic_load(&carry[prev_wave][r], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        ok = (unsigned)e == (unsigned)c;
        h_in = __uint_as_float((unsigned)(e >> 32));
        if (__all(ok) || ++polls > limit) break;
        __builtin_amdgcn_s_sleep(1);
      }
      gave_up |= !__all(ok);
      if (!ok) h_in = __builtin_nanf("");
    }
    const float h_end = fmaf(A_t, h_in, H_t);
    const float h_mid = fmaf(A_lo, h_in, H_lo);
    if (hf == 0) __hip_atomic_store(&carry[wave][r], ((unsigned long long)__float_as_uint(h_end) << 32) | (unsigned long long)(unsigned)(c + 1),
                                    __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    BufIo<float>::store(h_end, rhl, (hf == 0 && c == nC - 1) ? ((unsigned)b * (unsigned)W + (unsigned)ch) * 4u : kOutOfRange, 0u);

    float h = hf ? h_mid : h_in;
    const int rows = (p.T - t0) < TR ? (p.T - t0) : TR;
    const rsrc_t ry = make_rsrc((IO*)p.y + ((long long)b * p.T + t0) * W, (unsigned)rows * row_bytes);
    wave_lds_fence();                                      // the x tile has been read: its area becomes the staging area
    unsigned char* my = stage + WaveStage<TR>::row_offset(hf * 16) + r * 2;
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      h = fmaf(a[e], h, z[e]);
      *reinterpret_cast<IO*>(my + e * WaveStage<TR>::kRowBytes) = (IO)h;
    }
    // checkpoint for the backward pass: the state after the lane's 16 tokens (slot = token / 16)
    BufIo<float>::store(h, rck, ((unsigned)(2 * c + hf) * (unsigned)W + (unsigned)ch) * 4u, 0u);
    wave_lds_fence();
    stage_flush<TR>(stage, ry, row_bytes, (unsigned)(col0 + sl * 32) * 2u, lane);
    wave_lds_fence();
  }
  if (gave_up && lane == 0) atomicOr(p.fail, 1u);
}

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

// ------------------------------------------------------------------------------------------
// Host side
// ------------------------------------------------------------------------------------------
static int check_geometry(const char* who, int64_t W, int64_t nb, int dtype) {
  if (dtype != RGLRU_F32 && dtype != RGLRU_BF16) return fail(RGLRU_E_ARG, "%s: dtype must be RGLRU_F32 or RGLRU_BF16, got %d", who, dtype);
  if (W <= 0 || nb <= 0 || W % nb != 0) return fail(RGLRU_E_ARG, "%s: width %lld is not divisible into %lld gate blocks", who, (long long)W, (long long)nb);
  if (W / nb > 512) return fail(RGLRU_E_UNSUPPORTED, "%s: gate block width %lld exceeds the supported maximum of 512", who, (long long)(W / nb));
  if (W >= (1 << 24)) return fail(RGLRU_E_UNSUPPORTED, "%s: width too large", who);
  return RGLRU_OK;
}

// Sizes the kernels address with 32-bit offsets.  Tiles and per-sequence slices of the workspace are
// reached through buffer descriptors whose lane offsets are 32-bit and whose "dropped access" offset
// is 0x7ffffff0, so every such extent has to stay below 2^31 bytes: the checkpoints of one sequence
// (the fp32 state after every 16 tokens, 4 W bytes each; the carry records of a sequence are no larger)
// and the [B, W] fp32 state tensors.
static int check_extents(const char* who, int64_t B, int64_t T, int64_t W) {
  if (B * T * W >= (1ll << 40) || B * T >= (1ll << 31)) return fail(RGLRU_E_UNSUPPORTED, "%s: tensor too large", who);
  const int64_t slots = 4 * ((T + 63) / 64);              // checkpoint slots per sequence
  if (slots * W * 4 >= (1ll << 31))
    return fail(RGLRU_E_UNSUPPORTED, "%s: one sequence of %lld tokens x %lld channels exceeds the 2 GiB per-sequence workspace limit; split the sequence and carry the state", who, (long long)T, (long long)W);
  if (B * W * 4 >= (1ll << 31)) return fail(RGLRU_E_UNSUPPORTED, "%s: state tensor [%lld, %lld] too large", who, (long long)B, (long long)W);
  return RGLRU_OK;
}

static size_t elem_size(int dtype) { return dtype == RGLRU_BF16 ? 2 : 4; }

static void fill_common(FusedArgs& a, const Geometry& g, const void* prep, int dtype) {
  PrepLayout pl = make_prep_layout(g, elem_size(dtype));
  const char* pb = (const char*)prep;
  a.wg = pb + pl.wg; a.bias = (const float*)(pb + pl.bias); a.sp = (const float*)(pb + pl.sp); a.cs = (const float*)(pb + pl.cs);
  a.w2t = pb + pl.w2t;
  a.W = (int)g.W; a.nb = (int)g.nb; a.bw = (int)g.bw; a.bwp = (int)g.bwp; a.S = (int)g.S; a.Wp = (int)g.Wp;
  a.groups = (int)g.groups; a.units = (int)g.units; a.bpu = 1;
  a.limit = spin_limit();
  a.full_slabs = (g.bw % 32 == 0) ? 1 : 0;
}

static const float* finish_dsp(const Geometry& g, const void* prep, int dtype) {
  return (const float*)((const char*)prep + make_prep_layout(g, elem_size(dtype)).dsp);
}

static int is_aligned(const void* ptr, int64_t W, int64_t bw, size_t es) {
  return ((uintptr_t)ptr % 16 == 0) && ((W * (int64_t)es) % 16 == 0) && ((bw * (int64_t)es) % 16 == 0);
}

// number of register-held K groups for this block width, or 0 for the streaming variant
static int held_groups(const Geometry& g, int dtype, int aligned) {
  if (dtype == RGLRU_BF16 && aligned && g.bw == g.bwp) {
    if (g.bwp == 128) return 8;
    if (g.bwp == 64) return 4;
    if (g.bwp == 32) return 2;
  }
  return 0;
}

// K steps of 32 channels of the decode kernels on 16 x 16 tiles (gate blocks of 32 .. 384 channels in steps
// of 32, 16-bit storage, aligned rows), or 0 for the portable decode kernels
static int step16_groups(const Geometry& g, int dtype, int aligned) {
  if (dtype != RGLRU_BF16 || !aligned || g.bw != g.bwp || g.bw > 384) return 0;
  return (int)(g.bw / 32);
}

// ... and for the blocks wider than a workgroup's four slabs whose weights the forward and the
// gate-gradient kernels hold in registers: K groups (bw / 16), or 0
static int wide_groups(const Geometry& g, int dtype, int aligned) {
  if (dtype != RGLRU_BF16 || !aligned) return 0;
  switch (g.bw) {
    case 160: case 192: case 224: case 256: case 288: case 320: case 352: case 384: return (int)(g.bw / 16);
    default: return 0;
  }
}

#define RGLRU_FWD_WIDE_CASE(N, grid, stream, args, dtype, nkg, masked)                                              \
    else if ((dtype) == RGLRU_BF16 && (nkg) == N && !(masked)) hipLaunchKernelGGL((fwd_kernel<__bf16, N, false>), grid, dim3(kThreads), 0, stream, args); \
    else if ((dtype) == RGLRU_BF16 && (nkg) == N) hipLaunchKernelGGL((fwd_kernel<__bf16, N, true>), grid, dim3(kThreads), 0, stream, args);
#define RGLRU_DISPATCH_FWD(grid, stream, args, dtype, nkg, masked)                                      \
  do {                                                                                                 \
    if ((dtype) == RGLRU_BF16 && (nkg) == 8 && !(masked)) hipLaunchKernelGGL((fwd_kernel<__bf16, 8, false>), grid, dim3(kThreads), 0, stream, args); \
    else if ((dtype) == RGLRU_BF16 && (nkg) == 8) hipLaunchKernelGGL((fwd_kernel<__bf16, 8, true>), grid, dim3(kThreads), 0, stream, args); \
    else if ((dtype) == RGLRU_BF16 && (nkg) == 4 && !(masked)) hipLaunchKernelGGL((fwd_kernel<__bf16, 4, false>), grid, dim3(kThreads), 0, stream, args); \
    else if ((dtype) == RGLRU_BF16 && (nkg) == 4) hipLaunchKernelGGL((fwd_kernel<__bf16, 4, true>), grid, dim3(kThreads), 0, stream, args); \
    else if ((dtype) == RGLRU_BF16 && (nkg) == 2 && !(masked)) hipLaunchKernelGGL((fwd_kernel<__bf16, 2, false>), grid, dim3(kThreads), 0, stream, args); \
    else if ((dtype) == RGLRU_BF16 && (nkg) == 2) hipLaunchKernelGGL((fwd_kernel<__bf16, 2, true>), grid, dim3(kThreads), 0, stream, args); \
    RGLRU_FWD_WIDE_CASE(10, grid, stream, args, dtype, nkg, masked) RGLRU_FWD_WIDE_CASE(12, grid, stream, args, dtype, nkg, masked) \
    RGLRU_FWD_WIDE_CASE(14, grid, stream, args, dtype, nkg, masked) RGLRU_FWD_WIDE_CASE(16, grid, stream, args, dtype, nkg, masked) \
    RGLRU_FWD_WIDE_CASE(18, grid, stream, args, dtype, nkg, masked) RGLRU_FWD_WIDE_CASE(20, grid, stream, args, dtype, nkg, masked) \
    RGLRU_FWD_WIDE_CASE(22, grid, stream, args, dtype, nkg, masked) RGLRU_FWD_WIDE_CASE(24, grid, stream, args, dtype, nkg, masked) \
    else if ((dtype) == RGLRU_BF16 && (nkg) < 0 && !(masked)) hipLaunchKernelGGL((fwd_kernel<__bf16, -1, false>), grid, dim3(kThreads), 0, stream, args); \
    else if ((dtype) == RGLRU_BF16 && (nkg) < 0) hipLaunchKernelGGL((fwd_kernel<__bf16, -1, true>), grid, dim3(kThreads), 0, stream, args); \
    else if ((dtype) == RGLRU_BF16) hipLaunchKernelGGL((fwd_kernel<__bf16, 0, true>), grid, dim3(kThreads), 0, stream, args); \
    else hipLaunchKernelGGL((fwd_kernel<float, 0, true>), grid, dim3(kThreads), 0, stream, args);      \
  } while (0)

#define RGLRU_DISPATCH(KERNEL, grid, stream, args, dtype, nkg)                                         \
  do {                                                                                                 \
    if ((dtype) == RGLRU_BF16) {                                                                       \
      if ((nkg) == 8) hipLaunchKernelGGL((KERNEL<__bf16, 8>), grid, dim3(kThreads), 0, stream, args);  \
      else if ((nkg) == 4) hipLaunchKernelGGL((KERNEL<__bf16, 4>), grid, dim3(kThreads), 0, stream, args); \
      else if ((nkg) == 2) hipLaunchKernelGGL((KERNEL<__bf16, 2>), grid, dim3(kThreads), 0, stream, args); \
      else hipLaunchKernelGGL((KERNEL<__bf16, 0>), grid, dim3(kThreads), 0, stream, args);             \
    } else {                                                                                           \
      hipLaunchKernelGGL((KERNEL<float, 0>), grid, dim3(kThreads), 0, stream, args);                   \
    }                                                                                                  \
  } while (0)

static int launch_clear(char* base, size_t begin, size_t end, hipStream_t s) {
  long long words = (long long)(end - begin) / 4;
  int cb = (int)((words + 1023) / 1024); if (cb > 2048) cb = 2048; if (cb < 1) cb = 1;
  hipLaunchKernelGGL(clear_words_kernel, dim3(cb), dim3(256), 0, s, (unsigned*)(base + begin), words);
  return check_launch("workspace clear");
}

// Optional event bracket around the main kernel of an entry point (measurement hook).
static std::atomic<int> g_timing{0};
struct TimingSlot { hipEvent_t start = nullptr, stop = nullptr; bool armed = false; };
static TimingSlot& timing_slot(int which) {
  static TimingSlot slots[4];       // process-wide: backward runs on PyTorch's autograd thread
  return slots[which];
}
struct KernelTimer {
  TimingSlot* slot = nullptr; hipStream_t stream;
  KernelTimer(int which, hipStream_t s) : stream(s) {
    if (!g_timing.load(std::memory_order_relaxed)) return;
    slot = &timing_slot(which);
    if (!slot->start && (hipEventCreate(&slot->start) != hipSuccess || hipEventCreate(&slot->stop) != hipSuccess)) { slot = nullptr; return; }
    (void)hipEventRecord(slot->start, stream);
  }
  ~KernelTimer() { if (slot) { (void)hipEventRecord(slot->stop, stream); slot->armed = true; } }
};

// Narrow blocks of the kernels with register-held weights share a unit (see kPackedWidth).
static void pack_units(FusedArgs& a, const Geometry& g, int nkg) {
  if (nkg == 4 || nkg == 2) {
    a.bpu = kPackedWidth / (int)g.bw;
    a.units = (int)((g.nb + a.bpu - 1) / a.bpu);
  }
}

static int pick_wg_per_unit(int units, long long tiles_per_unit, int per_cu, long long cap) {
  long long target = (long long)num_compute_units() * per_cu;
  long long n = (target + units - 1) / units;
  if (n > tiles_per_unit) n = tiles_per_unit;
  if (n > cap) n = cap;
  if (n < 1) n = 1;
  return (int)n;
}

// How many ticket queues a unit's workgroups share.  Queue j owns the sequences j, j + q, ... and is served by
// the workgroups j, j + q, ...; the launch ends with the queue that has the most sequences per workgroup, so
// take the q that makes that ratio smallest (9 sequences on 16 workgroups: one queue, not nine of which seven
// have two workgroups and two have one).  Among equals the largest q, which spreads the ticket atomics.
static int pick_queues(long long B, int wg) {
  long long qmax = B < wg ? B : wg;
  if (qmax > kMaxQueues) qmax = kMaxQueues;
  int best = 1;
  long long best_num = B, best_den = wg;                  // one queue: B sequences on wg workgroups
  for (int q = 2; q <= qmax; ++q) {
    long long num = 0, den = 1;
    for (int j = 0; j < q; ++j) {
      const long long n = (B - j + q - 1) / q, w = (wg - j + q - 1) / q;
      if (n * den > num * w) { num = n; den = w; }
    }
    if (num * best_den <= best_num * den) { best = q; best_num = num; best_den = den; }
  }
  return best;
}

}  // namespace rglru

using namespace rglru;

extern "C" {


int rglru_hip_max_block_width(void) { return 512; }

size_t rglru_hip_prep_bytes(int64_t W, int64_t nb, int dtype) {
  if (check_geometry("prep_bytes", W, nb, dtype)) return 0;
  return make_prep_layout(make_geometry(W, nb), elem_size(dtype)).total;
}

// The arguments of a parameter conversion (validated), and its launch.
static int build_prep_args(const void* w_a, const void* b_a, const void* w_x, const void* b_x,
                           const void* lambda, float c, int64_t W, int64_t nb, int dtype, int vec_dtype,
                           void* prep, void* clear, size_t clear_bytes, PrepArgs& a) {
  int rc = check_geometry("prepare", W, nb, dtype);
  if (rc) return rc;
  if (vec_dtype != RGLRU_F32 && vec_dtype != RGLRU_BF16) return fail(RGLRU_E_ARG, "prepare: unknown vector dtype %d", vec_dtype);
  if (!w_a || !b_a || !w_x || !b_x || !lambda || !prep) return fail(RGLRU_E_ARG, "prepare: null pointer");
  Geometry g = make_geometry(W, nb);
  PrepLayout pl = make_prep_layout(g, elem_size(dtype));
  char* pb = (char*)prep;
  a.w_a = w_a; a.w_x = w_x; a.b_a = b_a; a.b_x = b_x; a.lambda = lambda;
  a.wg = pb + pl.wg; a.bias = (float*)(pb + pl.bias); a.sp = (float*)(pb + pl.sp); a.cs = (float*)(pb + pl.cs);
  a.dsp = (float*)(pb + pl.dsp); a.vec_dtype = vec_dtype;
  a.w2t = pb + pl.w2t;
  a.W = (int)W; a.nb = (int)nb; a.bw = (int)g.bw; a.bwp = (int)g.bwp; a.Wp = (int)g.Wp; a.c = c;
  a.clear = (uint4*)clear; a.clear_n = (long long)(clear_bytes / 16);
  a.vec_ok = dtype == RGLRU_BF16 && g.bw == g.bwp && g.bw % 8 == 0 && (uintptr_t)w_a % 16 == 0 && (uintptr_t)w_x % 16 == 0 &&
             (uintptr_t)a.wg % 16 == 0 && (uintptr_t)a.w2t % 16 == 0;
  return RGLRU_OK;
}

static int launch_prepare(const PrepArgs& a, int dtype, void* stream) {
  const long long cells = (long long)a.nb * a.bwp * a.bwp;
  long long total = a.vec_ok ? 4 * cells / 8 + a.Wp : 4 * cells + a.Wp;
  if (a.clear_n > total) total = a.clear_n;
  int blocks = (int)((total + 255) / 256); if (blocks > 2048) blocks = 2048;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == RGLRU_BF16) hipLaunchKernelGGL(prepare_kernel<__bf16>, dim3(blocks), dim3(256), 0, s, a);
  else hipLaunchKernelGGL(prepare_kernel<float>, dim3(blocks), dim3(256), 0, s, a);
  return check_launch("prepare");
}

static int prepare_impl(const void* w_a, const void* b_a, const void* w_x, const void* b_x,
                        const void* lambda, float c, int64_t W, int64_t nb, int dtype, int vec_dtype,
                        void* prep, void* clear, size_t clear_bytes, void* stream) {
  PrepArgs a;
  const int rc = build_prep_args(w_a, b_a, w_x, b_x, lambda, c, W, nb, dtype, vec_dtype, prep, clear, clear_bytes, a);
  if (rc) return rc;
  return launch_prepare(a, dtype, stream);
}

int rglru_hip_prepare(const void* w_a, const void* b_a, const void* w_x, const void* b_x,
                      const void* lambda, float c, int64_t W, int64_t nb, int dtype, int vec_dtype,
                      void* prep, void* stream) {
  return prepare_impl(w_a, b_a, w_x, b_x, lambda, c, W, nb, dtype, vec_dtype, prep, nullptr, 0, stream);
}

size_t rglru_hip_workspace_bytes(int64_t B, int64_t T, int64_t W, int64_t nb) {
  if (B <= 0 || T <= 0 || W <= 0 || nb <= 0 || W % nb) return 0;
  return make_work_layout(B, T, make_geometry(W, nb)).total;
}

int rglru_hip_wide_path(int64_t W, int64_t nb, int dtype);

int rglru_hip_block_fwd_path(int64_t W, int64_t nb, int64_t K, int dtype) {
  if (dtype != RGLRU_BF16 || W <= 0 || nb <= 0 || W % nb || K < 1 || K > 4) return 0;
  const int64_t bw = W / nb;
  return (bw == 32 || bw == 64 || bw == 128) ? 1 : 0;
}

size_t rglru_hip_bwd_scratch_bytes(int64_t B, int64_t T, int64_t W, int64_t nb, int dtype) {
  if (B <= 0 || T <= 0 || W <= 0 || nb <= 0 || W % nb) return 0;
  const int kind = rglru_hip_fast_path(W, nb, dtype) ? kScratchFast : rglru_hip_wide_path(W, nb, dtype) ? kScratchWide : kScratchPlain;
  return make_scratch_layout(B, T, make_geometry(W, nb), kind).total;
}

// What the block forward adds to the scan's arguments (x is then the block's first projection).
struct BlockFwd {
  const void* v; int64_t x_stride, v_stride;
  const void* conv_state; const void* taps; const void* conv_bias; int64_t K; int vec_dtype;
  void* x_conv; void* gated; void* new_conv_state;
};

// Whether the forward runs one workgroup per chain (fwd_chain_kernel) instead of tiles with look-back:
// 0 = by shape, 1 = never, 2 = whenever that kernel covers the shape (tests).
static std::atomic<int> g_chain_forward{0};
static bool fwd_chain_pays(int64_t B, int64_t T, int64_t W) {
  const int mode = g_chain_forward.load(std::memory_order_relaxed);
  if (mode == 1) return false;
  if (mode == 2) return true;
  // Two time models, in microseconds for the forward and the reverse scan together, fitted to both kernel
  // pairs timed on 358 shapes (widths 512 to 4096, blocks of 32 to 128 channels, 16 to 8192 chains, 128 to 8192
  // tokens); the faster model wins.  A chain workgroup fills a compute unit, so the chains run in
  // ceil(chains / units) rounds, each as long as its sequence (a start-up cost, then a time per token that
  // grows with the share of the units that are busy, since they share the memory system); the tiled kernels
  // spread any shape over the whole chip, pay two longer launches plus one for the parameters, and their time
  // per token is 1.1 to 1.2 times the chain kernels' when those fill their rounds.
  static const int units = [] {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) n = 0;
    return n;
  }();
  if (units <= 0) return false;
  const double chains = (double)B * (double)(W / 32), tokens = (double)T;
  const double rounds = std::ceil(chains / units), last = (chains - (rounds - 1) * units) / units;
  const double full_round = 4.7 + tokens * (0.01465 + 0.01208), last_round = 4.7 + tokens * (0.01465 + 0.01208 * last);
  const double t_chain = 6.6 + (rounds - 1) * full_round + last_round;
  const double work = chains * tokens * (256.0 / units);
  const double t_tiled = std::max(31.4, 24.2 + 1.025e-4 * work + 0.0030 * tokens);
  return t_chain < t_tiled;
}

static int fwd_impl(const void* x, const void* prep, const float* h0, const uint8_t* flags,
                    void* y, float* h_last, void* ws,
                    int64_t B, int64_t T, int64_t W, int64_t nb, int dtype, bool cleared, void* stream,
                    const void* pre = nullptr, const BlockFwd* blk = nullptr, const PrepArgs* fuse = nullptr) {
  int rc = check_geometry("fwd", W, nb, dtype);
  if (rc) return rc;
  if (B <= 0 || T <= 0) return fail(RGLRU_E_ARG, "fwd: B and T must be positive (got %lld, %lld)", (long long)B, (long long)T);
  if (!x || !prep || (!y && !blk) || !ws) return fail(RGLRU_E_ARG, "fwd: null pointer");
  rc = check_extents("fwd", B, T, W);
  if (rc) return rc;
  Geometry g = make_geometry(W, nb);
  WorkLayout L = make_work_layout(B, T, g);
  hipStream_t s = (hipStream_t)stream;
  char* wb = (char*)ws;
  FusedArgs a;
  memset(&a, 0, sizeof(a));
  fill_common(a, g, prep, dtype);
  const bool first_reset = flags == RGLRU_FLAGS_FIRST_RESET;    // no flag array: token 0 of every row starts a document
  if (first_reset) flags = nullptr;
  a.first_reset = first_reset;
  a.x = x; a.h0 = h0; a.flags = flags; a.y = y; a.h_last = h_last;
  a.flags_vec = (T % 16 == 0) && ((uintptr_t)flags % 16 == 0);
  a.ckpt = (float*)(wb + L.ckpt); a.rec_a = (rec_t*)(wb + L.f_rec_a);
  a.ticket = (unsigned*)(wb + L.f_ticket); a.fail = (unsigned*)(wb + L.fail);
  a.B = (int)B; a.T = (int)T; a.nC = (int)L.nC; a.ckpt_nC = 2 * (int)L.nC;
  a.aligned = is_aligned(x, W, g.bw, elem_size(dtype)) && ((uintptr_t)y % 16 == 0);
  int nkg = held_groups(g, dtype, a.aligned);
  if (!nkg && !pre) nkg = wide_groups(g, dtype, a.aligned);
  if (pre) {
    if (!rglru_hip_pre_path(W, nb, dtype)) return fail(RGLRU_E_UNSUPPORTED, "fwd_pre: needs bf16 storage and gate blocks of a multiple of 32 channels");
    if (!a.aligned || (uintptr_t)pre % 16) return fail(RGLRU_E_UNSUPPORTED, "fwd_pre: x, pre and y must be 16-byte aligned");
    a.pre = pre; a.rows_total = B * T;
    nkg = -1;
    rc = launch_gate_pre_gemm(x, a.wg, const_cast<void*>(pre), B * T, g, s);
    if (rc) return rc;
  }
  if (blk) {
    const int64_t xs = blk->x_stride ? blk->x_stride : W, vs = blk->v_stride ? blk->v_stride : W;
    if (!rglru_hip_block_fwd_path(W, nb, blk->K, dtype))
      return fail(RGLRU_E_UNSUPPORTED, "block_fwd: needs bf16 storage, gate blocks of 32, 64 or 128 channels and 1 to 4 taps");
    if (blk->vec_dtype != RGLRU_F32 && blk->vec_dtype != RGLRU_BF16) return fail(RGLRU_E_ARG, "block_fwd: unknown vector dtype %d", blk->vec_dtype);
    if (!blk->v || !blk->taps || !blk->gated) return fail(RGLRU_E_ARG, "block_fwd: null pointer");
    if (xs < W || vs < W) return fail(RGLRU_E_ARG, "block_fwd: a row stride is smaller than the width %lld", (long long)W);
    const void* ptrs[] = {x, blk->v, blk->conv_state, blk->x_conv, blk->gated, blk->new_conv_state, y};
    for (const void* q : ptrs) if ((uintptr_t)q % 16) return fail(RGLRU_E_UNSUPPORTED, "block_fwd: tensors must be 16-byte aligned");
    if ((W * 2) % 16 || (xs * 2) % 16 || (vs * 2) % 16) return fail(RGLRU_E_UNSUPPORTED, "block_fwd: rows must be a multiple of 16 bytes");
    if (!nkg) return fail(RGLRU_E_UNSUPPORTED, "block_fwd: no kernel for this shape");
    a.gate_v = blk->v; a.ld_gate = vs; a.ld_x = xs;
    // rows that start a document have no history
    a.conv_state = (blk->K > 1 && !first_reset) ? blk->conv_state : nullptr; a.conv_taps = blk->taps; a.conv_bias = blk->conv_bias;
    a.conv_k = (int)blk->K; a.conv_vec_dtype = blk->vec_dtype;
    a.x_out = blk->x_conv; a.gated = blk->gated; a.conv_new_state = blk->K > 1 ? blk->new_conv_state : nullptr;
  }
  // The tiled kernels need the forward records, tickets and failure word zeroed; the chain kernel needs the
  // failure word only and clears it itself.  (Every backward entry point that uses records clears its own.)
  const bool chain = !blk && !pre && (nkg == 8 || nkg == 4 || nkg == 2) && fwd_chain_pays(B, T, W);
  if (!cleared && !chain) {
    rc = launch_clear(wb, L.f_begin, L.f_end, s);
    if (rc) return rc;
  }
  // fuse: the parameter conversion (and, for the tiled kernels, the clearing of the workspace region it names)
  // still has to happen.  The chain kernel converts by itself when the caller's weights can be read as 16-byte
  // vectors; else one launch first.
  const bool fused_prepare = fuse && chain && fuse->vec_ok;
  if (fuse && !fused_prepare) {
    PrepArgs pa = *fuse;
    if (chain) { pa.clear = nullptr; pa.clear_n = 0; }
    rc = launch_prepare(pa, dtype, stream);
    if (rc) return rc;
  }
  if (chain) {
    const int S = (int)(g.bw / 32);
    const dim3 grid((unsigned)(8 * ((B * nb + 7) / 8) * S));
    const int masked = (flags != nullptr) || (T % 32 != 0);
    if (fused_prepare) a.prep = *fuse;
    KernelTimer timer(0, s);
#define RGLRU_CHAIN_LAUNCH(N, M, P) hipLaunchKernelGGL((fwd_chain_kernel<__bf16, N, M, P>), grid, dim3(kChainWaves * 64), 0, s, a)
#define RGLRU_CHAIN_CASE(N)                                                                                            \
    if (nkg == N) {                                                                                                    \
      if (fused_prepare) { if (masked) RGLRU_CHAIN_LAUNCH(N, true, true); else RGLRU_CHAIN_LAUNCH(N, false, true); }   \
      else { if (masked) RGLRU_CHAIN_LAUNCH(N, true, false); else RGLRU_CHAIN_LAUNCH(N, false, false); }               \
    }
    RGLRU_CHAIN_CASE(8) RGLRU_CHAIN_CASE(4) RGLRU_CHAIN_CASE(2)
#undef RGLRU_CHAIN_CASE
#undef RGLRU_CHAIN_LAUNCH
    return check_launch("fwd");
  }
  pack_units(a, g, nkg);
  const int tile_tokens = 32 * fwd_mt(nkg);
  a.nCf = (int)((T + tile_tokens - 1) / tile_tokens);
  // without weights in registers three workgroups fit a compute unit
  a.wg_per_unit = pick_wg_per_unit(a.units, B * (long long)a.nCf, blk ? 2 : nkg < 0 ? RGLRU_GIVEN_OCC : ((nkg == 4 || nkg == 2) ? RGLRU_NARROW_OCC : nkg > 8 ? fwd_wide_occ(nkg) : 2), 1 << 20);
  a.queues = pick_queues(B, a.wg_per_unit);
  dim3 grid((unsigned)(a.wg_per_unit * a.units));
  if (nkg > 8) {
    a.xcd_map = 1;
    grid = dim3((unsigned)(8 * (((long long)nb * a.wg_per_unit + 7) / 8) * a.groups));
  }
  {
    KernelTimer timer(0, s);
    // the plain kernels with register-held weights of up to 128 channels know first_reset; the others take it
    // through the flag logic of their masked variant
    const int masked = (flags != nullptr) || (T % tile_tokens != 0) || (first_reset && !(nkg == 8 || nkg == 4 || nkg == 2));
    if (blk) {
#define RGLRU_BLOCK_CASE(N)                                                                                            \
      if (nkg == N) {                                                                                                  \
        if (masked) hipLaunchKernelGGL((fwd_kernel<__bf16, N, true, true>), grid, dim3(kThreads), 0, s, a);            \
        else hipLaunchKernelGGL((fwd_kernel<__bf16, N, false, true>), grid, dim3(kThreads), 0, s, a);                  \
      }
      RGLRU_BLOCK_CASE(8) RGLRU_BLOCK_CASE(4) RGLRU_BLOCK_CASE(2)
#undef RGLRU_BLOCK_CASE
    } else {
      RGLRU_DISPATCH_FWD(grid, s, a, dtype, nkg, masked);
    }
  }
  return check_launch("fwd");
}

int rglru_hip_fwd(const void* x, const void* prep, const float* h0, const uint8_t* flags,
                  void* y, float* h_last, void* ws,
                  int64_t B, int64_t T, int64_t W, int64_t nb, int dtype, void* stream) {
  return fwd_impl(x, prep, h0, flags, y, h_last, ws, B, T, W, nb, dtype, false, stream);
}

// Forward pass for callers that cannot allocate: the workspace is a file-scope device array of this
// library.  Every device holds its own copy of the array at its own address; the name `static_scratch`
// is only a handle in host code, the address comes from hipGetSymbolAddress, once per device.
static __device__ __align__(256) unsigned char static_scratch[RGLRU_STATIC_WORKSPACE_BYTES];

static void* static_scratch_address() {
  static std::atomic<void*> cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) { fail(RGLRU_E_LAUNCH, "fwd_static: no current device"); return nullptr; }
  void* ptr = cached[dev].load(std::memory_order_acquire);
  if (ptr) return ptr;
  const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(static_scratch));
  if (e != hipSuccess || !ptr) { fail(RGLRU_E_LAUNCH, "fwd_static: hipGetSymbolAddress: %s", hipGetErrorString(e)); return nullptr; }
  cached[dev].store(ptr, std::memory_order_release);     // racing first calls store the same address
  return ptr;
}

size_t rglru_hip_static_workspace_bytes(void) { return (size_t)RGLRU_STATIC_WORKSPACE_BYTES; }

int rglru_hip_fwd_static(const void* x, const void* prep, const float* h0, const uint8_t* flags,
                         void* y, float* h_last,
                         int64_t B, int64_t T, int64_t W, int64_t nb, int dtype, void* stream) {
  int rc = check_geometry("fwd_static", W, nb, dtype);
  if (rc) return rc;
  if (B <= 0 || T <= 0) return fail(RGLRU_E_ARG, "fwd_static: B and T must be positive (got %lld, %lld)", (long long)B, (long long)T);
  const size_t need = make_work_layout(B, T, make_geometry(W, nb)).total;
  if (need > (size_t)RGLRU_STATIC_WORKSPACE_BYTES)
    return fail(RGLRU_E_UNSUPPORTED, "fwd_static: B=%lld T=%lld W=%lld needs a workspace of %zu bytes, the built-in one holds %zu; use rglru_hip_fwd with a caller-provided workspace",
                (long long)B, (long long)T, (long long)W, need, (size_t)RGLRU_STATIC_WORKSPACE_BYTES);
  void* ws = static_scratch_address();
  if (!ws) return RGLRU_E_LAUNCH;
  return fwd_impl(x, prep, h0, flags, y, h_last, ws, B, T, W, nb, dtype, false, stream);
}

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

int rglru_hip_pre_path(int64_t W, int64_t nb, int dtype) {
  if (dtype != RGLRU_BF16 || W <= 0 || nb <= 0 || W % nb) return 0;
  const int64_t bw = W / nb;
  return (bw % 32 == 0 && bw <= 512) ? 1 : 0;
}

int rglru_hip_fwd_pre(const void* x, void* pre, const void* prep, const float* h0, const uint8_t* flags,
                      void* y, float* h_last, void* ws,
                      int64_t B, int64_t T, int64_t W, int64_t nb, int dtype, void* stream) {
  if (!pre) return fail(RGLRU_E_ARG, "fwd_pre: null pointer");
  return fwd_impl(x, prep, h0, flags, y, h_last, ws, B, T, W, nb, dtype, false, stream, pre);
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

int rglru_hip_prepare_fwd(const void* w_a, const void* b_a, const void* w_x, const void* b_x,
                          const void* lambda, float c, int vec_dtype, void* prep,
                          const void* x, const float* h0, const uint8_t* flags,
                          void* y, float* h_last, void* ws,
                          int64_t B, int64_t T, int64_t W, int64_t nb, int dtype, void* stream) {
  int rc = check_geometry("prepare_fwd", W, nb, dtype);
  if (rc) return rc;
  if (B <= 0 || T <= 0) return fail(RGLRU_E_ARG, "prepare_fwd: B and T must be positive (got %lld, %lld)", (long long)B, (long long)T);
  if (!ws) return fail(RGLRU_E_ARG, "prepare_fwd: null pointer");
  // The parameter conversion also zeroes the forward records, tickets and failure word of `ws`.  It is a launch
  // of its own in front of the forward kernel, or part of the forward launch where that kernel can do it (fwd_impl).
  const WorkLayout L = make_work_layout(B, T, make_geometry(W, nb));
  PrepArgs pa;
  rc = build_prep_args(w_a, b_a, w_x, b_x, lambda, c, W, nb, dtype, vec_dtype, prep, (char*)ws + L.f_begin, L.f_end - L.f_begin, pa);
  if (rc) return rc;
  return fwd_impl(x, prep, h0, flags, y, h_last, ws, B, T, W, nb, dtype, true, stream, nullptr, nullptr, &pa);
}

int rglru_hip_block_fwd(const void* u, int64_t u_stride, const void* v, int64_t v_stride,
                        const void* conv_state, const void* taps, const void* conv_bias, int64_t K, int vec_dtype,
                        const void* prep, const float* h0, const uint8_t* flags,
                        void* x_conv, void* y, void* gated, void* new_conv_state, float* h_last, void* ws,
                        int64_t B, int64_t T, int64_t W, int64_t nb, int dtype, void* stream) {
  const BlockFwd blk = {v, u_stride, v_stride, conv_state, taps, conv_bias, K, vec_dtype, x_conv, gated, new_conv_state};
  return fwd_impl(u, prep, h0, flags, y, h_last, ws, B, T, W, nb, dtype, false, stream, nullptr, &blk);
}

int rglru_hip_prepare_block_fwd(const void* w_a, const void* b_a, const void* w_x, const void* b_x,
                                const void* lambda, float c, int vec_dtype, void* prep,
                                const void* u, int64_t u_stride, const void* v, int64_t v_stride,
                                const void* conv_state, const void* taps, const void* conv_bias, int64_t K,
                                const float* h0, const uint8_t* flags,
                                void* x_conv, void* y, void* gated, void* new_conv_state, float* h_last, void* ws,
                                int64_t B, int64_t T, int64_t W, int64_t nb, int dtype, void* stream) {
  int rc = check_geometry("prepare_block_fwd", W, nb, dtype);
  if (rc) return rc;
  if (B <= 0 || T <= 0) return fail(RGLRU_E_ARG, "prepare_block_fwd: B and T must be positive (got %lld, %lld)", (long long)B, (long long)T);
  if (!ws) return fail(RGLRU_E_ARG, "prepare_block_fwd: null pointer");
  const WorkLayout L = make_work_layout(B, T, make_geometry(W, nb));
  rc = prepare_impl(w_a, b_a, w_x, b_x, lambda, c, W, nb, dtype, vec_dtype, prep, (char*)ws + L.f_begin, L.f_end - L.f_begin, stream);
  if (rc) return rc;
  const BlockFwd blk = {v, u_stride, v_stride, conv_state, taps, conv_bias, K, vec_dtype, x_conv, gated, new_conv_state};
  return fwd_impl(u, prep, h0, flags, y, h_last, ws, B, T, W, nb, dtype, true, stream, nullptr, &blk);
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

int rglru_hip_set_chain_forward(int mode) { return g_chain_forward.exchange(mode < 0 || mode > 2 ? 0 : mode); }
int rglru_hip_set_timing(int enable) { return g_timing.exchange(enable ? 1 : 0); }

float rglru_hip_kernel_ms(int which) {
  if (which < 0 || which > 3) return -1.f;
  TimingSlot& slot = timing_slot(which);
  if (!slot.armed) return -1.f;
  float ms = -1.f;
  if (hipEventSynchronize(slot.stop) != hipSuccess || hipEventElapsedTime(&ms, slot.start, slot.stop) != hipSuccess) return -1.f;
  return ms;
}

int rglru_hip_workspace_status(const void* ws, int64_t B, int64_t T, int64_t W, int64_t nb,
                               int scan_only, void* stream, int* status) {
  if (!ws || !status) return fail(RGLRU_E_ARG, "workspace_status: null pointer");
  size_t off;
  if (scan_only) off = make_scan_layout(B, T, W).fail;
  else {
    if (nb <= 0 || W % nb) return fail(RGLRU_E_ARG, "workspace_status: bad geometry");
    off = make_work_layout(B, T, make_geometry(W, nb)).fail;
  }
  unsigned word = 0;
  hipError_t e = hipMemcpyAsync(&word, (const char*)ws + off, 4, hipMemcpyDeviceToHost, (hipStream_t)stream);
  if (e == hipSuccess) e = hipStreamSynchronize((hipStream_t)stream);
  if (e != hipSuccess) return fail(RGLRU_E_LAUNCH, "workspace_status: %s", hipGetErrorString(e));
  *status = (int)word;
  return RGLRU_OK;
}

}  // extern "C"
