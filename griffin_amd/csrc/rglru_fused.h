// Shared by the translation units of the fused RG-LRU kernels (forward, backward, decode): kernel
// arguments, the wave/tile helpers the kernels have in common, and the host-side checks and launch
// helpers of their entry points.
#pragma once

#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
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

// Waves of a chain kernel's workgroup (fwd_chain_kernel, bwd_delta_chain_kernel: one workgroup per chain).
constexpr int kChainWaves = 16;

RGLRU_DEVICE WaveId wave_identity(const FusedArgs& p, int block, bool scalar_wave = false) {
  WaveId w;
  w.lane = threadIdx.x & 63; w.r = w.lane & 31; w.hf = w.lane >> 5;
  // scalar_wave: the wave index is made known to be wave-uniform, so what derives from it (slab, block, buffer
  // descriptors) stays in scalar registers; where registers are short that costs more than it saves
  w.wave = scalar_wave ? __builtin_amdgcn_readfirstlane(threadIdx.x >> 6) : (int)(threadIdx.x >> 6);
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

// Register-resident weights: the wave's 32 rows of both gate matrices, NKG K groups each.  The last LDSG K
// groups can live in LDS instead (`spill`: [group][gate][lane] fragments private to the wave): where the registers
// run out, the compiler's own spill goes to scratch memory, whose reloads count as vector memory operations and
// make the wave wait for every load it has in flight.
template <typename IO, int NKG, int LDSG = 0>
struct HeldWeights {
  static constexpr int kRegs = NKG > 0 ? NKG - LDSG : 1;
  typename Io<IO>::Frag a[kRegs], x[kRegs];
  RGLRU_DEVICE void load(const IO* w_a_row, const IO* w_x_row, typename Io<IO>::Frag* spill = nullptr, int lane = 0) {
    if constexpr (NKG > 0) {
#pragma unroll
      for (int kg = 0; kg < NKG - LDSG; ++kg) {
        a[kg] = *reinterpret_cast<const typename Io<IO>::Frag*>(w_a_row + kg * Io<IO>::KG);
        x[kg] = *reinterpret_cast<const typename Io<IO>::Frag*>(w_x_row + kg * Io<IO>::KG);
      }
#pragma unroll
      for (int g = 0; g < LDSG; ++g) {
        spill[(2 * g) * 64 + lane] = *reinterpret_cast<const typename Io<IO>::Frag*>(w_a_row + (NKG - LDSG + g) * Io<IO>::KG);
        spill[(2 * g + 1) * 64 + lane] = *reinterpret_cast<const typename Io<IO>::Frag*>(w_x_row + (NKG - LDSG + g) * Io<IO>::KG);
      }
    }
  }
};

// MFMA phase for register-held weights, one accumulator tile: the whole block width (NKG * KG
// columns) is in LDS with row stride NKG * KG + HW.  Also returns the 16 x values of the tile in
// accumulator layout.
template <typename IO, int MT, int NKG, int TW = NKG * Io<IO>::KG, int LDSG = 0>
RGLRU_DEVICE void gate_mfma_held(const IO* lds, const HeldWeights<IO, NKG, LDSG>& hw, int mt, int slab, int r, int hf,
                                 float bias_a, float bias_x, f32x16& ua, f32x16& ux, float (&xv)[16], int kb = 0,
                                 const typename Io<IO>::Frag* spill = nullptr, int lane = 0) {
  typedef Io<IO> Tr;
  typedef typename Tr::Frag Frag;
  constexpr int KG = Tr::KG, HW = Tr::HW;
  constexpr int LDSROW = TW + HW;                          // the tile is TW columns wide; the block starts at kb
#pragma unroll
  for (int v = 0; v < 16; ++v) { ua[v] = bias_a; ux[v] = bias_x; }
  const IO* row = lds + tile_row<MT>(mt, r) * LDSROW + kb + hf * HW;
#pragma unroll
  for (int kg = 0; kg < NKG - LDSG; ++kg) {
    Frag xa = *reinterpret_cast<const Frag*>(row + kg * KG);
    Tr::mma(ua, xa, hw.a[kg]);
    Tr::mma(ux, xa, hw.x[kg]);
  }
#pragma unroll
  for (int g = 0; g < LDSG; ++g) {
    Frag xa = *reinterpret_cast<const Frag*>(row + (NKG - LDSG + g) * KG);
    Tr::mma(ua, xa, spill[(2 * g) * 64 + lane]);
    Tr::mma(ux, xa, spill[(2 * g + 1) * 64 + lane]);
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
// Host side
// ------------------------------------------------------------------------------------------
inline int check_geometry(const char* who, int64_t W, int64_t nb, int dtype) {
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
inline int check_extents(const char* who, int64_t B, int64_t T, int64_t W) {
  if (B * T * W >= (1ll << 40) || B * T >= (1ll << 31)) return fail(RGLRU_E_UNSUPPORTED, "%s: tensor too large", who);
  const int64_t slots = 4 * ((T + 63) / 64);              // checkpoint slots per sequence
  if (slots * W * 4 >= (1ll << 31))
    return fail(RGLRU_E_UNSUPPORTED, "%s: one sequence of %lld tokens x %lld channels exceeds the 2 GiB per-sequence workspace limit; split the sequence and carry the state", who, (long long)T, (long long)W);
  if (B * W * 4 >= (1ll << 31)) return fail(RGLRU_E_UNSUPPORTED, "%s: state tensor [%lld, %lld] too large", who, (long long)B, (long long)W);
  return RGLRU_OK;
}

inline size_t elem_size(int dtype) { return dtype == RGLRU_BF16 ? 2 : 4; }

inline void fill_common(FusedArgs& a, const Geometry& g, const void* prep, int dtype) {
  PrepLayout pl = make_prep_layout(g, elem_size(dtype));
  const char* pb = (const char*)prep;
  a.wg = pb + pl.wg; a.bias = (const float*)(pb + pl.bias); a.sp = (const float*)(pb + pl.sp); a.cs = (const float*)(pb + pl.cs);
  a.w2t = pb + pl.w2t;
  a.W = (int)g.W; a.nb = (int)g.nb; a.bw = (int)g.bw; a.bwp = (int)g.bwp; a.S = (int)g.S; a.Wp = (int)g.Wp;
  a.groups = (int)g.groups; a.units = (int)g.units; a.bpu = 1;
  a.limit = spin_limit();
  a.full_slabs = (g.bw % 32 == 0) ? 1 : 0;
}

inline const float* finish_dsp(const Geometry& g, const void* prep, int dtype) {
  return (const float*)((const char*)prep + make_prep_layout(g, elem_size(dtype)).dsp);
}

inline int is_aligned(const void* ptr, int64_t W, int64_t bw, size_t es) {
  return ((uintptr_t)ptr % 16 == 0) && ((W * (int64_t)es) % 16 == 0) && ((bw * (int64_t)es) % 16 == 0);
}

// number of register-held K groups for this block width, or 0 for the streaming variant
inline int held_groups(const Geometry& g, int dtype, int aligned) {
  if (dtype == RGLRU_BF16 && aligned && g.bw == g.bwp) {
    if (g.bwp == 128) return 8;
    if (g.bwp == 64) return 4;
    if (g.bwp == 32) return 2;
  }
  return 0;
}

// K steps of 32 channels of the decode kernels on 16 x 16 tiles (gate blocks of 32 .. 384 channels in steps
// of 32, 16-bit storage, aligned rows), or 0 for the portable decode kernels
inline int step16_groups(const Geometry& g, int dtype, int aligned) {
  if (dtype != RGLRU_BF16 || !aligned || g.bw != g.bwp || g.bw > 384) return 0;
  return (int)(g.bw / 32);
}

// ... and for the blocks wider than a workgroup's four slabs whose weights the forward and the
// gate-gradient kernels hold in registers: K groups (bw / 16), or 0
inline int wide_groups(const Geometry& g, int dtype, int aligned) {
  if (dtype != RGLRU_BF16 || !aligned) return 0;
  switch (g.bw) {
    case 160: case 192: case 224: case 256: case 288: case 320: case 352: case 384: return (int)(g.bw / 16);
    default: return 0;
  }
}

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

inline int launch_clear(char* base, size_t begin, size_t end, hipStream_t s) {
  long long words = (long long)(end - begin) / 4;
  int cb = (int)((words + 1023) / 1024); if (cb > 2048) cb = 2048; if (cb < 1) cb = 1;
  hipLaunchKernelGGL(clear_words_kernel, dim3(cb), dim3(256), 0, s, (unsigned*)(base + begin), words);
  return check_launch("workspace clear");
}

// Optional event bracket around the main kernel of an entry point (measurement hook).
inline std::atomic<int> g_timing{0};
struct TimingSlot { hipEvent_t start = nullptr, stop = nullptr; bool armed = false; };
inline TimingSlot& timing_slot(int which) {
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
inline void pack_units(FusedArgs& a, const Geometry& g, int nkg) {
  if (nkg == 4 || nkg == 2) {
    a.bpu = kPackedWidth / (int)g.bw;
    a.units = (int)((g.nb + a.bpu - 1) / a.bpu);
  }
}

inline int pick_wg_per_unit(int units, long long tiles_per_unit, int per_cu, long long cap) {
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
inline int pick_queues(long long B, int wg) {
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


// Whether the forward runs one workgroup per chain (fwd_chain_kernel) instead of tiles with look-back:
// 0 = by shape, 1 = never, 2 = whenever that kernel covers the shape (tests).
inline std::atomic<int> g_chain_forward{0};
inline bool fwd_chain_pays(int64_t B, int64_t T, int64_t W) {
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

}  // namespace rglru
