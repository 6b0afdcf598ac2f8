// Fused RG-LRU kernels for gfx950: parameter preparation and forward (this file), backward
// (rglru_fused_bwd.hip), decode step (rglru_decode.hip); what they share is in rglru_fused.h.
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


#include "rglru_fused.h"

namespace rglru {

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
// K groups of the weights that a wave keeps in LDS instead of registers (HeldWeights) where two workgroups a
// compute unit leave too few registers.  The compiler's own spill goes to scratch memory: its reloads sit at the top of
// the gate products and wait for every vector memory operation in flight, the record prefetch of the look-back
// included.  Chosen so that nothing spills (224-wide masked: 4 registers still do) and two workgroups still fit the
// LDS (8 KB per group and workgroup).  Forward at B1 T32768, us: 224-wide 163 -> 158, 320-wide 314 -> 292.
constexpr int fwd_lds_groups(int nkg, bool masked) {
  return nkg == 14 ? (masked ? 4 : 3) : nkg == 18 ? (masked ? 5 : 0) : nkg == 20 ? (masked ? 6 : 4) : 0;
}

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

  const WaveId w = wave_identity(p, blockIdx.x, NKG > 8);
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
    constexpr int LDSG = NKG > 0 ? fwd_lds_groups(NKG, MASKED) : 0;
    Frag* spill = nullptr;
    if constexpr (LDSG > 0) {
      __shared__ __attribute__((aligned(16))) Frag lds_hw[kWaves * 2 * LDSG * 64];
      spill = lds_hw + w.wave * (2 * LDSG * 64);
    }
    HeldWeights<IO, NKG, LDSG> hw;
    hw.load(w_a_row, w_x_row, spill, w.lane);
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
          gate_mfma_held<IO, MT, NKG, KC, LDSG>(lds, hw, mt, w.slab, w.r, hf, 0.0f, 0.0f, ua, ux, xv, NKG >= 8 ? 0 : w.kb, spill, w.lane);
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
