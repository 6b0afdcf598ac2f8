// Device-side building blocks shared by the RG-LRU kernels (gfx950 / CDNA4, wave64).
//
//  * MFMA fragment wrappers for the two storage types (bf16 -> v_mfma_f32_32x32x16_bf16,
//    fp32 -> 4 x v_mfma_f32_32x32x2_f32), with one common 16-byte-per-lane fragment shape;
//  * the time <-> matrix-row permutation that makes every lane of an accumulator tile own a run
//    of consecutive time steps of one channel;
//  * the chunk carry protocol (publish / look back) used by all scans;
//  * the per-element gate math of griffin/griffin.py:237-255.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace rglru {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

constexpr int kChunk = 32;          // tokens per backward chunk (RGLRU_CHUNK); checkpoints every kChunk / 2
constexpr int kWaves = 4;           // waves per workgroup in the fused kernels
constexpr int kThreads = 64 * kWaves;
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

#define RGLRU_DEVICE __device__ __forceinline__

// ------------------------------------------------------------------------------------------
// Storage-type traits.  A "fragment" is 16 bytes per lane: lane (r = lane % 32, hf = lane / 32)
// holds, for matrix row (A operand) or column (B operand) r, the HW consecutive K elements that
// start at hf * HW inside a K group of KG elements.
// ------------------------------------------------------------------------------------------
template <typename IO> struct Io;

template <> struct Io<__bf16> {
  typedef bf16x8 Frag;
  static constexpr int KG = 16;      // K elements consumed per fragment pair
  static constexpr int HW = 8;       // elements per lane
  static constexpr int KCMAX = 256;  // widest K slice staged in LDS at once
  static RGLRU_DEVICE void mma(f32x16& acc, const Frag& a, const Frag& b) {
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc, 0, 0, 0);
  }
  static RGLRU_DEVICE Frag zero() { Frag f; for (int i = 0; i < 8; ++i) f[i] = (__bf16)0.0f; return f; }
};

template <> struct Io<float> {
  typedef f32x4 Frag;
  static constexpr int KG = 8;
  static constexpr int HW = 4;
  static constexpr int KCMAX = 128;
  static RGLRU_DEVICE void mma(f32x16& acc, const Frag& a, const Frag& b) {
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[0], b[0], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[1], b[1], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[2], b[2], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[3], b[3], acc, 0, 0, 0);
  }
  static RGLRU_DEVICE Frag zero() { Frag f = {0.f, 0.f, 0.f, 0.f}; return f; }
};

// ------------------------------------------------------------------------------------------
// Buffer addressing.  Tiles are read and written through raw buffer descriptors whose base is the
// first row of the tile and whose extent covers only the rows that exist: 32-bit lane offsets, a
// scalar row offset, and accesses past the extent are dropped by the hardware (loads return 0),
// which removes every bounds branch from the streaming code.  Only the per-lane offset takes part
// in the range check, so code that relies on it puts the row term into the lane offset.
// ------------------------------------------------------------------------------------------
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef __amdgpu_buffer_rsrc_t rsrc_t;
// Offset that no extent reaches.  It is 16-byte aligned: atomics must be naturally aligned even
// when the range check is going to drop them.
constexpr unsigned kOutOfRange = 0x7ffffff0u;

RGLRU_DEVICE rsrc_t make_rsrc(const void* base, unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}

template <typename IO> struct BufIo;
template <> struct BufIo<__bf16> {
  static RGLRU_DEVICE void store(__bf16 v, rsrc_t r, unsigned voff, unsigned soff) {
    __builtin_amdgcn_raw_buffer_store_b16(__builtin_bit_cast(short, v), r, voff, soff, 0);
  }
  static RGLRU_DEVICE float load(rsrc_t r, unsigned voff, unsigned soff) {
    return (float)__builtin_bit_cast(__bf16, (short)__builtin_amdgcn_raw_buffer_load_b16(r, voff, soff, 0));
  }
};
template <> struct BufIo<float> {
  static RGLRU_DEVICE void store(float v, rsrc_t r, unsigned voff, unsigned soff) {
    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(int, v), r, voff, soff, 0);
  }
  static RGLRU_DEVICE float load(rsrc_t r, unsigned voff, unsigned soff) {
    return __builtin_bit_cast(float, (int)__builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, 0));
  }
};
RGLRU_DEVICE void buf_store_b128(i32x4 v, rsrc_t r, unsigned voff) {
  __builtin_amdgcn_raw_buffer_store_b128(v, r, voff, 0, 0);
}
template <typename Frag> RGLRU_DEVICE Frag buf_load_frag(rsrc_t r, unsigned voff) {
  return __builtin_bit_cast(Frag, __builtin_amdgcn_raw_buffer_load_b128(r, voff, 0, 0));
}

// ------------------------------------------------------------------------------------------
// Per-wave output staging.  After the scan a lane holds consecutive time steps of ONE channel,
// while memory wants consecutive channels of one time step.  Two-byte stores straight from that
// layout cost one address per lane and element; instead each wave transposes its ROWS x 32 tile of
// 16-bit values through a private LDS area (two-byte LDS writes, 16-byte LDS reads) and writes
// 64-byte row segments with 16-byte stores.  The upper half-wave's rows are skewed by 64 bytes so
// that the two halves use different banks.
// ------------------------------------------------------------------------------------------
template <int ROWS> struct WaveStage {
  static constexpr int kRowBytes = 64;
  static constexpr int kBytes = ROWS * kRowBytes + 128;
  static RGLRU_DEVICE unsigned row_offset(int row) { return (unsigned)row * kRowBytes + (row >= ROWS / 2 ? 64u : 0u); }
};

// LDS operations of one wave execute in program order, so lanes of the same wave may exchange data
// through LDS as long as the COMPILER keeps the order: the asm statement is a full compiler barrier
// for memory accesses (a fence alone does not order plain accesses of different types).
RGLRU_DEVICE void wave_lds_fence() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Store a staged ROWS x 32 tile of 16-bit values: `r` covers the tile's rows (row stride
// row_bytes), col_bytes is the byte offset of the wave's first channel inside a row.
template <int ROWS>
RGLRU_DEVICE void stage_flush(const unsigned char* stage, rsrc_t r, unsigned row_bytes, unsigned col_bytes, int lane) {
#pragma unroll
  for (int i = 0; i < ROWS / 16; ++i) {
    const int row = 16 * i + (lane >> 2);
    const unsigned seg = (unsigned)(lane & 3) * 16u;
    i32x4 v = *reinterpret_cast<const i32x4*>(stage + WaveStage<ROWS>::row_offset(row) + seg);
    buf_store_b128(v, r, (unsigned)row * row_bytes + col_bytes + seg);
  }
}

// Matrix operand from a row-major bf16 tile in LDS whose ROWS are the contraction index (ds_read_b64_tr_b16, a
// gfx950 instruction).  Within a group of 16 lanes, lane s names four consecutive elements and lane i receives
// element i % 4 of the lanes i / 4, i / 4 + 4, i / 4 + 8, i / 4 + 12.  With lane s pointing at row s / 4,
// columns 4 (s % 4) .. + 3 of a 4 x 16 patch, lane i ends up with the patch's column i, rows 0 .. 3.  Two
// such reads give the fragment of a 32 x 32 x 16 product: lane (n = lane % 32, hf = lane / 32) holds rows
// k0 + 8 hf .. + 7 of column col0 + n.  (The 16-byte row-wise read needs the tile transposed first.)
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4_lds;
RGLRU_DEVICE bf16x8 lds_transposed_frag(const __bf16* tile, int row_stride, int k0, int col0, int lane) {
  typedef __attribute__((address_space(3))) bf16x4_lds* lds_ptr_t;
  const int i = lane & 15, g = lane >> 4;
  const __bf16* src = tile + (k0 + 8 * (g >> 1) + (i >> 2)) * row_stride + col0 + 16 * (g & 1) + 4 * (i & 3);
  const bf16x4_lds lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_ptr_t)(src));
  const bf16x4_lds hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_ptr_t)(src + 4 * row_stride));
  return __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
}

// Row m (0..31) of accumulator tile mt holds local time step tile_row(mt, m).  With this map,
// register v of tile mt in lane half hf is local time hf * 16 * MT + 16 * mt + v: each lane
// owns 16 * MT consecutive steps, the lower half-wave the first half of the tile.
template <int MT> RGLRU_DEVICE int tile_row(int mt, int m) {
  return ((m >> 2) & 1) * (16 * MT) + mt * 16 + ((m >> 3) << 2) + (m & 3);
}

// Value held by the lane 32 positions away (lower <-> upper half-wave).
RGLRU_DEVICE float xhalf(float v, int hf) {
  unsigned u = __float_as_uint(v);
  auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __uint_as_float(hf ? r[0] : r[1]);
}

// ------------------------------------------------------------------------------------------
// Chunk carry protocol.  A scan over time is cut into chunks that are processed by different
// waves.  Each (sequence, chunk, channel) owns ONE 64-bit record that describes the chunk as an
// affine map of the carry, carry_out = A * carry_in + H:  low word = bits of A with the lowest
// mantissa bit forced to 1, high word = bits of H.
//   low word == 0   nothing published yet (records start out cleared)
//   low word == 1   A = 0: the chunk knows its carry_in and H is its carry_out; a walk ends here
//   otherwise       (A, H) is the chunk's own map and the reader goes on to the chunk before
// The record travels in one naturally aligned 8-byte access issued at device scope (sc1), so a reader
// sees it entirely or not at all and no fence is needed on either side; a chunk that learns its
// carry simply overwrites its record.  A wave that needs its carry_in loads the records of the
// kDepth chunks before it in one round trip and composes them in chain order until A becomes 0 or
// the boundary is reached.  Chunks are handed out through ticket counters in chain order, so every
// record a wave waits for belongs to a wave that is already running.
// ------------------------------------------------------------------------------------------
typedef unsigned long long rec_t;
#ifndef RGLRU_DEPTH
#define RGLRU_DEPTH 2
#endif
constexpr int kDepth = RGLRU_DEPTH;

RGLRU_DEVICE void rec_store(rec_t* p, float a, float h) {
  const rec_t bits = ((rec_t)__float_as_uint(h) << 32) | (rec_t)(__float_as_uint(a) | 1u);
  __hip_atomic_store(p, bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// cache policy of a record access issued through a buffer descriptor: device scope (sc1)
constexpr int kRecPolicy = 16;

RGLRU_DEVICE rec_t rec_load(const rec_t* p) {
  return __hip_atomic_load(const_cast<rec_t*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

struct CarryChain {
  rec_t* rec;         // per-lane pointer, already offset to (sequence, channel); chunk c at + c * stride
  long long stride;
};

// Publish the chunk's own map (final = false) or its carry_out (final = true, `a` is ignored).
RGLRU_DEVICE void carry_publish(const CarryChain& ch, int c, float a, float h, bool final) {
  rec_store(ch.rec + c * ch.stride, final ? 0.f : a, h);
}

// State of one walk along a chain: the composed map of the chunks consumed so far.
struct CarryWalk {
  float acc_a, acc_h;
  bool done;
  int p;              // next chunk to consume
};

// DEPTH = records requested per round trip.  Measured, two is the best choice for every kernel here:
// deeper batches shorten no walk in practice and every extra device-scope load costs (reverse scan at
// B8 T2048 W1024: 36 / 38 / 43 us with 2 / 4 / 8 records per round trip, forward 38 / 40 / 42 us).

// Compose one batch of records (chunks p, p + step, ...) into the walk.  Returns true when the
// batch ran into a record that is not published yet; p then names that chunk.
// finals_only: a record counts as published only once it is final, so every chunk takes its carry from
// the chunk right before it and the result does not depend on which records happened to be final when
// they were read (bit-reproducible; the chain is then as slow as one round trip per chunk).
template <int DEPTH>
RGLRU_DEVICE bool carry_compose(const rec_t (&rec)[DEPTH], CarryWalk& wk, int step, int end, float boundary,
                                bool finals_only = false) {
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) {
    const int q = wk.p + d * step;
    if (q == end) {                                      // wave-uniform
      if (!wk.done) { wk.acc_h = fmaf(wk.acc_a, boundary, wk.acc_h); wk.acc_a = 0.f; wk.done = true; }
      return false;
    }
    const unsigned lo = (unsigned)rec[d];
    if (!__all(wk.done || (finals_only ? lo == 1u : lo != 0u))) { wk.p = q; return true; }
    if (!wk.done) {
      wk.acc_h = fmaf(wk.acc_a, __uint_as_float((unsigned)(rec[d] >> 32)), wk.acc_h);
      if (lo == 1u) { wk.acc_a = 0.f; wk.done = true; }
      else wk.acc_a *= __uint_as_float(lo);
    }
  }
  wk.p += DEPTH * step;
  return false;
}

// Polling part of a walk: load a batch, compose, repeat until every lane has its carry.  After
// `limit` fruitless polls the wave records the failure and returns NaN as the carry of the lanes that
// are still waiting, so every wave still reaches the end of the kernel and the failure is visible in
// the results themselves (the chunk's outputs and the carry it hands on turn NaN) without anybody
// having to read the failure word.
// A negative `limit` asks for finals_only with -limit polls (one argument carries both through the kernels).
template <int DEPTH>
RGLRU_DEVICE float carry_walk(const CarryChain& ch, CarryWalk& wk, int step, int end, float boundary,
                              long long limit, unsigned* fail_word) {
  const bool finals_only = limit < 0;
  if (finals_only) limit = -limit;
  long long polls = 0;
  while (!__all(wk.done)) {
    rec_t rec[DEPTH];
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      const int q = wk.p + d * step;
      const bool inside = (step < 0) ? (q > end) : (q < end);
      rec[d] = 0;
      if (inside && !wk.done) rec[d] = rec_load(ch.rec + q * ch.stride);
    }
    if (carry_compose<DEPTH>(rec, wk, step, end, boundary, finals_only)) {
      if (++polls > limit) {
        if ((threadIdx.x & 63) == 0) atomicOr(fail_word, 1u);
        if (!wk.done) wk.acc_h = __builtin_nanf("");
        break;
      }
      __builtin_amdgcn_s_sleep(1);
    }
  }
  return wk.acc_h;
}

// carry_in of chunk c.  `step` is -1 when the chain runs forward in time (the chunk before c is
// c - 1) and +1 when it runs backward; `end` is the index one past the first chunk of the chain
// (-1 or the chunk count), where `boundary` is the carry.
template <int DEPTH = kDepth>
RGLRU_DEVICE float carry_lookback(const CarryChain& ch, int c, int step, int end, float boundary,
                                  bool lane_ok, long long limit, unsigned* fail_word) {
  CarryWalk wk;
  wk.acc_a = 1.f; wk.acc_h = 0.f; wk.done = !lane_ok; wk.p = c + step;
  return carry_walk<DEPTH>(ch, wk, step, end, boundary, limit, fail_word);
}

// The first batch of a walk requested ahead of time.  A device-scope load takes a few
// microseconds under load, far more than the gate math of a tile, so a caller that knows early
// which chunk it will finish issues these loads before other work and resolves them afterwards.
// They go through a buffer descriptor that covers the sequence's records (`lane_off` = byte offset
// of the lane's channel, or kOutOfRange for a lane without one): chunks outside the chain are
// masked by the offset instead of a branch, so the number of loads in flight is fixed and the
// hardware counter can be waited on precisely.
template <int DEPTH = kDepth>
struct CarryBatch {
  rec_t rec[DEPTH];
};

// Record store through the same kind of descriptor; voff = kOutOfRange drops it.
RGLRU_DEVICE void rec_store_buf(rsrc_t recs, unsigned voff, float a, float h) {
  typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
  u32x2 v;
  v[0] = __float_as_uint(a) | 1u; v[1] = __float_as_uint(h);
  __builtin_amdgcn_raw_buffer_store_b64(v, recs, voff, 0, kRecPolicy);
}

template <int DEPTH>
RGLRU_DEVICE void carry_prefetch(rsrc_t recs, unsigned lane_off, unsigned stride_bytes, int c, int step, int end,
                                 CarryBatch<DEPTH>& batch) {
  typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) {
    const int q = c + step + d * step;
    const bool inside = (step < 0) ? (q > end) : (q < end);
    const unsigned voff = (inside && lane_off != kOutOfRange) ? (unsigned)q * stride_bytes + lane_off : kOutOfRange;
    const u32x2 v = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(recs, voff, 0, kRecPolicy));
    batch.rec[d] = ((rec_t)v[1] << 32) | (rec_t)v[0];
  }
}

template <int DEPTH>
RGLRU_DEVICE float carry_lookback_from(const CarryBatch<DEPTH>& first, const CarryChain& ch, int c, int step, int end,
                                       float boundary, bool lane_ok, long long limit, unsigned* fail_word) {
  CarryWalk wk;
  wk.acc_a = 1.f; wk.acc_h = 0.f; wk.done = !lane_ok; wk.p = c + step;
  carry_compose<DEPTH>(first.rec, wk, step, end, boundary, limit < 0);
  return carry_walk<DEPTH>(ch, wk, step, end, boundary, limit, fail_word);
}

// ------------------------------------------------------------------------------------------
// Gate math for one element (griffin/griffin.py:237-255), fp32.
//   ua, ux : gate pre-activations W_a x + b_a, W_x x + b_x
//   sp     : c * log2(sigmoid(Lambda)) for this channel  (so log2 a = r * sp)
//   fl     : RGLRU_FLAG_* bits of this token
// ------------------------------------------------------------------------------------------
struct GateOut {
  float r, i, a, g, g2, z;   // a, g, g2 = g * g and z include the token's masks
};

// sigmoid(u + b) with the bias passed as nb = -log2(e) * b: the addition rides on the multiplication
// the exponent needs anyway, and a matrix product that feeds u can start from a zero accumulator.
RGLRU_DEVICE float sigmoid_fast(float u, float nb = 0.0f) {
  return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(fmaf(-kLog2e, u, nb)));
}

// 1 - exp(y) for y <= 0 without cancellation: Taylor series near zero, direct form elsewhere.
// PRECISE (fp32 storage): degree-7 series below |y| = 0.25, relative error < 1e-7 everywhere.
// Otherwise (bf16 storage): two-term series below |y| = 2^-7, relative error < 2e-5.
template <bool PRECISE>
RGLRU_DEVICE float one_minus_exp(float y, float a) {
  const float direct = fmaf(-a, a, 1.0f);
  if constexpr (PRECISE) {
    float q = 1.0f / 5040.0f;
    q = fmaf(q, y, 1.0f / 720.0f);
    q = fmaf(q, y, 1.0f / 120.0f);
    q = fmaf(q, y, 1.0f / 24.0f);
    q = fmaf(q, y, 1.0f / 6.0f);
    q = fmaf(q, y, 0.5f);
    q = fmaf(q, y, 1.0f);
    return y > -0.25f ? -y * q : direct;
  } else {
    const float series = -y * fmaf(y, 0.5f, 1.0f);
    return y > -0.0078125f ? series : direct;
  }
}

// g^2 = 1 - a^2 for a = 2^l2, l2 <= 0.  PRECISE: the series above in y = 2 ln2 l2, clamped at zero.  Otherwise the
// two-term series written as a polynomial in l2 itself, -y (1 + y / 2) = l2 (k1 + k2 l2), so that no product
// with 2 ln2 is spent on an argument; neither branch can turn negative for l2 <= 0 (a <= 1), so there is no clamp
// (a NaN then stays a NaN instead of turning into g = 0).
template <bool PRECISE>
RGLRU_DEVICE float one_minus_a2(float l2, float a) {
  if constexpr (PRECISE) {
    return fmaxf(one_minus_exp<true>(l2 * (2.0f * kLn2), a), 0.0f);
  } else {
    constexpr float k1 = -2.0f * kLn2, k2 = -2.0f * kLn2 * kLn2;
    const float series = l2 * fmaf(l2, k2, k1);
    return l2 > -0.0078125f / (2.0f * kLn2) ? series : fmaf(-a, a, 1.0f);
  }
}

// log2 of the decay under the token's flags.  Both masks of the reference act through it alone:
//   padding (a <- 1, z <- 0): log2 a = 0 gives a = 1 and, through the series branch of
//     one_minus_exp, g = 0 exactly, hence z = 0;
//   reset (a <- 0, g <- 1): log2 a = -126 gives a = 2^-126 (the state it lets through is below
//     1e-38 of its value) and g = sqrt(1 - a^2) = 1 exactly.
// Padding wins when both are set, as in griffin/griffin.py:248-255.
constexpr float kResetLog2 = -126.0f;
RGLRU_DEVICE float masked_log2_decay(float l2, unsigned fl) {
  l2 = (fl & 1u) ? kResetLog2 : l2;
  return (fl & 2u) ? 0.0f : l2;
}
// The same for token e of a packed run (two flag bits per token): bit-field extracts that sign-extend
// a flag into an all-ones mask and bitwise selects, so no compare results are kept per token.
RGLRU_DEVICE float masked_log2_decay_run(float l2, unsigned flbits, int e) {
  unsigned m_reset = (unsigned)__builtin_amdgcn_sbfe((int)flbits, 2 * e, 1);
  unsigned m_pad = (unsigned)__builtin_amdgcn_sbfe((int)flbits, 2 * e + 1, 1);
  asm("" : "+v"(m_reset), "+v"(m_pad));          // opaque: keeps the compiler from turning the masks back into compares
  unsigned u = __builtin_bit_cast(unsigned, l2);
  u = (u & ~m_reset) | (__builtin_bit_cast(unsigned, kResetLog2) & m_reset);
  u &= ~m_pad;
  return __builtin_bit_cast(float, u);
}

// Gate outputs from the two sigmoids and the (possibly masked) log2 of the decay.
template <bool PRECISE>
RGLRU_DEVICE GateOut gate_outputs(float r, float i, float x, float l2) {
  GateOut o;
  o.r = r; o.i = i;
  const float a = __builtin_amdgcn_exp2f(l2);
  const float g2 = one_minus_a2<PRECISE>(l2, a);
  const float g = __builtin_amdgcn_sqrtf(g2);
  o.g2 = g2;
  o.a = a; o.g = g; o.z = g * i * x;
  return o;
}
// MASKED = false: the token is known to be an ordinary one (no reset, active), fl is ignored.
template <bool PRECISE, bool MASKED>
RGLRU_DEVICE GateOut gate_forward(float ua, float ux, float x, float sp, unsigned fl, float nba = 0.0f, float nbx = 0.0f) {
  const float r = sigmoid_fast(ua, nba), i = sigmoid_fast(ux, nbx);
  float l2 = r * sp;                           // log2(a) <= 0
  if constexpr (MASKED) l2 = masked_log2_decay(l2, fl);
  return gate_outputs<PRECISE>(r, i, x, l2);
}
// Token e of a run whose flags are packed two bits per token.
template <bool PRECISE>
RGLRU_DEVICE GateOut gate_forward_run(float ua, float ux, float x, float sp, unsigned flbits, int e,
                                      float nba = 0.0f, float nbx = 0.0f) {
  const float r = sigmoid_fast(ua, nba), i = sigmoid_fast(ux, nbx);
  return gate_outputs<PRECISE>(r, i, x, masked_log2_decay_run(r * sp, flbits, e));
}

// gelu_tanh(v) = v/2 * (1 + tanh(u)), u = sqrt(2/pi) * (v + 0.044715 v^3), and its derivative
// (activation of the recurrent block's second branch, griffin/griffin.py:464).
struct GeluParts { float gelu, dgelu; };
RGLRU_DEVICE GeluParts gelu_tanh_parts(float v) {
  const float k0 = 0.7978845608028654f, k1 = 0.044715f;
  const float v2 = v * v;
  const float u = k0 * v * fmaf(k1, v2, 1.0f);
  // tanh(u) = 1 - 2 / (1 + exp(2u)); exp overflows to +inf for large u, which gives tanh = 1
  const float e = __builtin_amdgcn_exp2f(u * (2.0f * kLog2e));
  const float t = 1.0f - 2.0f * __builtin_amdgcn_rcpf(1.0f + e);
  GeluParts g;
  g.gelu = 0.5f * v * (1.0f + t);
  const float du = k0 * fmaf(3.0f * k1, v2, 1.0f);
  g.dgelu = fmaf(0.5f * v * fmaf(-t, t, 1.0f), du, 0.5f * (1.0f + t));
  return g;
}

template <typename IO> struct Precise { static constexpr bool value = true; };
template <> struct Precise<__bf16> { static constexpr bool value = false; };

}  // namespace rglru
