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

constexpr int kChunk = 32;          // tokens per checkpoint chunk (RGLRU_CHUNK)
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
constexpr unsigned kOutOfRange = 0x7fffffffu;

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
#ifdef RGLRU_EXP_STOREWAIT
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#endif
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
// waves.  Each (sequence, chunk, channel) owns two 64-bit records {fp32 value, 32-bit version}
// that describe the chunk as an affine map of the carry: carry_out = A * carry_in + H.
//   version 0            nothing published yet (records start out cleared)
//   version kVerLocal    (A, H) is the chunk's own map: the reader must go on to the chunk before
//   version kVerFinal    the chunk knows its carry_in: A = 0 and H = carry_out, the walk ends here
// Value and version travel in one naturally aligned 8-byte access issued at device scope (sc1), so
// a reader sees a record entirely or not at all and no fence is needed on either side; a reader
// that catches the two records of a chunk at different versions simply polls again.  A wave that
// needs its carry_in loads the records of the kDepth chunks before it in one round trip and
// composes them in chain order until the accumulated A becomes 0 or the boundary is reached.
// Chunks are handed out through ticket counters in chain order, so every record a wave waits for
// belongs to a wave that is already running.
// ------------------------------------------------------------------------------------------
typedef unsigned long long rec_t;
constexpr unsigned kVerLocal = 1u, kVerFinal = 2u;
constexpr int kDepth = 4;

RGLRU_DEVICE void rec_store(rec_t* p, float v, unsigned ver) {
  __hip_atomic_store(p, ((rec_t)ver << 32) | (rec_t)__float_as_uint(v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
RGLRU_DEVICE rec_t rec_load(const rec_t* p) {
  return __hip_atomic_load(const_cast<rec_t*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
RGLRU_DEVICE unsigned rec_ver(rec_t r) { return (unsigned)(r >> 32); }
RGLRU_DEVICE float rec_val(rec_t r) { return __uint_as_float((unsigned)r); }

struct CarryChain {
  rec_t* rec_a;       // per-lane pointers, already offset to (sequence, channel); chunk c at + c * stride
  rec_t* rec_h;
  long long stride;
};

RGLRU_DEVICE void carry_publish(const CarryChain& ch, int c, float a, float h, unsigned ver) {
  rec_store(ch.rec_a + c * ch.stride, a, ver);
  rec_store(ch.rec_h + c * ch.stride, h, ver);
}

// carry_in of chunk c.  `step` is -1 when the chain runs forward in time (the chunk before c is
// c - 1) and +1 when it runs backward; `end` is the index one past the first chunk of the chain
// (-1 or the chunk count), where `boundary` is the carry.  After `limit` fruitless polls the wave
// records the failure and returns an unspecified value, so every wave still reaches the end of the
// kernel.
RGLRU_DEVICE float carry_lookback(const CarryChain& ch, int c, int step, int end, float boundary,
                                  bool lane_ok, long long limit, unsigned* fail_word) {
  float acc_a = 1.f, acc_h = 0.f;
  bool done = !lane_ok;
  int p = c + step;
  long long polls = 0;
  for (;;) {
    rec_t ra[kDepth], rh[kDepth];
#pragma unroll
    for (int d = 0; d < kDepth; ++d) {
      const int q = p + d * step;
      const bool inside = (step < 0) ? (q > end) : (q < end);
      ra[d] = 0; rh[d] = 0;
      if (inside && !done) {
        ra[d] = rec_load(ch.rec_a + q * ch.stride);
        rh[d] = rec_load(ch.rec_h + q * ch.stride);
      }
    }
    bool stalled = false;
#pragma unroll
    for (int d = 0; d < kDepth; ++d) {
      if (stalled) break;
      const int q = p + d * step;
      if (q == end) {                                    // wave-uniform
        if (!done) { acc_h = fmaf(acc_a, boundary, acc_h); acc_a = 0.f; done = true; }
        break;
      }
      const unsigned va = rec_ver(ra[d]), vh = rec_ver(rh[d]);
      const bool ready = done || (va == vh && va != 0u);
      if (!__all(ready)) { stalled = true; p = q; break; }
      if (!done) {
        acc_h = fmaf(acc_a, rec_val(rh[d]), acc_h);
        acc_a *= rec_val(ra[d]);
        if (va == kVerFinal) { acc_a = 0.f; done = true; }
      }
    }
    if (__all(done)) break;
    if (stalled) {
      if (++polls > limit) {
        if ((threadIdx.x & 63) == 0) atomicOr(fail_word, 1u);
        break;
      }
      __builtin_amdgcn_s_sleep(1);
    } else {
      p += kDepth * step;
    }
  }
  return acc_h;
}

// ------------------------------------------------------------------------------------------
// Gate math for one element (griffin/griffin.py:237-255), fp32.
//   ua, ux : gate pre-activations W_a x + b_a, W_x x + b_x
//   sp     : c * log2(sigmoid(Lambda)) for this channel  (so log2 a = r * sp)
//   fl     : RGLRU_FLAG_* bits of this token
// ------------------------------------------------------------------------------------------
struct GateOut {
  float r, i, a, g, g2, z;   // a, g, z are post-mask; g2 = 1 - a_raw^2 is pre-mask
};

RGLRU_DEVICE float sigmoid_fast(float u) {
  return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-kLog2e * u));
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

// MASKED = false: the token is known to be an ordinary one (no reset, active), fl is ignored.
template <bool PRECISE, bool MASKED>
RGLRU_DEVICE GateOut gate_forward(float ua, float ux, float x, float sp, unsigned fl) {
  GateOut o;
#ifdef RGLRU_EXP_NOGATES
  o.r = ua; o.i = ux; o.a = 0.9f; o.g = 0.4f; o.g2 = 0.16f; o.z = x * ux; return o;
#endif
  o.r = sigmoid_fast(ua);
  o.i = sigmoid_fast(ux);
  float l2 = o.r * sp;                         // log2(a) <= 0
  float a = __builtin_amdgcn_exp2f(l2);
  float g2 = fmaxf(one_minus_exp<PRECISE>(l2 * (2.0f * kLn2), a), 0.0f);
  float g = __builtin_amdgcn_sqrtf(g2);
  o.g2 = g2;
  if constexpr (MASKED) { if (fl & 1u) { a = 0.f; g = 1.f; } }
  float z = g * o.i * x;
  if constexpr (MASKED) { if (fl & 2u) { a = 1.f; z = 0.f; } }
  o.a = a; o.g = g; o.z = z;
  return o;
}

template <typename IO> struct Precise { static constexpr bool value = true; };
template <> struct Precise<__bf16> { static constexpr bool value = false; };

}  // namespace rglru
