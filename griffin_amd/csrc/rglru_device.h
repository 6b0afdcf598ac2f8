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
// waves.  Each (sequence, chunk, 32-channel slab) owns one status word and three fp32 records
// per channel: the chunk's affine map (A, H) with carry_out = A * carry_in + H, and, once its
// own carry_in is known, the carry it hands on ("inclusive").  Status: 0 = nothing yet,
// 1 = (A, H) valid, 2 = inclusive valid.  A wave that needs its carry_in walks towards the
// start of the chain, composing (A, H) records until it meets an inclusive one or the boundary.
// Chunks are handed out through a ticket counter in chain order, so every record a wave waits
// for belongs to a wave that is already running.
// ------------------------------------------------------------------------------------------
RGLRU_DEVICE void st_coherent(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
RGLRU_DEVICE float ld_coherent(const float* p) {
  return __hip_atomic_load(const_cast<float*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

RGLRU_DEVICE void carry_publish(unsigned* status, unsigned value) {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
  if ((threadIdx.x & 63) == 0)
    __hip_atomic_store(status, value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Poll one status word until it is non-zero (wave-uniform).  Returns 0 after `limit` polls and
// records the failure, so that every wave still reaches the end of the kernel.
RGLRU_DEVICE unsigned carry_wait(unsigned* status, long long limit, unsigned* fail_word) {
  unsigned v = __hip_atomic_load(status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  v = __builtin_amdgcn_readfirstlane(v);
  long long polls = 0;
  while (v == 0) {
    if (++polls > limit) {
      if ((threadIdx.x & 63) == 0) atomicOr(fail_word, 1u);
      return 0;
    }
    __builtin_amdgcn_s_sleep(2);
    v = __hip_atomic_load(status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    v = __builtin_amdgcn_readfirstlane(v);
  }
  return v;
}

struct CarryChain {
  float* agg_a;       // per-lane pointers, already offset to (sequence, channel); chunk c at + c * stride
  float* agg_h;
  float* incl;
  unsigned* status;   // wave-uniform pointer, chunk c at + c * status_stride
  long long stride;
  long long incl_stride;
  long long status_stride;
};

// carry_in of chunk c.  `step` is -1 when the chain runs forward in time (the predecessor of c is
// c - 1) and +1 when it runs backward; `end` is the index one past the first chunk of the chain
// (-1 or the chunk count), where `boundary` is the carry.
RGLRU_DEVICE float carry_lookback(const CarryChain& ch, int c, int step, int end, float boundary,
                                  bool lane_ok, long long limit, unsigned* fail_word) {
  float acc_a = 1.f, acc_h = 0.f;
  int p = c + step;
  for (;;) {
    if (p == end) return acc_a * boundary + acc_h;
    unsigned s = carry_wait(ch.status + p * ch.status_stride, limit, fail_word);
    if (s == 0) return acc_h;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    if (s == 2) {
      float v = lane_ok ? ld_coherent(ch.incl + p * ch.incl_stride) : 0.f;
      return acc_a * v + acc_h;
    }
    float pa = lane_ok ? ld_coherent(ch.agg_a + p * ch.stride) : 1.f;
    float ph = lane_ok ? ld_coherent(ch.agg_h + p * ch.stride) : 0.f;
    acc_h = acc_a * ph + acc_h;
    acc_a *= pa;
    p += step;
  }
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
RGLRU_DEVICE float one_minus_exp(float y, float a_squared) {
  float q = 1.0f / 5040.0f;
  q = fmaf(q, y, 1.0f / 720.0f);
  q = fmaf(q, y, 1.0f / 120.0f);
  q = fmaf(q, y, 1.0f / 24.0f);
  q = fmaf(q, y, 1.0f / 6.0f);
  q = fmaf(q, y, 0.5f);
  q = fmaf(q, y, 1.0f);
  float series = -y * q;
  float direct = 1.0f - a_squared;
  return y > -0.25f ? series : direct;
}

RGLRU_DEVICE GateOut gate_forward(float ua, float ux, float x, float sp, unsigned fl) {
  GateOut o;
  o.r = sigmoid_fast(ua);
  o.i = sigmoid_fast(ux);
  float l2 = o.r * sp;                         // log2(a) <= 0
  float a = __builtin_amdgcn_exp2f(l2);
  float g2 = one_minus_exp(l2 * (2.0f * kLn2), a * a);
  g2 = fmaxf(g2, 0.0f);
  float g = __builtin_amdgcn_sqrtf(g2);
  o.g2 = g2;
  if (fl & 1u) { a = 0.f; g = 1.f; }
  float z = g * o.i * x;
  if (fl & 2u) { a = 1.f; z = 0.f; }
  o.a = a; o.g = g; o.z = z;
  return o;
}

}  // namespace rglru
