// The two block-diagonal GEMMs of the gate gradients (griffin/griffin.py:149-154 under autograd) for the
// configurations whose backward kernel leaves the gradients at the gate pre-activations in memory
// (rglru_hip_bwd: fp32 storage, block widths that are no multiple of 32, unaligned tensors, bf16 blocks
// wider than 384 channels):
//
//     dx[n, k bw + j] += sum_o du_a[n, k bw + o] W_a[k][o][j] + du_x[n, k bw + o] W_x[k][o][j]
//     dW_g[k][o][j]    = sum_n du_g[n, k bw + o] x[n, k bw + j]                 (g = a, x)
//
// over the flattened token axis n = b T + t.  Both run on the matrix unit (v_mfma_f32_32x32x2_f32 for fp32
// storage, v_mfma_f32_32x32x16_bf16 for bf16) and take every operand from memory in fragment layout, so
// neither needs LDS or a barrier:
//   - the first contracts over kappa = 2 o + gate.  Its B operand is the transposed, gate-interleaved copy
//     w2t[k][j][kappa] of the parameter image (16 contiguous bytes per lane); its A operand pairs du_a and
//     du_x of the same channel in registers (8 contiguous bytes from each per lane);
//   - the second contracts over tokens.  A fragment element is one token of one channel, so a lane
//     gathers its tokens one by one, and a wave-wide load is two rows of 32 consecutive channels: coalesced
//     without any transposition.  The token axis is split over workgroups; every split writes a partial
//     set [k][gate][o][j] that finish_kernel sums in a fixed order.
// Any width up to 512 per block: rows and columns outside the block and tokens outside the tensor are
// masked through the offsets of buffer loads (they read as zero) and stores (dropped).
#include <hip/hip_runtime.h>

#include <cstring>

#include "rglru_device.h"
#include "rglru_host.h"
#include "rglru_layout.h"

namespace rglru {

struct GateGemmArgs {
  const void* x; const void* du_a; const void* du_x; const void* w2t; const void* wg;
  void* dx; float* dw_partial; void* pre;
  long long N;                    // tokens, B * T
  long long tokens_per_split;     // dW: tokens of one split (a multiple of the K group)
  long long du_ld, du_blk;        // du_g[n][k][o] sits at du_g + k * du_blk + n * du_ld + o (elements)
  int W, nb, bw, bwp;
};

constexpr int kGemmJG = 4;        // 32-column tiles per wave and pass (64 accumulator registers per gate)

// dx += du . w2t^T.  A workgroup of four waves covers 128 tokens of one gate block; a wave owns 32 tokens and
// walks the block's 32-column tiles kGemmJG at a time.
template <typename IO, bool VEC>
__global__ __launch_bounds__(kThreads) void gate_dx_gemm_kernel(GateGemmArgs p) {
  typedef Io<IO> Tr;
  typedef typename Tr::Frag Frag;
  constexpr int KG = Tr::KG, HW = Tr::HW, ES = (int)sizeof(IO);
  const int lane = threadIdx.x & 63, r = lane & 31, hf = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int k = blockIdx.y;
  const long long n0 = ((long long)blockIdx.x * kWaves + wave) * 32;
  if (n0 >= p.N) return;
  const int rows = (int)((p.N - n0) < 32 ? (p.N - n0) : 32);
  const unsigned row_bytes = (unsigned)p.W * ES;
  const unsigned du_row_bytes = (unsigned)p.du_ld * ES;
  const rsrc_t ra = make_rsrc((const IO*)p.du_a + (long long)k * p.du_blk + n0 * p.du_ld, (unsigned)rows * du_row_bytes);
  const rsrc_t rx = make_rsrc((const IO*)p.du_x + (long long)k * p.du_blk + n0 * p.du_ld, (unsigned)rows * du_row_bytes);
  const rsrc_t rdx = make_rsrc((IO*)p.dx + n0 * p.W, (unsigned)rows * row_bytes);
  const IO* w2 = (const IO*)p.w2t + (long long)k * p.bwp * (2 * p.bwp);
  const unsigned col0 = (unsigned)(k * p.bw) * ES;
  const int JT = p.bwp / 32, NKG = 2 * p.bwp / KG;

  for (int jt0 = 0; jt0 < JT; jt0 += kGemmJG) {
    f32x16 acc[kGemmJG];
#pragma unroll
    for (int jj = 0; jj < kGemmJG; ++jj) {
      const int j = (jt0 + jj) * 32 + r;
      const bool col_ok = jt0 + jj < JT && j < p.bw;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int m = 8 * (v >> 2) + 4 * hf + (v & 3);
        acc[jj][v] = BufIo<IO>::load(rdx, col_ok ? (unsigned)m * row_bytes + col0 + (unsigned)j * ES : kOutOfRange, 0u);
      }
    }
    for (int kg = 0; kg < NKG; ++kg) {
      // kappa = kg KG + hf HW + i  <->  channel o = kappa / 2, gate = kappa % 2
      const int o = (kg * KG + hf * HW) / 2;
      const unsigned off = (unsigned)r * du_row_bytes + (unsigned)o * ES;
      Frag fa;
      if constexpr (ES == 4) {
        typedef float f32x2 __attribute__((ext_vector_type(2)));
        f32x2 a, x;
        if constexpr (VEC) {
          const unsigned voff = o < p.bw ? off : kOutOfRange;     // bw is even on the vector path
          a = __builtin_bit_cast(f32x2, __builtin_amdgcn_raw_buffer_load_b64(ra, voff, 0, 0));
          x = __builtin_bit_cast(f32x2, __builtin_amdgcn_raw_buffer_load_b64(rx, voff, 0, 0));
        } else {
#pragma unroll
          for (int i = 0; i < 2; ++i) {
            const unsigned voff = o + i < p.bw ? off + 4u * i : kOutOfRange;
            a[i] = BufIo<float>::load(ra, voff, 0u); x[i] = BufIo<float>::load(rx, voff, 0u);
          }
        }
        fa[0] = a[0]; fa[1] = x[0]; fa[2] = a[1]; fa[3] = x[1];
      } else {
        typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
        bf16x4 a, x;
        if constexpr (VEC) {
          const unsigned voff = o < p.bw ? off : kOutOfRange;     // bw is a multiple of 8 on the vector path
          a = __builtin_bit_cast(bf16x4, __builtin_amdgcn_raw_buffer_load_b64(ra, voff, 0, 0));
          x = __builtin_bit_cast(bf16x4, __builtin_amdgcn_raw_buffer_load_b64(rx, voff, 0, 0));
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const unsigned voff = o + i < p.bw ? off + 2u * i : kOutOfRange;
            a[i] = (__bf16)BufIo<__bf16>::load(ra, voff, 0u); x[i] = (__bf16)BufIo<__bf16>::load(rx, voff, 0u);
          }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) { fa[2 * i] = a[i]; fa[2 * i + 1] = x[i]; }
      }
#pragma unroll
      for (int jj = 0; jj < kGemmJG; ++jj) {
        if (jt0 + jj < JT) {                                   // wave-uniform
          const int j = (jt0 + jj) * 32 + r;                   // a padded row of the image is all zeros
          const Frag fb = *reinterpret_cast<const Frag*>(w2 + (long long)j * (2 * p.bwp) + kg * KG + hf * HW);
          Tr::mma(acc[jj], fa, fb);
        }
      }
    }
#pragma unroll
    for (int jj = 0; jj < kGemmJG; ++jj) {
      const int j = (jt0 + jj) * 32 + r;
      const bool col_ok = jt0 + jj < JT && j < p.bw;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int m = 8 * (v >> 2) + 4 * hf + (v & 3);
        BufIo<IO>::store((IO)acc[jj][v], rdx, col_ok ? (unsigned)m * row_bytes + col0 + (unsigned)j * ES : kOutOfRange, 0u);
      }
    }
  }
}

// dW partials.  grid = (token splits, gate blocks, tile groups); a workgroup's four waves own four consecutive
// 32-row tiles of output channels o and share kGemmJG 32-column tiles of input channels j, both gates.
template <typename IO>
__global__ __launch_bounds__(kThreads) void gate_dw_gemm_kernel(GateGemmArgs p) {
  typedef Io<IO> Tr;
  typedef typename Tr::Frag Frag;
  constexpr int KG = Tr::KG, HW = Tr::HW, ES = (int)sizeof(IO);
  const int lane = threadIdx.x & 63, r = lane & 31, hf = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int k = blockIdx.y, split = blockIdx.x;
  const int T32 = p.bwp / 32;
  const int jgroups = (T32 + kGemmJG - 1) / kGemmJG;
  const int og = blockIdx.z / jgroups, jt0 = (blockIdx.z - og * jgroups) * kGemmJG;
  const int ot = og * kWaves + wave;
  if (ot >= T32) return;
  const long long n_begin = (long long)split * p.tokens_per_split;
  const long long n_end = (n_begin + p.tokens_per_split) < p.N ? (n_begin + p.tokens_per_split) : p.N;
  const unsigned row_bytes = (unsigned)p.W * ES;
  const unsigned du_row_bytes = (unsigned)p.du_ld * ES;
  const int o = ot * 32 + r;
  const unsigned a_col = o < p.bw ? (unsigned)o * ES : kOutOfRange;
  unsigned b_col[kGemmJG];
#pragma unroll
  for (int jj = 0; jj < kGemmJG; ++jj) {
    const int j = (jt0 + jj) * 32 + r;
    b_col[jj] = (jt0 + jj < T32 && j < p.bw) ? (unsigned)(k * p.bw + j) * ES : kOutOfRange;
  }
  f32x16 acc[2][kGemmJG];
#pragma unroll
  for (int g = 0; g < 2; ++g)
#pragma unroll
    for (int jj = 0; jj < kGemmJG; ++jj)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[g][jj][v] = 0.f;

  for (long long nk = n_begin; nk < n_end; nk += KG) {
    const int rows = (int)((n_end - nk) < KG ? (n_end - nk) : KG);
    const rsrc_t ra = make_rsrc((const IO*)p.du_a + (long long)k * p.du_blk + nk * p.du_ld, (unsigned)rows * du_row_bytes);
    const rsrc_t rx = make_rsrc((const IO*)p.du_x + (long long)k * p.du_blk + nk * p.du_ld, (unsigned)rows * du_row_bytes);
    const rsrc_t rb = make_rsrc((const IO*)p.x + nk * p.W, (unsigned)rows * row_bytes);
    Frag fa, fx, fb[kGemmJG];
#pragma unroll
    for (int i = 0; i < HW; ++i) {
      const unsigned tok = (unsigned)(hf * HW + i);            // a token past the end lies past the extent
      const unsigned off = a_col == kOutOfRange ? kOutOfRange : tok * du_row_bytes + a_col;
      fa[i] = (IO)BufIo<IO>::load(ra, off, 0u);
      fx[i] = (IO)BufIo<IO>::load(rx, off, 0u);
#pragma unroll
      for (int jj = 0; jj < kGemmJG; ++jj)
        fb[jj][i] = (IO)BufIo<IO>::load(rb, b_col[jj] == kOutOfRange ? kOutOfRange : tok * row_bytes + b_col[jj], 0u);
    }
#pragma unroll
    for (int jj = 0; jj < kGemmJG; ++jj) {
      if (jt0 + jj < T32) {                                    // wave-uniform
        Tr::mma(acc[0][jj], fa, fb[jj]);
        Tr::mma(acc[1][jj], fx, fb[jj]);
      }
    }
  }
  // partial set of this split: [split][k][gate][o][j], padded width; rows and columns of the padding are zero
  float* part = p.dw_partial + ((long long)split * p.nb + k) * 2 * p.bwp * p.bwp;
#pragma unroll
  for (int g = 0; g < 2; ++g)
#pragma unroll
    for (int jj = 0; jj < kGemmJG; ++jj) {
      if (jt0 + jj < T32) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int m = 8 * (v >> 2) + 4 * hf + (v & 3);
          part[((long long)g * p.bwp + ot * 32 + m) * p.bwp + (jt0 + jj) * 32 + r] = acc[g][jj][v];
        }
      }
    }
}

// Gate pre-activations without the bias for the bf16 block widths whose scan kernels take them as an operand
// (multiples of 32 with no register-held variant): pre[k][n][g bw + o] = sum_j x[n, k bw + j] W_g[k][o][j].
// A wave owns 32 tokens and walks the 2 bw / 32 output tiles kGemmJG at a time; both operands are 16 contiguous
// bytes per lane (x rows; rows of the image's [gate][k][o][j] copy).
__global__ __launch_bounds__(kThreads) void gate_pre_gemm_kernel(GateGemmArgs p) {
  typedef Io<__bf16> Tr;
  typedef Tr::Frag Frag;
  constexpr int KG = Tr::KG, HW = Tr::HW;
  const int lane = threadIdx.x & 63, r = lane & 31, hf = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int k = blockIdx.y;
  const long long n0 = ((long long)blockIdx.x * kWaves + wave) * 32;
  if (n0 >= p.N) return;
  const int rows = (int)((p.N - n0) < 32 ? (p.N - n0) : 32);
  const unsigned row_bytes = (unsigned)p.W * 2u, out_row_bytes = 4u * (unsigned)p.bw;
  const rsrc_t rx = make_rsrc((const __bf16*)p.x + n0 * p.W, (unsigned)rows * row_bytes);
  const rsrc_t rp = make_rsrc((__bf16*)p.pre + ((long long)k * p.N + n0) * (2 * p.bw), (unsigned)rows * out_row_bytes);
  const __bf16* wg = (const __bf16*)p.wg;
  const int T32 = p.bw / 32, OT = 2 * T32, NKG = p.bw / KG;
  for (int ot0 = 0; ot0 < OT; ot0 += kGemmJG) {
    f32x16 acc[kGemmJG];
#pragma unroll
    for (int jj = 0; jj < kGemmJG; ++jj)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[jj][v] = 0.f;
    for (int kg = 0; kg < NKG; ++kg) {
      const Frag fa = buf_load_frag<Frag>(rx, (unsigned)r * row_bytes + (unsigned)(k * p.bw + kg * KG + hf * HW) * 2u);
#pragma unroll
      for (int jj = 0; jj < kGemmJG; ++jj) {
        const int ot = ot0 + jj;
        if (ot < OT) {                                         // wave-uniform
          const int g = ot / T32, o = (ot - g * T32) * 32 + r;
          const Frag fb = *reinterpret_cast<const Frag*>(wg + ((long long)(g * p.nb + k) * p.bwp + o) * p.bwp + kg * KG + hf * HW);
          Tr::mma(acc[jj], fa, fb);
        }
      }
    }
#pragma unroll
    for (int jj = 0; jj < kGemmJG; ++jj) {
      const int ot = ot0 + jj;
      if (ot < OT) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int m = 8 * (v >> 2) + 4 * hf + (v & 3);
          BufIo<__bf16>::store((__bf16)acc[jj][v], rp, (unsigned)m * out_row_bytes + (unsigned)(ot * 32 + r) * 2u, 0u);
        }
      }
    }
  }
}

// Partial sets of the weight-gradient GEMM for B * T = N tokens: enough splits of the token axis to give every
// compute unit of a 256-unit part a workgroup, at least 64 tokens per split, at most kGemmWgPerUnit sets.
int gate_dw_splits(long long N, const Geometry& g) {
  const long long T32 = g.bwp / 32;
  const long long per_block = ((T32 + kWaves - 1) / kWaves) * ((T32 + kGemmJG - 1) / kGemmJG);
  long long s = 256 / (g.nb * per_block);
  const long long by_tokens = (N + 63) / 64;
  if (s > by_tokens) s = by_tokens;
  if (s > kGemmWgPerUnit) s = kGemmWgPerUnit;
  if (s < 1) s = 1;
  return (int)s;
}

int launch_gate_pre_gemm(const void* x, const void* wg, void* pre, long long N, const Geometry& g, hipStream_t s) {
  GateGemmArgs a;
  memset(&a, 0, sizeof(a));
  a.x = x; a.wg = wg; a.pre = pre;
  a.N = N; a.W = (int)g.W; a.nb = (int)g.nb; a.bw = (int)g.bw; a.bwp = (int)g.bwp;
  const dim3 grid((unsigned)((N + 32 * kWaves - 1) / (32 * kWaves)), (unsigned)g.nb);
  hipLaunchKernelGGL(gate_pre_gemm_kernel, grid, dim3(kThreads), 0, s, a);
  return check_launch("gate pre-activation GEMM");
}

int launch_gate_gemms(const void* x, const void* du_a, const void* du_x, long long du_ld, long long du_blk,
                      const void* w2t, void* dx, float* dw_partial, long long N, const Geometry& g, int dtype,
                      int n_split, hipStream_t s) {
  GateGemmArgs a;
  memset(&a, 0, sizeof(a));
  a.x = x; a.du_a = du_a; a.du_x = du_x; a.w2t = w2t; a.dx = dx; a.dw_partial = dw_partial;
  a.du_ld = du_ld; a.du_blk = du_blk;
  a.N = N; a.W = (int)g.W; a.nb = (int)g.nb; a.bw = (int)g.bw; a.bwp = (int)g.bwp;
  const int es = dtype == RGLRU_BF16 ? 2 : 4;
  const int kgroup = dtype == RGLRU_BF16 ? 16 : 8;
  long long per = (N + n_split - 1) / n_split;
  per = (per + kgroup - 1) / kgroup * kgroup;
  a.tokens_per_split = per;
  // vector loads: every row and every block start on an 8-byte boundary and a du pair never straddles the block's end
  const bool vec = ((uintptr_t)du_a % 8 == 0) && ((uintptr_t)du_x % 8 == 0) && ((du_ld * es) % 8 == 0) &&
                   ((du_blk * es) % 8 == 0) && ((g.bw * es) % 8 == 0);
  const dim3 grid_dx((unsigned)((N + 32 * kWaves - 1) / (32 * kWaves)), (unsigned)g.nb);
  if (dtype == RGLRU_BF16) {
    if (vec) hipLaunchKernelGGL((gate_dx_gemm_kernel<__bf16, true>), grid_dx, dim3(kThreads), 0, s, a);
    else hipLaunchKernelGGL((gate_dx_gemm_kernel<__bf16, false>), grid_dx, dim3(kThreads), 0, s, a);
  } else {
    if (vec) hipLaunchKernelGGL((gate_dx_gemm_kernel<float, true>), grid_dx, dim3(kThreads), 0, s, a);
    else hipLaunchKernelGGL((gate_dx_gemm_kernel<float, false>), grid_dx, dim3(kThreads), 0, s, a);
  }
  int rc = check_launch("gate gradients: input gradient GEMM");
  if (rc) return rc;
  const long long T32 = g.bwp / 32;
  const unsigned groups = (unsigned)(((T32 + kWaves - 1) / kWaves) * ((T32 + kGemmJG - 1) / kGemmJG));
  const dim3 grid_dw((unsigned)n_split, (unsigned)g.nb, groups);
  if (dtype == RGLRU_BF16) hipLaunchKernelGGL(gate_dw_gemm_kernel<__bf16>, grid_dw, dim3(kThreads), 0, s, a);
  else hipLaunchKernelGGL(gate_dw_gemm_kernel<float>, grid_dw, dim3(kThreads), 0, s, a);
  return check_launch("gate gradients: weight gradient GEMM");
}

}  // namespace rglru
