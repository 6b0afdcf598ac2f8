// Byte layouts of the two opaque buffers of the C ABI, computed identically on host and device.
#pragma once

#include <stddef.h>
#include <stdint.h>

namespace rglru {

inline int64_t round_up(int64_t v, int64_t m) { return (v + m - 1) / m * m; }

// Geometry derived from (W, nb): block width, padded block width, 32-channel slabs.
struct Geometry {
  int64_t W, nb, bw, bwp, S, Wp;      // Wp = nb * bwp padded channels; S slabs per block
  int64_t groups;                      // workgroups needed to cover one block (4 slabs each)
  int64_t units;                       // nb * groups: independent weight sets
};

inline Geometry make_geometry(int64_t W, int64_t nb) {
  Geometry g;
  g.W = W; g.nb = nb; g.bw = W / nb;
  g.bwp = round_up(g.bw, 32);
  g.S = g.bwp / 32;
  g.Wp = nb * g.bwp;
  g.groups = (g.S + 3) / 4;
  g.units = nb * g.groups;
  return g;
}

// Prepared parameter image.
//   wg    [2][nb][bwp][bwp]  storage type, zero padded: gate weights, row = output channel
//   bias  [2][Wp]            fp32
//   sp    [Wp]               fp32   c * log2(sigmoid(Lambda))
//   cs    [Wp]               fp32   c * log(sigmoid(Lambda))
//   dsp   [Wp]               fp32   c * sigmoid(-Lambda), the factor of the Lambda gradient
//   w2t   [nb][bwp][2*bwp]   storage type: w2t[k][j][2*o + gate] = W_gate[k][o][j], the operand
//                            of the input-gradient GEMM dx += du W
struct PrepLayout {
  size_t wg, bias, sp, cs, dsp, w2t, total;
};

inline PrepLayout make_prep_layout(const Geometry& g, size_t elem) {
  PrepLayout p;
  size_t off = 0;
  p.wg = off;   off += (size_t)round_up(2 * g.nb * g.bwp * g.bwp * (int64_t)elem, 256);
  p.bias = off; off += (size_t)round_up(2 * g.Wp * 4, 256);
  p.sp = off;   off += (size_t)round_up(g.Wp * 4, 256);
  p.cs = off;   off += (size_t)round_up(g.Wp * 4, 256);
  p.dsp = off;  off += (size_t)round_up(g.Wp * 4, 256);
  p.w2t = off;  off += (size_t)round_up(2 * g.nb * g.bwp * g.bwp * (int64_t)elem, 256);
  p.total = off;
  return p;
}

// Workspace of one forward/backward pair: what has to survive from forward to backward, plus the
// carry records of both passes.  nC = chunks of 32 tokens (rounded up to even), nCf = forward tiles
// of 64 tokens.
//   ckpt        [B][2 nC][W]    fp32 state after every 16 tokens (kept for backward: each lane of the
//                               backward scan owns 16 consecutive tokens and starts from one of these)
//   --- [f_begin, f_end) is cleared at the start of a forward pass that uses records (the kernels with one
//       workgroup per chain use none and clear the failure word only) ---
//   f_rec_a     [B][<=nC][W]    64-bit carry records of the forward chain
//   f_ticket    [units][kMaxQueues]
//   fail        [1]             failure word (either pass sets it; only forward clears it)
//   --- [b_begin, b_end): cleared at the start of every backward pass that uses records ---
//   b_rec_a     [B][nC][W]      64-bit carry records of the backward chain
//   b_ticket    [units][kMaxQueues]
constexpr int kMaxQueues = 64;          // ticket queues per unit (sequences are dealt round-robin to them)
constexpr int kGemmWgPerUnit = 32;      // workgroups per unit in the gradient kernel of the fast backward
constexpr int kWideWgPerUnit = 8;       // ... and in the gate-gradient kernel of blocks wider than 128 channels

struct WorkLayout {
  int64_t nC, nCf, max_wg;
  size_t ckpt;
  size_t f_begin, f_rec_a, f_ticket, f_end;
  size_t b_begin, b_rec_a, b_ticket, fail, b_end, total;
};

inline WorkLayout make_work_layout(int64_t B, int64_t T, const Geometry& g) {
  WorkLayout w;
  w.nCf = (T + 63) / 64;
  w.nC = 2 * w.nCf;
  w.max_wg = 256;                      // most workgroups one unit may use in backward
  size_t off = 0;
  auto take = [&](int64_t bytes) { size_t at = off; off += (size_t)round_up(bytes, 256); return at; };
  w.ckpt = take(B * 2 * w.nC * g.W * 4);
  w.f_begin = off;
  w.f_rec_a = take(B * w.nC * g.W * 8);
  w.f_ticket = take(g.units * kMaxQueues * 4);
  w.fail = take(4);
  w.f_end = off;
  w.b_begin = off;
  w.b_rec_a = take(B * w.nC * g.W * 8);
  w.b_ticket = take(g.units * kMaxQueues * 4);
  w.b_end = off;
  w.total = off;
  return w;
}

// Splits of the token axis (= partial sets) of the weight-gradient GEMM of the paths without a fused one
// (rglru_gate_gemm.hip).
int gate_dw_splits(long long N, const Geometry& g);

// Scratch of one backward call; nothing in it outlives the call, its contents on entry do not matter.
//   partial     [maxWg][3][Wp]  per-workgroup sums for db_a, db_x, dLambda
//   delta       fast backward (blocks of 32, 64, 128 channels): [B][T][W] 16-bit, dL/dh_t after the
//               reverse scan; wide backward (blocks of 160 .. 384 channels): [B][T][nb][2 bw] 16-bit,
//               the gradients at the gate pre-activations as pairs (element 2 o + gate)
//   dw_partial  [sets][nb][2][bwp][bwp] per-workgroup weight-gradient sums, sets = kGemmWgPerUnit (fast),
//               kWideWgPerUnit (wide) or gate_dw_splits (the other paths); fp32, or bf16 in the fast backward
//               when 16-bit gradients are asked for (sized for fp32 either way)
enum ScratchKind { kScratchPlain = 0, kScratchFast = 1, kScratchWide = 2 };
struct ScratchLayout {
  size_t partial, delta, dw_partial, total;
};

inline ScratchLayout make_scratch_layout(int64_t B, int64_t T, const Geometry& g, int kind) {
  ScratchLayout s;
  size_t off = 0;
  auto take = [&](int64_t bytes) { size_t at = off; off += (size_t)round_up(bytes, 256); return at; };
  s.partial = take((int64_t)256 * 3 * g.Wp * 4);
  s.delta = take(kind == kScratchFast ? B * T * g.W * 2 : kind == kScratchWide ? B * T * g.W * 4 : 0);
  const int64_t sets = kind == kScratchFast ? kGemmWgPerUnit : kind == kScratchWide ? kWideWgPerUnit : gate_dw_splits(B * T, g);
  s.dw_partial = take(sets * g.nb * g.bwp * 2 * g.bwp * 4);
  s.total = off;
  return s;
}

// Scan-only workspace of one forward / backward pair: two regions of the same layout, the forward pass uses
// the first and the backward pass the second.  Tickets and the failure word come first in a region, so that a
// clearing launch covers them and only as many records as the kernel variant needs (one per sequence, channel
// and 32-token chunk, or one per 128-token run of the vector kernels).  The forward call clears the used part
// of BOTH regions in its one clearing launch; a backward call clears its region itself unless told that the
// workspace is fresh from its forward call.  The failure word of the pair is the first region's.
//   ticket [B][groups]; fail; rec_a [B][nC][W] 64-bit carry records.
struct ScanLayout {
  int64_t nC, groups;
  size_t ticket, fail, rec_a, region, total;
};

inline ScanLayout make_scan_layout(int64_t B, int64_t T, int64_t W) {
  ScanLayout s;
  s.nC = (T + 31) / 32;
  s.groups = (W + 63) / 64;
  size_t off = 0;
  auto take = [&](int64_t bytes) { size_t at = off; off += (size_t)round_up(bytes, 256); return at; };
  s.ticket = take(B * s.groups * 4);
  s.fail = take(4);
  s.rec_a = take(B * s.nC * W * 8);
  s.region = off;
  s.total = 2 * off;
  return s;
}

}  // namespace rglru
