/*
 * C ABI of the MI355X (gfx950) RG-LRU library, librglru_hip.so.
 *
 * This is the boundary a host binds instead of the reference's Triton operator and the
 * PyTorch gate chain that feeds it:
 *
 *   reference interface replaced                         entry point here
 *   ---------------------------------------------------  -------------------------------
 *   griffin/triton_scan.py:207-244  _FusedRGLRUScan.forward   rglru_hip_scan_fwd
 *   griffin/triton_scan.py:246-271  _FusedRGLRUScan.backward  rglru_hip_scan_bwd
 *   griffin/griffin.py:237-289      RG_LRU.forward (gates + scan, T > 1)   rglru_hip_prepare + rglru_hip_fwd
 *   autograd of griffin/griffin.py:237-289                                   rglru_hip_bwd_full (blocks of 32/64/128 channels),
 *                                                                            rglru_hip_bwd_wide (160 .. 384), rglru_hip_bwd (any)
 *   the same for bf16 blocks of 416 .. 512 channels (gate projections of griffin/griffin.py:149-154 as a GEMM kernel of their own)   rglru_hip_fwd_pre, rglru_hip_bwd_pre
 *   griffin/griffin.py:279-284 with T == 1 (decode step, carried state)     rglru_hip_step, rglru_hip_steps (K steps a launch)
 *   (no counterpart: forward for callers that cannot allocate)              rglru_hip_fwd_static
 *   griffin/griffin.py:474-487      causal depthwise convolution of the caller   rglru_hip_conv_fwd
 *   autograd of griffin/griffin.py:474-487                                   rglru_hip_conv_bwd
 *   griffin/griffin.py:488-510      the same over right-padded batches and its autograd   rglru_hip_conv_padded_fwd, _bwd
 *   griffin/griffin.py:464, :520    x_branch * gelu_tanh(linear_y(x))        rglru_hip_gelu_gate_fwd, _bwd
 *   griffin/griffin.py:464-520      convolution, RG-LRU and output gate in one launch   rglru_hip_block_fwd, rglru_hip_prepare_block_fwd
 *   griffin/griffin.py:68-80        RMSNorm in front of the block and its autograd   rglru_hip_rmsnorm_fwd, _bwd
 *   griffin/griffin.py:459-528 with T == 1 (block decode: positions, conv, step, gate)   rglru_hip_decode_prepare + rglru_hip_step_gated
 *   autograd of the bias of griffin/griffin.py:379-389 (the block's Linear layers)      rglru_hip_colsum
 *   the sum that ends their weight gradient when its contraction is split             rglru_hip_sum_sets
 *
 * Conventions
 *   - every pointer is a DEVICE pointer owned by the caller; tensors are row-major with the
 *     width axis contiguous; nothing here allocates, frees or synchronises;
 *   - work is enqueued on `stream` (a hipStream_t passed as void*; NULL = the null stream);
 *   - every function returns 0 on success or a non-zero code (RGLRU_E_*); the text of the
 *     last failure on the calling thread is returned by rglru_hip_last_error();
 *   - the library keeps no per-call state: forward and backward may be issued from different
 *     host threads (PyTorch runs backward on its autograd thread);
 *   - `dtype` selects the storage type of x / y / dy / dx and of the gate weights:
 *     RGLRU_F32 or RGLRU_BF16.  The state is always fp32.  Biases and Lambda are read in
 *     `vec_dtype` and the parameter gradients written in `grad_dtype` (each RGLRU_F32 or
 *     RGLRU_BF16), so a caller never has to convert its parameters or their gradients; the
 *     arithmetic and the accumulation are fp32 either way.
 *   - `flags` is one byte per token, [B, T]: bit 0 = reset (griffin/griffin.py:248-249: a <- 0,
 *     g <- 1), bit 1 = inactive / padding (griffin/griffin.py:252-255: a <- 1, z <- 0).
 *     NULL means no reset and all tokens active.
 */
#ifndef RGLRU_HIP_H
#define RGLRU_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define RGLRU_ABI_VERSION 19

enum { RGLRU_F32 = 0, RGLRU_BF16 = 1 };

enum {
  RGLRU_OK = 0,
  RGLRU_E_ARG = 1,      /* bad shape / null pointer / unsupported dtype */
  RGLRU_E_UNSUPPORTED = 2, /* shape outside what the kernels cover (e.g. gate block wider than 512) */
  RGLRU_E_LAUNCH = 3    /* the HIP runtime refused a launch; see rglru_hip_last_error() */
};

#define RGLRU_FLAG_RESET 1u
#define RGLRU_FLAG_INACTIVE 2u
/* In place of a flag array (the forward and backward entry points of whole sequences, not the decode steps):
 * token 0 of every sequence carries RGLRU_FLAG_RESET and no other token any flag -- what the recurrent block
 * passes when every row holds one document from its beginning (griffin/griffin.py:309-338 without cache).  The
 * kernels then need no per-token flags; rglru_hip_block_fwd also takes the rows' convolution history as empty. */
#define RGLRU_FLAGS_FIRST_RESET ((const uint8_t*)(uintptr_t)1)
/* Bits 2-3 of a flag byte are read by rglru_hip_block_fwd only (convolution lags that reach in front of the
 * token's document); every other entry point ignores them. */
#define RGLRU_FLAG_CONV_SHIFT 2

/* Tokens per chunk of the backward scan (one carry record per sequence, chunk and channel).  Forward
 * stores the fp32 state after every RGLRU_CHUNK / 2 tokens and backward restarts its recomputation
 * from those checkpoints. */
#define RGLRU_CHUNK 32

int rglru_hip_abi_version(void);
const char* rglru_hip_last_error(void);

/* Largest gate-block width (W / nb) the fused kernels accept. */
int rglru_hip_max_block_width(void);

/* ---- scan-only contract: h_t = a_t * h_{t-1} + z_t, all fp32 ------------------------------
 * Replaces griffin/triton_scan.py:31-60 and :63-122.  a, z, h, dh, da, dz are [B, T, W];
 * h0, dh0 are [B, W].  `ws` is scratch of rglru_hip_scan_workspace_bytes(B, T, W) bytes with a part for each
 * pass; its contents on entry to a forward call do not matter, and a forward and a backward call may not
 * use it concurrently.  The forward call clears both parts in its one clearing launch, so a training step pays
 * for one such launch: pass ws_fresh != 0 to the FIRST backward call that is given the workspace of its forward
 * call; ws_fresh == 0 (any other workspace, or a repeated backward call) makes the backward call clear its part
 * itself.  Nothing but that is carried from forward to backward in `ws`. */
size_t rglru_hip_scan_workspace_bytes(int64_t B, int64_t T, int64_t W);
int rglru_hip_scan_fwd(const float* a, const float* z, const float* h0, float* h, void* ws,
                       int64_t B, int64_t T, int64_t W, void* stream);
int rglru_hip_scan_bwd(const float* a, const float* h0, const float* h, const float* dh,
                       float* da, float* dz, float* dh0, void* ws, int ws_fresh,
                       int64_t B, int64_t T, int64_t W, void* stream);

/* ---- fused RG-LRU ---------------------------------------------------------------------------
 * Parameters follow griffin/griffin.py:138-141, 174-176: w_a, w_x are [nb, bw, bw] (out, in) in
 * `dtype`; b_a, b_x are [nb, bw] and lambda is [W], in `vec_dtype`.  rglru_hip_prepare converts
 * them once into the padded, kernel-friendly image `prep` (rglru_hip_prep_bytes bytes) that fwd,
 * bwd and step consume (it also holds c * log sigmoid(Lambda) and c * sigmoid(-Lambda), so the
 * other entry points take neither c nor Lambda); it must be re-run after the parameters change. */
size_t rglru_hip_prep_bytes(int64_t W, int64_t nb, int dtype);
int rglru_hip_prepare(const void* w_a, const void* b_a, const void* w_x, const void* b_x,
                      const void* lambda, float c, int64_t W, int64_t nb, int dtype, int vec_dtype,
                      void* prep, void* stream);

/* Workspace shared by one forward call and its backward call(s).  Forward initialises it (chunk
 * checkpoints of the fp32 state, the failure word, its own carry records where the kernel uses any),
 * so its contents on entry to forward do not matter; a backward call must be given the workspace of its
 * forward call, reads the checkpoints, clears and uses its own part as scratch, and any number of backward
 * calls may follow one forward call. */
size_t rglru_hip_workspace_bytes(int64_t B, int64_t T, int64_t W, int64_t nb);

/* Scratch of one backward call (per-workgroup partial sums; for the fast configurations also the
 * gate pre-activation gradients between the two backward kernels).  Nothing in it outlives the
 * call, so it is allocated when backward runs instead of being held since forward; its contents on
 * entry do not matter.  The size depends on which backward entry point the configuration takes. */
size_t rglru_hip_bwd_scratch_bytes(int64_t B, int64_t T, int64_t W, int64_t nb, int dtype);

/* y[B,T,W] (dtype) and h_last[B,W] (fp32, may be NULL) from x[B,T,W], h0[B,W] (fp32, NULL = 0). */
int rglru_hip_fwd(const void* x, const void* prep, const float* h0, const uint8_t* flags,
                  void* y, float* h_last, void* ws,
                  int64_t B, int64_t T, int64_t W, int64_t nb, int dtype, void* stream);

/* rglru_hip_fwd without a workspace argument and without any allocation.  It has no counterpart in
 * the reference: it exists for callers that cannot allocate device memory around the call -- code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc -- and want the
 * forward pass (inference: prefill of a prompt, T > 1) only.  The workspace is a device array built
 * into the library, RGLRU_STATIC_WORKSPACE_BYTES per GPU, held until the process ends; shapes whose
 * rglru_hip_workspace_bytes() exceed it are rejected with RGLRU_E_UNSUPPORTED.  All calls on one GPU
 * share that array: calls that overlap in time on one GPU (different streams, different threads)
 * race and give wrong results; calls on one stream are safe.  Nothing of a call survives in it, so
 * there is no backward pass for this entry point.  Same results as rglru_hip_fwd. */
#define RGLRU_STATIC_WORKSPACE_BYTES (16u << 20)
size_t rglru_hip_static_workspace_bytes(void);
int rglru_hip_fwd_static(const void* x, const void* prep, const float* h0, const uint8_t* flags,
                         void* y, float* h_last,
                         int64_t B, int64_t T, int64_t W, int64_t nb, int dtype, void* stream);

/* rglru_hip_prepare followed by rglru_hip_fwd on the same stream with fewer launches: the
 * parameter conversion and the clearing of the workspace share a kernel, and where the forward runs
 * one workgroup per chain (see rglru_hip_set_chain_forward) that kernel is the forward kernel itself,
 * one launch in all.  For training, where every forward (griffin/griffin.py:237-289) sees freshly
 * updated parameters; `prep` is written and stays valid for the matching backward call. */
int rglru_hip_prepare_fwd(const void* w_a, const void* b_a, const void* w_x, const void* b_x,
                          const void* lambda, float c, int vec_dtype, void* prep,
                          const void* x, const float* h0, const uint8_t* flags,
                          void* y, float* h_last, void* ws,
                          int64_t B, int64_t T, int64_t W, int64_t nb, int dtype, void* stream);

/* Backward of rglru_hip_fwd for any configuration (fp32 storage, block widths that are no multiple of 32,
 * unaligned tensors).  Recomputes the gates and the decay from x (nothing but the chunk checkpoints in `ws`
 * is kept from forward).  dy[B,T,W] (dtype); dh_last[B,W] fp32 or NULL.  Outputs, all complete: dx[B,T,W]
 * (dtype), dw_a, dw_x [nb,bw,bw], db_a, db_x [nb*bw] and dlambda [W] (grad_dtype), dh0 [B,W] (fp32, may be
 * NULL).  du_a, du_x [B,T,W] (dtype) are scratch of the call: the scan kernel leaves the gradients at the two
 * gate pre-activations there, and two GEMM kernels of this library (matrix unit; griffin/griffin.py:149-154
 * under autograd) form dW = du^T x and dx += du W from them. */
int rglru_hip_bwd(const void* x, const void* prep, const float* h0,
                  const uint8_t* flags, const void* dy, const float* dh_last, void* ws, void* scratch,
                  void* dx, void* du_a, void* du_x, void* dw_a, void* dw_x, void* db_a, void* db_x, void* dlambda,
                  float* dh0, int64_t B, int64_t T, int64_t W, int64_t nb, int dtype, int grad_dtype,
                  void* stream);

/* Complete backward for the fast configurations (rglru_hip_fast_path(W, nb, dtype) != 0: 16-bit
 * storage, gate blocks of 32, 64 or 128 channels, 16-byte aligned tensors).  Same inputs as
 * rglru_hip_bwd plus y[B,T,W], the output of the forward call as it was stored (the state in front of
 * token t is read from row t - 1 of it; the checkpoints in `ws` are not used).  dx[B,T,W] is the full
 * input gradient and dw_a, dw_x [nb,bw,bw] (grad_dtype) the weight gradients.  Two hand-written
 * kernels: the reverse scan for dL/dh_t, which recomputes only the decay, then one kernel that
 * recomputes both gates and forms every gradient including the two block-diagonal GEMMs, so the
 * gradients at the gate pre-activations never reach memory.  Returns RGLRU_E_UNSUPPORTED for other
 * configurations. */
int rglru_hip_fast_path(int64_t W, int64_t nb, int dtype);
int rglru_hip_bwd_full(const void* x, const void* y, const void* prep, const float* h0,
                       const uint8_t* flags, const void* dy, const float* dh_last, void* ws, void* scratch,
                       void* dx, void* dw_a, void* dw_x, void* db_a, void* db_x, void* dlambda,
                       float* dh0, int64_t B, int64_t T, int64_t W, int64_t nb, int dtype, int grad_dtype,
                       void* stream);

/* Complete backward for gate blocks of 160 to 384 channels in steps of 32 (rglru_hip_wide_path(W, nb,
 * dtype) != 0: 16-bit storage; griffin/griffin.py:149-154 at those widths and its autograd).  For these
 * widths rglru_hip_fwd and rglru_hip_prepare_fwd hold a block's weights in the registers of several
 * workgroups (four 32-channel slabs each), and this entry point is the matching backward: same inputs
 * and outputs as rglru_hip_bwd_full without y (the states come from the checkpoints in `ws`).  Two
 * hand-written kernels: reverse scan and gate math (direct part of dx, the gradients at the gate
 * pre-activations as 16-bit pairs in `scratch`), then the two block-diagonal GEMMs on the matrix unit
 * (dx += du W and dW = du^T x).  Returns RGLRU_E_UNSUPPORTED for other configurations. */
int rglru_hip_wide_path(int64_t W, int64_t nb, int dtype);
int rglru_hip_bwd_wide(const void* x, const void* prep, const float* h0,
                       const uint8_t* flags, const void* dy, const float* dh_last, void* ws, void* scratch,
                       void* dx, void* dw_a, void* dw_x, void* db_a, void* db_x, void* dlambda,
                       float* dh0, int64_t B, int64_t T, int64_t W, int64_t nb, int dtype, int grad_dtype,
                       void* stream);

/* Variant for the block widths that neither rglru_hip_fast_path nor rglru_hip_wide_path covers (any
 * multiple of 32 channels up to 512, i.e. 416, 448, 480 or 512; bf16 storage, 16-byte aligned tensors;
 * rglru_hip_pre_path() says whether a configuration qualifies).  The two block-diagonal projections of
 * griffin/griffin.py:149-154 run as a GEMM kernel of their own in front of the scan kernel, which takes
 * their result as an operand.  `pre` and `du` are scratch of the call, [nb][B*T][2*bw] (dtype) each:
 *   pre[k][n][o] = sum_j W_a[k][o][j] x[n][k*bw+j],  pre[k][n][bw+o] = the same with W_x  (biases not added)
 *   du: the gradients at the pre-activations in the same two halves.
 * rglru_hip_fwd_pre is rglru_hip_fwd with that scratch operand.  rglru_hip_bwd_pre recomputes `pre`, runs
 * the reverse scan and the gate math, and finishes with the two gate-gradient GEMM kernels:
 *   dx[n][k*bw+j] += sum_o du[k][n][o] W_a[k][o][j] + du[k][n][bw+o] W_x[k][o][j]
 *   dW_a[k][o][j] = sum_n du[k][n][o] x[n][k*bw+j],  dW_x likewise from the second half.
 * Outputs as rglru_hip_bwd_full.  `prep`, `ws` and `scratch` (rglru_hip_bwd_scratch_bytes) are those of
 * rglru_hip_fwd / rglru_hip_bwd. */
int rglru_hip_pre_path(int64_t W, int64_t nb, int dtype);
int rglru_hip_fwd_pre(const void* x, void* pre, const void* prep, const float* h0, const uint8_t* flags,
                      void* y, float* h_last, void* ws,
                      int64_t B, int64_t T, int64_t W, int64_t nb, int dtype, void* stream);
int rglru_hip_bwd_pre(const void* x, void* pre, const void* prep, const float* h0,
                      const uint8_t* flags, const void* dy, const float* dh_last, void* ws, void* scratch,
                      void* dx, void* du, void* dw_a, void* dw_x, void* db_a, void* db_x, void* dlambda, float* dh0,
                      int64_t B, int64_t T, int64_t W, int64_t nb, int dtype, int grad_dtype, void* stream);

/* Which backward entry point (and kernel family) covers a configuration: what a host wrapper dispatches on,
 * and what a test asserts.  `aligned`: every activation tensor of the call (x, y, dy, dx) is 16-byte aligned.
 * Returns one of RGLRU_PATH_*, or -1 for a geometry the library rejects.
 *   RGLRU_PATH_FAST_CHAIN  rglru_hip_bwd_full, reverse scan with one workgroup per chain (and the forward likewise)
 *   RGLRU_PATH_FAST_TILED  rglru_hip_bwd_full, reverse scan in tiles with a look-back between workgroups
 *   RGLRU_PATH_WIDE        rglru_hip_bwd_wide
 *   RGLRU_PATH_PRE         rglru_hip_fwd_pre / rglru_hip_bwd_pre
 *   RGLRU_PATH_PORTABLE    rglru_hip_bwd
 * (the choice between chain and tiles also follows rglru_hip_set_chain_forward). */
enum { RGLRU_PATH_PORTABLE = 0, RGLRU_PATH_FAST_TILED = 1, RGLRU_PATH_FAST_CHAIN = 2, RGLRU_PATH_WIDE = 3, RGLRU_PATH_PRE = 4 };
int rglru_hip_backward_path(int64_t B, int64_t T, int64_t W, int64_t nb, int dtype, int aligned);

/* One decode step (T == 1): h[B,W] fp32 is updated in place, y[B,W] (dtype) = h as stored. */
int rglru_hip_step(const void* x, const void* prep, float* h, const uint8_t* flags, void* y,
                   int64_t B, int64_t W, int64_t nb, int dtype, void* stream);

/* K consecutive decode steps in one launch, for inputs that are known in advance (scoring a given
 * continuation, speculative verification, replaying a prefix token by token): x[K,B,W] and y[K,B,W]
 * (dtype), flags[K,B] or NULL, h[B,W] fp32 updated in place to the state after the last step.  The
 * same arithmetic as K calls of rglru_hip_step (griffin/griffin.py:279-284 with T == 1, K times), with
 * the state in registers and the weights loaded once. */
int rglru_hip_steps(const void* x, const void* prep, float* h, const uint8_t* flags, void* y,
                    int64_t K, int64_t B, int64_t W, int64_t nb, int dtype, void* stream);

/* Causal depthwise temporal convolution that feeds the RG-LRU inside the recurrent block, all
 * tokens active (griffin/griffin.py:474-487):
 *   out[b,t,c] = bias[c] + sum_{lag<K} taps[c][K-1-lag] * [segment_pos[b,t] >= lag] * padded[b,t-lag,c]
 * with padded = state[B,K-1,W] (NULL: zeros) followed by u[B,T,W].  taps[W,K] is the weight of a
 * depthwise nn.Conv1d viewed as [W][K] (tap K-1 multiplies the current token), bias[W] may be NULL;
 * both are read in vec_dtype.  u, state, out and new_state are `dtype`; segment_pos[B,T] is int64.
 * new_state[B,K-1,W] (may be NULL) receives the last K-1 rows of padded (griffin/griffin.py:487).
 * K = 1 .. rglru_hip_conv_max_kernel_size(); arithmetic in fp32. */
int rglru_hip_conv_max_kernel_size(void);
int rglru_hip_conv_fwd(const void* u, const void* state, const void* taps, const void* bias,
                       const int64_t* segment_pos, void* out, void* new_state,
                       int64_t B, int64_t T, int64_t W, int64_t K, int dtype, int vec_dtype, void* stream);

/* Reverse mode of rglru_hip_conv_fwd.  dout[B,T,W] (dtype) is the gradient at `out`.  Writes
 * du[B,T,W] and, when not NULL, dstate[B,K-1,W] (dtype), dtaps[W,K] and dbias[W] (grad_dtype).
 * du_stride is the distance between rows of du in elements (0 or W: contiguous; larger: du is a
 * column range of a wider [B*T, du_stride] matrix, e.g. the left half of the stacked gradient of
 * two projections that one GEMM then consumes).
 * `scratch` holds rglru_hip_conv_scratch_bytes(B, T, W, K) bytes of per-run partial sums; its
 * contents on entry do not matter. */
size_t rglru_hip_conv_scratch_bytes(int64_t B, int64_t T, int64_t W, int64_t K);
int rglru_hip_conv_bwd(const void* u, const void* state, const void* taps, const int64_t* segment_pos,
                       const void* dout, void* scratch, void* du, int64_t du_stride, void* dstate, void* dtaps, void* dbias,
                       int64_t B, int64_t T, int64_t W, int64_t K, int dtype, int vec_dtype, int grad_dtype,
                       void* stream);

/* The same convolution over right-padded batches (griffin/griffin.py:488-510): tokens with
 * active[b,t] == 0 produce zeros and never enter the window of the K-1 previous ACTIVE inputs; an
 * active token with segment_pos == 0 clears that window (and the carried state) before it is used.
 * active[B,T] is one byte per token; new_state[B,K-1,W] (may be NULL) receives the window after the
 * last token; `scratch` holds rglru_hip_conv_padded_scratch_bytes(B, T) bytes.
 * rglru_hip_conv_padded_bwd is its reverse mode (the reference gets it from autograd through a
 * per-token Python loop): dout[B,T,W] in; du[B,T,W] (zero at inactive tokens), dstate[B,K-1,W],
 * dtaps[W,K], dbias[W] out (the last three may be NULL).  `index_scratch` holds
 * rglru_hip_conv_padded_scratch_bytes(B, T) bytes and `scratch` rglru_hip_conv_scratch_bytes(B, T, W, K)
 * bytes; their contents on entry do not matter.  Both index buffers must be 8-byte aligned.
 * Rows whose active tokens are a prefix of the row (all rows of a right-padded batch) run at the speed of
 * rglru_hip_conv_fwd / _bwd; rows with holes take kernels that gather through an index. */
size_t rglru_hip_conv_padded_scratch_bytes(int64_t B, int64_t T);
int rglru_hip_conv_padded_fwd(const void* u, const void* state, const void* taps, const void* bias,
                              const int64_t* segment_pos, const uint8_t* active, void* scratch,
                              void* out, void* new_state,
                              int64_t B, int64_t T, int64_t W, int64_t K, int dtype, int vec_dtype, void* stream);
int rglru_hip_conv_padded_bwd(const void* u, const void* state, const void* taps,
                              const int64_t* segment_pos, const uint8_t* active, const void* dout,
                              void* index_scratch, void* scratch, void* du, void* dstate, void* dtaps, void* dbias,
                              int64_t B, int64_t T, int64_t W, int64_t K, int dtype, int vec_dtype, int grad_dtype,
                              void* stream);

/* Output gate of the recurrent block, out = h * gelu_tanh(v) (griffin/griffin.py:464 and :520: the
 * GeLU of the second branch and the product with the RG-LRU output in one pass), flat over n
 * elements of `dtype`; and its reverse mode: dh = dout * gelu_tanh(v), dv = dout * h * gelu_tanh'(v).
 * The reverse mode can write dv as rows of W elements that lie dv_stride elements apart (n a multiple
 * of W; a column range of a wider matrix, as for du of rglru_hip_conv_bwd); dv_stride 0 or W: flat like
 * the other tensors, W is then not used.  Arithmetic in fp32. */
int rglru_hip_gelu_gate_fwd(const void* h, const void* v, void* out, int64_t n, int dtype, void* stream);
int rglru_hip_gelu_gate_bwd(const void* dout, const void* h, const void* v, void* dh, void* dv,
                            int64_t n, int64_t W, int64_t dv_stride, int dtype, void* stream);

/* RMSNorm in front of the block (griffin/griffin.py:68-80), over the last axis of x[rows, D]:
 *   y = x * rsqrt(mean(x^2) + eps) * (1 + g),   g[D] read in vec_dtype;
 * inv[rows] (fp32, may be NULL) receives rsqrt(mean(x^2) + eps) for the backward pass, which writes
 * dx[rows, D] (dtype) and, when not NULL, dg[D] (grad_dtype); `scratch` holds
 * rglru_hip_rmsnorm_scratch_bytes(rows, D) bytes.  D is at most rglru_hip_rmsnorm_max_width(dtype,
 * aligned) (aligned: 16-byte aligned tensors and rows).  Arithmetic in fp32. */
int rglru_hip_rmsnorm_max_width(int dtype, int aligned);
int rglru_hip_rmsnorm_fwd(const void* x, const void* g, void* y, float* inv, int64_t rows, int64_t D, float eps,
                          int dtype, int vec_dtype, void* stream);
size_t rglru_hip_rmsnorm_scratch_bytes(int64_t rows, int64_t D);
int rglru_hip_rmsnorm_bwd(const void* x, const void* g, const float* inv, const void* dy, void* scratch,
                          void* dx, void* dg, int64_t rows, int64_t D, int dtype, int vec_dtype, int grad_dtype,
                          void* stream);

/* Column sums of x[rows, D] (dtype) into out[D] (out_dtype), fp32 accumulation in a fixed order: the
 * bias gradient of the block's three Linear layers (griffin/griffin.py:379-389; autograd of
 * `nn.Linear`: db = sum over tokens of dy), which the caller's BLAS library leaves to a generic reduction.
 * `scratch` holds rglru_hip_colsum_scratch_bytes(rows, D) bytes. */
size_t rglru_hip_colsum_scratch_bytes(int64_t rows, int64_t D);
int rglru_hip_colsum(const void* x, void* scratch, void* out, int64_t rows, int64_t D, int dtype, int out_dtype,
                     void* stream);

/* out[i] = sum over s < sets of x[s * n + i] (both `dtype`, fp32 accumulation in the order of the sets): the last
 * step of the weight gradient of the block's Linear layers (griffin/griffin.py:379-389; autograd of `nn.Linear`:
 * dW = dy^T x) where the caller splits the contraction over all tokens into a batch of shorter GEMMs of its BLAS
 * library and has their results added. */
int rglru_hip_sum_sets(const void* x, void* out, int64_t sets, int64_t n, int dtype, void* stream);

/* Single-token step of the recurrent block (griffin/griffin.py:459-528 with one token per row) in
 * two launches around the caller's three Linear layers:
 *   rglru_hip_decode_prepare: per row, the position (prev_pos + 1, prev_pos NULL = -1, or
 *     segment_pos[B] when given), the flags for the step (reset at position 0, inactive), the
 *     convolved input x[B,W] = conv(u[B,W], conv_state[B,K-1,W] or NULL = zeros), the shifted state
 *     new_conv_state[B,K-1,W] (must not alias conv_state) and new_pos[B].  active[B] (one byte per
 *     row) NULL selects the all-active path (:476-487); otherwise the padded path (:488-510): a
 *     document start clears the history, an inactive row keeps state and position, x = 0 for it.
 *   rglru_hip_step_gated: rglru_hip_step with the state read from h_in and written to h_out (the two
 *     may be the same buffer) and out[B,W] = h * gelu_tanh(v[B,W]) (v NULL: out = h), which is the
 *     operand of the block's output projection (:520).
 * u and v may be rows of a wider buffer (the two halves of one GEMM that computes both projections):
 * u_stride and v_stride are the distances between their rows in elements, 0 meaning W. */
int rglru_hip_decode_prepare(const void* u, int64_t u_stride, const void* conv_state, const void* taps, const void* bias,
                             const int64_t* prev_pos, const int64_t* segment_pos, const uint8_t* active,
                             void* x, void* new_conv_state, int64_t* new_pos, uint8_t* flags,
                             int64_t B, int64_t W, int64_t K, int dtype, int vec_dtype, void* stream);
int rglru_hip_step_gated(const void* x, const void* prep, const float* h_in, float* h_out, const uint8_t* flags,
                         const void* v, int64_t v_stride, void* out, int64_t B, int64_t W, int64_t nb, int dtype,
                         void* stream);

/* The recurrent block's forward between its projections in ONE launch (griffin/griffin.py:474-487, the
 * RG-LRU of :97-286, and :464, :520): x = causal depthwise convolution of u[B,T,W] (taps[W][K], K <= 4,
 * conv_bias[W] or NULL, both in vec_dtype; conv_state[B,K-1,W] or NULL = zeros in front of every row),
 * y = RG-LRU(x) and gated[B,T,W] = y * gelu_tanh(v[B,T,W]).  u and v may be rows of wider buffers
 * (u_stride, v_stride in elements, 0 = W).  Every token is active; the flag bytes carry, next to
 * RGLRU_FLAG_RESET, in bits 2-3 how many convolution lags reach in front of the token's document,
 * 3 - min(segment_pos, 3) (rglru_hip_block_flags writes them from segment_pos[n]); flags NULL means no
 * document starts inside the rows and position >= K - 1 or an all-zero history at their beginning.
 * Optional outputs (NULL to skip): x_conv[B,T,W] and y[B,T,W] (what a backward pass needs),
 * new_conv_state[B,K-1,W], h_last[B,W].  No output may overlap an input (a tile reads the three rows of u in
 * front of it while its neighbour writes).  ws as for rglru_hip_fwd.  Only where
 * rglru_hip_block_fwd_path() returns 1 (bf16 storage, gate blocks of 32, 64 or 128 channels, 16-byte
 * aligned rows); otherwise RGLRU_E_UNSUPPORTED, and the caller runs rglru_hip_conv_fwd, rglru_hip_fwd and
 * rglru_hip_gelu_gate_fwd one after the other.  rglru_hip_prepare_block_fwd is rglru_hip_prepare +
 * rglru_hip_block_fwd in two launches (as rglru_hip_prepare_fwd). */
int rglru_hip_block_fwd_path(int64_t W, int64_t nb, int64_t K, int dtype);
int rglru_hip_block_flags(const int64_t* segment_pos, uint8_t* flags, int64_t n, void* stream);
int rglru_hip_block_fwd(const void* u, int64_t u_stride, const void* v, int64_t v_stride,
                        const void* conv_state, const void* taps, const void* conv_bias, int64_t K, int vec_dtype,
                        const void* prep, const float* h0, const uint8_t* flags,
                        void* x_conv, void* y, void* gated, void* new_conv_state, float* h_last, void* ws,
                        int64_t B, int64_t T, int64_t W, int64_t nb, int dtype, void* stream);
int rglru_hip_prepare_block_fwd(const void* w_a, const void* b_a, const void* w_x, const void* b_x,
                                const void* lambda, float c, int vec_dtype, void* prep,
                                const void* u, int64_t u_stride, const void* v, int64_t v_stride,
                                const void* conv_state, const void* taps, const void* conv_bias, int64_t K,
                                const float* h0, const uint8_t* flags,
                                void* x_conv, void* y, void* gated, void* new_conv_state, float* h_last, void* ws,
                                int64_t B, int64_t T, int64_t W, int64_t nb, int dtype, void* stream);

/* Test hook: number of polls a wave may spend waiting for a neighbouring chunk's carry before it
 * gives up, records the failure in the workspace and finishes with unspecified results.  The
 * default is large enough never to trigger in normal operation.  Returns the previous value. */
int64_t rglru_hip_set_spin_limit(int64_t polls);
/* Reproducible mode (off by default; no counterpart in the reference, whose scans are sequential and therefore
 * reproducible).  Chunks of a sequence exchange carries through a look-back that normally combines whatever
 * records it finds, final or not, so results agree between runs to rounding only.  With the mode on, a chunk
 * waits for the FINAL record of the chunk before it: y, h_last and everything the backward entry points
 * rglru_hip_bwd_full, rglru_hip_scan_fwd and rglru_hip_scan_bwd return are then bit-identical from run to run
 * (the bias and Lambda gradients of the other backward entry points still add per-workgroup sums whose
 * composition follows the ticket order).  The chain becomes one memory round trip per chunk: slower,
 * mostly for long sequences.  Applies to launches made after the call; returns the previous setting. */
int rglru_hip_set_reproducible(int enable);
/* Which forward kernel rglru_hip_fwd uses for bf16 storage and gate blocks of 32, 64 or 128 channels (no
 * counterpart in the reference).  0 (default): by shape -- the library estimates the time of both kernel pairs
 * from the number of (sequence, 32-channel slab) chains, the compute units and the sequence length and takes
 * the faster: one workgroup walks a whole chain (no exchange between workgroups, bit-reproducible) for small
 * and short problems and where the chains fill one to a few rounds over the compute units; tiles with a
 * look-back between workgroups for few long sequences and for very large batches.  1: always the
 * tiled kernel.  2: the chain kernel whenever it covers the storage type and block width (tests).  Applies to
 * launches made after the call; returns the previous setting. */
int rglru_hip_set_chain_forward(int mode);
/* Synchronising debug helper: copies the failure word of a workspace to the host (0 = clean). */
int rglru_hip_workspace_status(const void* ws, int64_t B, int64_t T, int64_t W, int64_t nb,
                               int scan_only, void* stream, int* status);

/* Measurement hook.  While enabled, rglru_hip_fwd / rglru_hip_bwd / rglru_hip_step bracket their
 * main kernel (not the small clear / reduce launches) with HIP events on the call's stream.
 * rglru_hip_kernel_ms(which) waits for the most recent bracket (process-wide, so enable it from one
 * thread and keep calls sequential) and returns its
 * duration in milliseconds (negative when none was recorded): which = 0 forward, 1 backward
 * (scan part), 2 step, 3 backward gradient kernel (rglru_hip_bwd_full only).  Not for use under stream capture. */
int rglru_hip_set_timing(int enable);
float rglru_hip_kernel_ms(int which);

#ifdef __cplusplus
}
#endif
#endif /* RGLRU_HIP_H */
