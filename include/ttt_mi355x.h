/*
 * ttt_mi355x.h -- C ABI of the MI355X (gfx950) fused TTT inner loop.
 *
 * Every entry point is what the reference's FFI for this path would bind.  Paths cited
 * are relative to the reference (kilyanni/ttt-rs) checkout.
 *
 * Conventions
 *  - All pointers are DEVICE pointers unless stated; the caller owns every buffer; the
 *    library never allocates or frees device memory and never synchronises: work is
 *    enqueued on `stream` (a hipStream_t passed as void*; NULL = the default stream).
 *  - Tensors are contiguous row-major, base pointers 16-byte aligned.
 *  - Activations xq/xk/xv/out/lr (and their gradients) are stored in `io_dtype`;
 *    state (W, b), LayerNorm parameters, token_eta and all parameter gradients are f32.
 *  - Return value: TTT_OK or a negative ttt_status; ttt_last_error() gives the message
 *    of the calling thread's last failure.  No call aborts the process.
 */
#ifndef TTT_MI355X_H
#define TTT_MI355X_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
  TTT_OK = 0,
  TTT_ERR_SHAPE = -1,       /* sizes inconsistent (e.g. seq not a multiple of mini_batch) */
  TTT_ERR_UNSUPPORTED = -2, /* no kernel instantiation for (mini_batch, head_dim, dtype) */
  TTT_ERR_HIP = -3,         /* a HIP runtime call failed; see ttt_last_error() */
  TTT_ERR_NULL = -4         /* a required pointer is NULL */
} ttt_status;

typedef enum { TTT_F32 = 0, TTT_BF16 = 1 } ttt_dtype;

/*
 * Replaces FusedTttConfig (rust/fused/src/lib.rs:285-328) plus the shapes the reference
 * reads off its tensors (rust/fused/src/linear_fused_tile/forward/launch.rs:199-226).
 */
typedef struct ttt_desc {
  int32_t batch;               /* B */
  int32_t heads;               /* H */
  int32_t seq;                 /* tokens per sequence; must be a multiple of mini_batch */
  int32_t head_dim;            /* d */
  int32_t mini_batch;          /* K: 1..16; for ttt_linear_fwd / ttt_linear_bwd at head_dim 32 also 17..32 (the
                                  reference's (mini_batch 32, head_dim 32) tile,
                                  rust/fused/src/linear_fused_tile/mod.rs:31-38), with f32 row-major checkpoints */
  float eps;                   /* LayerNorm epsilon (reference default 1e-6) */
  int32_t checkpoint_interval; /* stages between W/b checkpoints, >= 1 */
  int32_t io_dtype;            /* ttt_dtype of xq, xk, xv, lr, out and their gradients */
  int32_t state_per_batch;     /* 0: W0/b0 are [H,d,d]/[H,d] shared over the batch
                                  (TTTLinear::init_state, rust/core/src/linear.rs:84-89);
                                  1: [B,H,d,d]/[B,H,d] as the reference kernel takes them */
  int32_t seq_stride;          /* tokens between consecutive (batch, head) units in xq, xk, xv, lr,
                                  out and their gradients; 0 = seq (dense).  A window of a longer
                                  sequence (the reference's slice_seq, rust/core/src/inner.rs:70-77)
                                  is processed in place by pointing at its first token and passing
                                  the full length here. */
  int32_t checkpoint_format;   /* 0: W checkpoints are f32 [d,d] row-major matrices (what the reference
                                  saves, rust/fused/src/linear_fused_tile/forward/launch.rs:117-208),
                                  any interval, readable by the caller.
                                  1 (TTT_CKPT_PACKED): checkpoint_interval 1 only; a W checkpoint is the
                                  state in the kernels' own operand order and operand type, written by
                                  ttt_linear_fwd and meaningful only to ttt_linear_bwd (same allocation).
                                  bf16 I/O: bf16 (the first d*d*2 bytes of each d*d*4-byte slot); the
                                  backward's products take bf16 operands anyway, so its results do not
                                  change; half the checkpoint traffic.  f32 I/O: f32.  Either way stored
                                  and fetched in whole 1 KiB rows instead of scattered 4-byte pieces.
                                  No counterpart in the reference.
                                  2 (TTT_CKPT_FACTORS): bf16 I/O, checkpoint_interval 1, head_dim <= 96.  No
                                  states are saved: ttt_linear_fwd writes, into the same W_ckpt / b_ckpt
                                  allocations, the state after the last mini-batch and per mini-batch the
                                  [16 x d] factor of its state update (32*d bytes instead of 2*d*d), and
                                  ttt_linear_bwd walks the state back from the end, W_t = W_{t+1} - XK_t^T G_t
                                  with the operands the forward multiplied: each state is recovered up to one
                                  f32 rounding per element and mini-batch, far below the bf16 rounding of the
                                  operands it then becomes.  A quarter of the packed format's traffic.  A
                                  sequence of one mini-batch is saved packed (the buffers are the same).
                                  Meaningful only to ttt_linear_bwd.  No counterpart in the reference. */
  int32_t kernel_hint;         /* 0 (TTT_HINT_AUTO): the library chooses the kernel from the shape.  Otherwise a
                                  tuning / testing request, read by the entry point the desc is passed to:
                                  low byte = wavefronts per (batch, head) unit for the TTT-Linear kernels
                                  (1, 2 or 4; clamped to what head_dim allows), TTT_HINT_LDS_TILES = the kernels
                                  that keep state and tiles in LDS / global memory and compute every product in
                                  f32 (TTT-Linear forward at head_dim 96/128, TTT-Linear backward at head_dim
                                  <= 64, TTT-MLP forward).  A hint that names no existing kernel for the desc is
                                  ignored.  The choice changes speed and, between bf16-operand and f32-operand
                                  kernels, rounding; never the meaning of a result.  No counterpart in the
                                  reference (its `threads` field, rust/fused/src/lib.rs:285-328, is the nearest). */
} ttt_desc;
#define TTT_CKPT_F32 0
#define TTT_CKPT_PACKED 1
#define TTT_CKPT_FACTORS 2
#define TTT_HINT_AUTO 0
#define TTT_HINT_WAVES_MASK 0xff
#define TTT_HINT_LDS_TILES 0x100
/* ttt_mlp_fwd, bf16 I/O at head_dim 96: spread every (batch, head) unit over a pair of CUs, as head_dim 128 always is
 * (see ttt_mlp_fwd), when the units number at most half the device's CUs.  Not the default: measured on MI355X the
 * pair gains 2 - 3 % at 128 units.  Ignored where only one of the two kernels exists. */
#define TTT_HINT_TWO_CU 0x400
/* ttt_linear_fwd, bf16 I/O at head_dim 64 with two waves per unit: TTT_HINT_OWN_LOADS = every wave loads only the
 * features it owns of xq, xk, xv and the full rows reach the waves through LDS (half the vector loads; the library's
 * choice above 256 units, where two workgroups share a CU); TTT_HINT_ALL_LOADS = every wave loads every row (the
 * library's choice up to 256 units).  Same results bit for bit.  Ignored where only one of the two exists.
 * ttt_linear_fwd, f32 I/O with one wave per feature tile (head_dim 32 / 64), whole mini-batches of 16 tokens and at
 * most one (batch, head) unit per CU: the library's choice is a kernel with a fifth wave that copies the operands
 * global -> LDS, so that the four compute waves issue no loads; TTT_HINT_ALL_LOADS keeps the loads in the compute
 * waves.  Same results bit for bit. */
#define TTT_HINT_OWN_LOADS 0x1000
#define TTT_HINT_ALL_LOADS 0x2000
/* ttt_mlp_bwd / ttt_mlp_bwd_static, bf16 I/O up to head_dim 96: the reverse scan normally rounds the operands of its
 * products to bf16, as the forward of the step did (f32 accumulation, f32 state and gradient accumulators);
 * TTT_HINT_F32_PRODUCTS keeps every product of the scan in f32 (about twice the time).  Ignored elsewhere: f32 I/O and
 * head_dim 128 always compute in f32. */
#define TTT_HINT_F32_PRODUCTS 0x4000
/* ttt_mlp_bwd and its variants: with at most 128 (batch, head) units every unit is worked on by two workgroups on two
 * CUs (see ttt_mlp_bwd); TTT_HINT_ONE_WORKGROUP keeps a unit on one.  Same results bit for bit (d_token_eta, which
 * is summed over the units with atomic additions, aside); the workspace is smaller. */
#define TTT_HINT_ONE_WORKGROUP 0x8000
/* Testing only: the two workgroups that share a (batch, head) unit in ttt_mlp_fwd at head_dim 128 (bf16 I/O) give
 * up waiting for each other at once, as if the partner had never become resident.  Exercises the failure path
 * described at ttt_mlp_fwd: every output of the affected units is NaN.  All kernels still run to their end. */
#define TTT_HINT_TEST_LOST_PARTNER 0x200
/* Testing only: the same two workgroups treat each other as running on different XCDs whatever they find at start,
 * i.e. take the path of a pair that was not placed on one XCD: every word they exchange is stored at device scope
 * instead of staying in the XCD's L2.  Slower; results identical. */
#define TTT_HINT_TEST_OTHER_XCD 0x800

/* Library / build identification. */
const char* ttt_version(void);
/* Message of the calling thread's last error ("" if none). */
const char* ttt_last_error(void);
/* TTT_OK if a TTT-Linear kernel exists for this desc, else the status ttt_linear_fwd would
 * return.  Replaces FusedTttConfig::is_supported (rust/fused/src/lib.rs:313-322). */
int ttt_linear_supported(const ttt_desc* desc);
/* Number of checkpoints per (batch, head): ceil((seq/mini_batch)/checkpoint_interval)
 * (rust/fused/src/linear_fused_tile/forward/launch.rs:221-226). */
int64_t ttt_linear_num_checkpoints(const ttt_desc* desc);
/* TTT_OK if ttt_linear_bwd has a kernel for this desc (it supports fewer combinations than the forward:
 * checkpoint_interval > 1 only for head_dim <= 96; f32 I/O at head_dim 128 and mini_batch > 16 with f32 row-major
 * checkpoints only), else the status
 * ttt_linear_bwd would return.  A training caller asks this before the forward, as the reference asks
 * FusedTttConfig::is_supported (rust/fused/src/lib.rs:313-322) before it builds the layer. */
int ttt_linear_bwd_supported(const ttt_desc* desc);
/* The checkpoint_format that makes ttt_linear_fwd + ttt_linear_bwd fastest for this desc (its own checkpoint_format
 * field is not read) when nothing but ttt_linear_bwd reads the checkpoints: TTT_CKPT_FACTORS for bf16 I/O,
 * checkpoint_interval 1, head_dim <= 96, two or more mini-batches and up to 512 (batch, head) units; else
 * TTT_CKPT_PACKED for checkpoint_interval 1; else TTT_CKPT_F32 -- always a format that ttt_linear_bwd accepts under
 * the desc's checkpoint_interval and kernel_hint (TTT_HINT_LDS_TILES reads f32 matrices only).  A negative ttt_status
 * if the desc is invalid or ttt_linear_bwd has no kernel for it in any format.  No counterpart in the reference (its
 * checkpoints have one format). */
int ttt_linear_best_checkpoint_format(const ttt_desc* desc);

/*
 * TTT-Linear multi-stage forward.  Replaces
 *   FusedKernelBackend<TttTileMultiKernel>::forward
 *     (rust/kernels/src/kernel.rs:62-69; rust/fused/src/linear_fused_tile/launch.rs:123-161)
 *   -> forward_multi (rust/fused/src/linear_fused_tile/forward/launch.rs:199-257)
 * with TttInputs{xq,xk,xv,weight,bias,token_eta,ttt_lr_eta,ln_weight,ln_bias} and
 * TttOutputs{output,weight,bias} (rust/fused/src/ttt/types.rs:3-13).
 *
 *  xq,xk,xv [B,H,seq,d] io   W0 [H,d,d] or [B,H,d,d] f32   b0 [H,d] or [B,H,d] f32
 *  token_eta [K] f32 (position inside the mini-batch; the reference kernel reads
 *            token_eta[0..K) of its [seq] tensor, helpers.rs:261-264)
 *  lr [B,H,seq] io (ttt_lr_eta)        gamma,beta [H,d] f32
 *  out [B,H,seq,d] io    W_out [B,H,d,d] f32    b_out [B,H,d] f32
 *  W_ckpt [B,H,C,d,d] f32, b_ckpt [B,H,C,d] f32 with C = ttt_linear_num_checkpoints();
 *  both may be NULL (no checkpoints written).  Checkpoint c holds the state ENTERING
 *  stage c*checkpoint_interval (forward/kernel.rs:143-150).
 */
int ttt_linear_fwd(const ttt_desc* desc, const void* xq, const void* xk, const void* xv,
                   const float* W0, const float* b0, const float* token_eta, const void* lr,
                   const float* gamma, const float* beta, void* out, float* W_out, float* b_out,
                   float* W_ckpt, float* b_ckpt, void* stream);

/*
 * TTT-Linear fused backward.  Replaces
 *   FusedKernelBackend<TttTileMultiKernel>::backward
 *     (rust/kernels/src/kernel.rs:71-75; rust/fused/src/linear_fused_tile/launch.rs:163-207)
 *   -> backward_multi (rust/fused/src/linear_fused_tile/backward/launch.rs:332-438).
 * Saved state = the nine forward inputs plus the checkpoints written by ttt_linear_fwd
 * with the same desc (TttSavedStateMulti, launch.rs:30-41).
 *
 *  d_out [B,H,seq,d] io.   d_W_out [B,H,d,d], d_b_out [B,H,d] f32: upstream gradients of the
 *  final state, may be NULL (= zero, which is what the reference assumes, launch.rs:188-194).
 *  Outputs: d_xq,d_xk,d_xv [B,H,seq,d] io; d_W0 [B,H,d,d] f32 and d_b0 [B,H,d] f32 (per batch
 *  element; the parameter gradient is their batch sum); d_lr [B,H,seq] io;
 *  d_token_eta [seq] f32 per position (summed over batch and heads, backward/kernel.rs:390);
 *  d_gamma,d_beta [H,d] f32 (summed over batch).  The three accumulated outputs
 *  (d_token_eta, d_gamma, d_beta) are zeroed by the library on `stream` before use.
 */
int ttt_linear_bwd(const ttt_desc* desc, const void* xq, const void* xk, const void* xv,
                   const float* W0, const float* b0, const float* token_eta, const void* lr,
                   const float* gamma, const float* beta, const float* W_ckpt,
                   const float* b_ckpt, const void* d_out, const float* d_W_out,
                   const float* d_b_out, void* d_xq, void* d_xk, void* d_xv, float* d_W0,
                   float* d_b0, void* d_lr, float* d_token_eta, float* d_gamma, float* d_beta,
                   void* stream);

/*
 * ttt_linear_bwd with a caller-owned workspace: the same call (same interface of the reference replaced, same
 * arguments, same results to rounding) for a caller that can hold ttt_linear_bwd_workspace_bytes(desc) bytes of
 * device memory (16-byte aligned, ordinary hipMalloc memory, nothing in it has to be kept between calls).  The
 * workspace argument itself has no counterpart in the reference.  Where that size is above zero -- f32 I/O,
 * checkpoint_interval 1 (row-major or packed checkpoints), head_dim 32 or 64, at most 128 (batch, head) units, no
 * TTT_HINT_ONE_WORKGROUP or wave hint -- and the device has two CUs per unit, the reverse scan of a unit runs on two
 * workgroups on two CUs: one recomputes what depends only on the saved state (Z1, G, Zbar, dZbar, the attention
 * block's gradients, d_xq), the other carries the state gradient (dZ1, d_xk, d_xv, d_lr, d_token_eta, dW, db); they
 * hand their data over through a ring of three slots per unit in the workspace and follow each other through two
 * counters there.  The f32 backward is bound by the matrix instructions of the CUs that hold a unit, and a batch of
 * 8 x 12 heads leaves 160 of 256 CUs idle: at that shape (head_dim 64, 2048 tokens) the backward takes 0.44 instead of
 * 0.72 ms.
 * Both workgroups must be resident together, and what ttt_mlp_fwd says of a GPU shared with other work holds here: a
 * workgroup that waits for its partner in vain (2^21 polls, seconds) gives up, both run to the end without waiting
 * again, the unit's d_b0 is NaN in every element (its other gradients are then meaningless) and
 * ttt_mlp_fwd_lost_workgroups counts the two workgroups.  With workspace == NULL, or where the size is zero, the call
 * is ttt_linear_bwd.  ttt_linear_bwd_workspace_bytes returns a negative ttt_status for a desc without a backward.
 */
int64_t ttt_linear_bwd_workspace_bytes(const ttt_desc* desc);
int ttt_linear_bwd_ws(const ttt_desc* desc, const void* xq, const void* xk, const void* xv,
                      const float* W0, const float* b0, const float* token_eta, const void* lr,
                      const float* gamma, const float* beta, const float* W_ckpt,
                      const float* b_ckpt, const void* d_out, const float* d_W_out,
                      const float* d_b_out, void* d_xq, void* d_xk, void* d_xv, float* d_W0,
                      float* d_b0, void* d_lr, float* d_token_eta, float* d_gamma, float* d_beta,
                      void* workspace, void* stream);

/*
 * TTT-MLP multi-stage forward (two-layer inner model d -> 4d -> d, tanh-GELU).  The reference
 * has no fused kernel for it; this is the fused counterpart of TTTMLP::forward
 * (rust/core/src/mlp.rs:127-208 looped as rust/core/src/inner.rs:25-50) behind the same
 * bundle convention.  W1_0 [H,d,4d] or [B,H,d,4d], b1_0 [H,4d] or [B,H,4d], W2_0 [H,4d,d] or
 * [B,H,4d,d], b2_0 [H,d] or [B,H,d] (state_per_batch selects); outputs are per batch element.
 *
 * head_dim 128 with bf16 I/O: a unit's state (512 KiB) is the whole register file of a CU, so a PAIR of
 * workgroups on two CUs of one XCD shares each unit and exchanges partial results once per mini-batch through
 * global memory, in the L2 cache those two CUs share (the two workgroups tell each other at start which XCD they run
 * on; a pair that was not placed on one XCD exchanges through device-scope stores instead: slower, same results).
 * head_dim 96 with bf16 I/O runs on one CU per unit, or on a pair like head_dim 128 when TTT_HINT_TWO_CU asks for it;
 * everything said here of head_dim 128 then holds for it too.  During the call W2_out is also that exchange area (the
 * library zero-fills it first; its contents are meaningless until the call's work has finished); it must be
 * ordinary device memory (hipMalloc), not fine-grained or host memory.  The library launches at most as many workgroups at a time as
 * the device has CUs, so on a GPU that is not shared both halves of every pair are resident together.  If a
 * workgroup nevertheless waits for its partner in vain (2^21 polls, seconds: CUs held by other processes or
 * streams), the
 * call cannot report it -- it returned TTT_OK when the work was enqueued -- so the failure is made impossible to
 * miss in the data instead: EVERY output of that unit (its rows of out, W1_out, b1_out, W2_out, b2_out) is NaN.
 * A caller that shares the GPU checks one output element per unit, reads the status word below, or passes
 * TTT_HINT_LDS_TILES to use the single-workgroup kernel (slower, f32 products).
 *
 * ttt_mlp_fwd_lost_workgroups: the device's status word of that kernel (and of the kernels of ttt_mlp_bwd and
 * ttt_linear_bwd_ws on two workgroups per unit, see there), the number of workgroups whose wait for
 * their partner ran out since the library was loaded on the current device (0 on a healthy run; it never
 * decreases, compare with the value before the call).  A blocking copy from the device: call it after the
 * stream's work has finished.  No counterpart in the reference.
 */
int ttt_mlp_supported(const ttt_desc* desc);
int ttt_mlp_fwd_lost_workgroups(int64_t* count);
int ttt_mlp_fwd(const ttt_desc* desc, const void* xq, const void* xk, const void* xv,
                const float* W1_0, const float* b1_0, const float* W2_0, const float* b2_0,
                const float* token_eta, const void* lr, const float* gamma, const float* beta,
                void* out, float* W1_out, float* b1_out, float* W2_out, float* b2_out,
                void* stream);

/*
 * TTT-MLP fused backward: gradients of sum(out * d_out) (plus the inner product of the final state
 * with d_W1_out .. d_b2_out, if given) through the inner loop that ttt_mlp_fwd runs.  The
 * reference has no fused MLP kernel: it differentiates TTTMLP::forward_mini_batch
 * (rust/core/src/mlp.rs:127-208) with Burn autodiff, and this call replaces that autodiff path
 * the way ttt_linear_bwd replaces fused_ttt_backward_kernel_multi (GELU second derivative:
 * rust/thundercube/src/unary_ops.rs:175-195; second-order LayerNorm:
 * rust/fused/src/linear_fused_tile/layer_norm.rs:428-709).
 *
 * Inputs are those of ttt_mlp_fwd (the call re-runs the forward sweep itself, so nothing has to be
 * saved by the caller) plus d_out [B,H,seq,d] io and the optional upstream gradients of the final
 * state (all four or none; NULL = zero): d_W1_out [B,H,d,4d], d_b1_out [B,H,4d],
 * d_W2_out [B,H,4d,d], d_b2_out [B,H,d], f32.
 * Outputs: d_xq,d_xk,d_xv [B,H,seq,d] io; d_W1 [B,H,d,4d], d_b1 [B,H,4d], d_W2 [B,H,4d,d],
 * d_b2 [B,H,d] f32 per batch element (the parameter gradients are their batch sums);
 * d_lr [B,H,seq] io; d_token_eta [seq] f32 per position (summed over batch and heads);
 * d_gamma, d_beta [H,d] f32 (summed over batch).  The accumulated outputs are zeroed by the
 * library on `stream`.
 * workspace: ttt_mlp_bwd_workspace_bytes(desc) bytes of device memory, 16-byte aligned, owned by
 * the caller and free to reuse after the call's work on `stream` has finished.  It holds the
 * rolling state, the per-mini-batch update factors of the forward sweep and scratch tiles.
 * seq must be a multiple of mini_batch.
 *
 * Two workgroups per unit.  With at most 128 (batch, head) units (and at least two CUs per unit on the device; no
 * TTT_HINT_ONE_WORKGROUP) the reverse scan of a unit runs on two workgroups on two CUs: one walks the state back and
 * recomputes the forward's intermediates a mini-batch ahead, the other carries the gradient; they hand their data
 * over in the workspace (which is larger for such a desc) and follow each other through two counters there.  Same
 * results as on one workgroup, bit for bit.  Both must be resident together, as in ttt_mlp_fwd at head_dim 128,
 * and what is said there of a GPU shared with other work holds here: a workgroup that waits for its partner in
 * vain (2^21 polls, seconds) gives up, both run to the end without waiting again, the unit's d_b1 is NaN in every
 * element (the unit's other gradients are then meaningless) and ttt_mlp_fwd_lost_workgroups counts the two
 * workgroups.  The workspace must be ordinary device memory (hipMalloc), not fine-grained or host memory.
 */
int64_t ttt_mlp_bwd_workspace_bytes(const ttt_desc* desc);
int ttt_mlp_bwd(const ttt_desc* desc, const void* xq, const void* xk, const void* xv,
                const float* W1_0, const float* b1_0, const float* W2_0, const float* b2_0,
                const float* token_eta, const void* lr, const float* gamma, const float* beta,
                const void* d_out, const float* d_W1_out, const float* d_b1_out,
                const float* d_W2_out, const float* d_b2_out, void* d_xq, void* d_xk, void* d_xv,
                float* d_W1, float* d_b1, float* d_W2, float* d_b2, void* d_lr, float* d_token_eta,
                float* d_gamma, float* d_beta, void* workspace, void* stream);

/*
 * Forward that saves for the backward, and the backward that uses what was saved: ttt_mlp_fwd_saving +
 * ttt_mlp_bwd_saved give the results of ttt_mlp_fwd + ttt_mlp_bwd (bit for bit) without the backward running the
 * forward sweep a second time.  The reference differentiates TTTMLP::forward_mini_batch with Burn autodiff, which
 * keeps the forward's activations for the backward (rust/core/src/mlp.rs:127-208); this pair is the fused counterpart
 * of that: the forward leaves in `saved` (ttt_mlp_bwd_workspace_bytes(desc) bytes of device memory, 16-byte aligned,
 * caller-owned) the two rank-16 factors of every mini-batch's state update and a copy of the final state, about
 * 2 K (5 d) floats per mini-batch and unit instead of the activations.  ttt_mlp_bwd_saved takes the arguments of
 * ttt_mlp_bwd with `saved` in place of the workspace, the same desc and the same inputs as the forward; it consumes
 * `saved` (the state in it is walked back), so a second backward needs a second forward or ttt_mlp_bwd.
 * Exists where the forward's kernel is also the backward's sweep: bf16 I/O up to head_dim 96 (one CU per unit) and
 * f32 I/O; ttt_mlp_fwd_saving_supported says so beforehand (TTT_ERR_UNSUPPORTED for the forward on pairs of CUs:
 * head_dim 128 with bf16 I/O, TTT_HINT_TWO_CU).
 */
int ttt_mlp_fwd_saving_supported(const ttt_desc* desc);
int ttt_mlp_fwd_saving(const ttt_desc* desc, const void* xq, const void* xk, const void* xv,
                       const float* W1_0, const float* b1_0, const float* W2_0, const float* b2_0,
                       const float* token_eta, const void* lr, const float* gamma, const float* beta,
                       void* out, float* W1_out, float* b1_out, float* W2_out, float* b2_out, void* saved,
                       void* stream);
int ttt_mlp_bwd_saved(const ttt_desc* desc, const void* xq, const void* xk, const void* xv,
                      const float* W1_0, const float* b1_0, const float* W2_0, const float* b2_0,
                      const float* token_eta, const void* lr, const float* gamma, const float* beta,
                      const void* d_out, const float* d_W1_out, const float* d_b1_out,
                      const float* d_W2_out, const float* d_b2_out, void* d_xq, void* d_xk, void* d_xv,
                      float* d_W1, float* d_b1, float* d_W2, float* d_b2, void* d_lr, float* d_token_eta,
                      float* d_gamma, float* d_beta, void* saved, void* stream);

/*
 * ttt_mlp_bwd without a workspace argument and without any allocation.  No counterpart in the
 * reference; it is for callers that cannot allocate device memory around the call (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  Same arguments, results
 * and kernels as ttt_mlp_bwd; the workspace is a buffer of TTT_MLP_BWD_STATIC_MAX_BYTES that is part of
 * the library's device image (each GPU the library runs on holds it until the process ends).
 * A desc with ttt_mlp_bwd_workspace_bytes(desc) > TTT_MLP_BWD_STATIC_MAX_BYTES is refused with
 * TTT_ERR_SHAPE (use ttt_mlp_bwd then).  All calls on one GPU share that buffer: calls that overlap on
 * one GPU (different streams or threads) race; calls on one stream, or otherwise ordered, are safe.
 * Nothing in the buffer has to survive between calls.
 */
#define TTT_MLP_BWD_STATIC_MAX_BYTES (32u << 20)
int ttt_mlp_bwd_static(const ttt_desc* desc, const void* xq, const void* xk, const void* xv,
                       const float* W1_0, const float* b1_0, const float* W2_0, const float* b2_0,
                       const float* token_eta, const void* lr, const float* gamma, const float* beta,
                       const void* d_out, const float* d_W1_out, const float* d_b1_out,
                       const float* d_W2_out, const float* d_b2_out, void* d_xq, void* d_xk, void* d_xv,
                       float* d_W1, float* d_b1, float* d_W2, float* d_b2, void* d_lr,
                       float* d_token_eta, float* d_gamma, float* d_beta, void* stream);

/*
 * A stack of inner models applied layer by layer (the long-context benchmark configuration: six TTT-Linear layers
 * followed by two TTT-MLP layers): layer l runs its inner loop on
 *     xq = x + pq_l,  xk = x + pk_l,  xv = x + pv_l      (x = output of layer l-1; layer 0: x = 0)
 * where the sums are formed in f32 and rounded to io_dtype, and hands its output to layer l+1; the last layer's
 * output is `out`.  One call enqueues everything: per layer and hand-over window one pass that forms the three
 * sums (x is read once for all three) and the layer's ttt_linear_fwd / ttt_mlp_fwd launch, with desc (shape, eps,
 * io_dtype, kernel_hint) shared by all layers and token_eta [mini_batch] shared too.
 *
 * Cross-layer wavefront.  A layer needs only tokens [0, t) of the layer below to process its own tokens [0, t),
 * and one launch of a long-context shape fills a fraction of the GPU (a (batch, head) unit is one or two
 * workgroups), so layers can run side by side: with chunk_tokens = c > 0 (a multiple of mini_batch that divides
 * seq) every layer works window by window of c tokens, carrying its state from window to window, and window j of
 * layer l is ready as soon as window j of layer l-1 and window j-1 of layer l are done.  The windows with
 * l + j = t (a diagonal) are independent of each other; those of one kind go in ONE launch (up to eight
 * argument blocks travel as kernel arguments and a workgroup picks its own), diagonal after diagonal, and so do
 * their input sums.  aux_stream = NULL: everything on `stream`, in that order, with no events.  aux_stream = a second
 * caller-owned stream (default priority, not the null stream): the TTT-MLP launches go there and run beside
 * the TTT-Linear launches, ordered by events where a layer follows a layer of the other kind; `stream` is joined
 * to it at the start and at the end, so for the caller the call is still one piece of work on `stream`.
 * chunk_tokens = 0: one launch per layer on `stream`, bit-identical to calling ttt_linear_fwd / ttt_mlp_fwd layer
 * by layer.  This is what the reference's streaming kernels are for (a layer's kernel stays resident and is fed
 * window by window, rust/fused/src/linear_fused_tile/streaming/d2d/kernel.rs:98-232), done with ordinary launches
 * in dependency order instead of a resident kernel polling a host-visible flag.
 * Results do not depend on the plan beyond the last bits (a layer splits its state into row means and the rest at
 * the start of every launch, see ttt_linear_fwd, so windows round differently from one long launch).
 *
 * kind: TTT_LAYER_LINEAR uses W1 = weight_init [H,d,d] (or [B,H,d,d]), b1 = bias_init; TTT_LAYER_MLP uses W1, b1,
 * W2, b2 as ttt_mlp_fwd does (state_per_batch selects the leading dimension).  W1_out .. b2_out receive the
 * layer's final state per batch element (Linear: W1_out [B,H,d,d], b1_out [B,H,d]; the other two unused).
 * workspace: ttt_stack_fwd_workspace_bytes(...) bytes for the same plan, 16-byte aligned, caller-owned, free again
 * when the call's work on `stream` has finished (three tensors of input sums; with a wavefront also one spare
 * copy of every layer's state).  `out` doubles as the hand-over tensor between layers:
 * it holds intermediate layers' outputs while the call runs.
 * checkpoint fields of desc are ignored (forward only); seq_stride must be 0.
 * A stack that holds a TTT-MLP layer at head_dim 128 with bf16 I/O runs the two-CU kernel of ttt_mlp_fwd, and what is
 * said there of a GPU shared with other work holds: the call returns when the work is enqueued, so a caller compares
 * ttt_mlp_fwd_lost_workgroups before the call and after the stream's work has finished (an affected unit's outputs
 * are NaN from that layer on).
 */
#define TTT_LAYER_LINEAR 0
#define TTT_LAYER_MLP 1
typedef struct ttt_stack_layer {
  int32_t kind;
  const void *pq, *pk, *pv; /* [B,H,seq,d] io */
  const float *W1, *b1, *W2, *b2;
  const void* lr;           /* [B,H,seq] io (ttt_lr_eta of this layer) */
  const float *gamma, *beta; /* [H,d] */
  float *W1_out, *b1_out, *W2_out, *b2_out;
} ttt_stack_layer;
int64_t ttt_stack_fwd_workspace_bytes(const ttt_desc* desc, int32_t n_layers, const ttt_stack_layer* layers,
                                      int32_t chunk_tokens);
int ttt_stack_fwd(const ttt_desc* desc, int32_t n_layers, const ttt_stack_layer* layers /* host memory */,
                  const float* token_eta, void* out, void* workspace, int32_t chunk_tokens,
                  void* aux_stream /* hipStream_t or NULL */, void* stream);

/*
 * The elementwise work either side of the inner loop, one HBM-bound pass each (the GEMMs of the
 * projections stay with the BLAS the caller uses).  desc supplies batch, heads, seq, head_dim,
 * mini_batch and io_dtype; the other fields are ignored.
 *
 * ttt_inner_inputs: TTT::get_inner_loop_inputs after the projections
 * (rust/layer/src/ttt.rs:147-194 get_qkv, :205-227 get_lr, :247-268).
 *   xq,xk,xv [B,seq,H,d] io as the q/k/v projections (and q/k convolutions) leave them;
 *   lr_logits [B,seq,H] io = x . learnable_ttt_lr_weight^T; lr_bias [H] f32; token_idx,
 *   learnable_token_idx [mini_batch] f32; rope_cos, rope_sin [npos, d/2] f32 as
 *   RotaryEmbedding::get_cos_sin builds them (rust/core/src/util.rs:289-322; its two halves are
 *   equal, pass one), or both NULL for no position encoding.  Token t uses table row
 *   (pos_offset + t), modulo pos_wrap when pos_wrap > 0 (ttt.rs:183-189: RopeGlobal passes
 *   (start_idx, none), the default passes (start_idx % mini_batch, mini_batch)).
 *   Outputs: xq_out,xk_out,xv_out [B,H,seq,d] io (head split; xq,xk rotated: permute_qk ->
 *   rotate-half RoPE -> undo_permute_qk, ttt.rs:26-41, util.rs:349-392); lr_out [B,H,seq] io =
 *   base_lr * sigmoid(lr_logits + lr_bias) / d; token_eta_out [seq] f32 =
 *   max(token_idx + learnable_token_idx, 0) tiled.  Outputs must not alias inputs.
 *
 * ttt_layer_epilogue: TTT::forward after the inner model (ttt.rs:285-297) up to the output
 * projection: inner_out [B,H,seq,d] io -> head merge -> post_norm LayerNorm over H*d (weight, bias
 * [H*d] f32, eps) -> times gelu_tanh(gate [B,seq,H*d] io) when gate is not NULL -> out [B,seq,H*d] io.
 * H*d <= 2048.
 */
int ttt_inner_inputs(const ttt_desc* desc, const void* xq, const void* xk, const void* xv,
                     const void* lr_logits, const float* lr_bias, float base_lr, const float* token_idx,
                     const float* learnable_token_idx, const float* rope_cos, const float* rope_sin,
                     int pos_offset, int pos_wrap, void* xq_out, void* xk_out, void* xv_out, void* lr_out,
                     float* token_eta_out, void* stream);
int ttt_layer_epilogue(const ttt_desc* desc, const void* inner_out, const float* post_norm_weight,
                       const float* post_norm_bias, float eps, const void* gate, void* out, void* stream);

/*
 * ttt_inner_inputs and ttt_linear_fwd in one kernel: the TTT-Linear forward on the projections as they leave the
 * GEMMs.  Replaces TTT::get_inner_loop_inputs after the projections (rust/layer/src/ttt.rs:147-194 get_qkv, :205-227
 * get_lr, :247-268) followed by FusedKernelBackend<TttTileMultiKernel>::forward (rust/kernels/src/kernel.rs:62-69):
 * the head split is a row stride of the kernel's loads, the rotary embedding of xq and xk and the lr gate are applied
 * to the tiles in registers (each feature by the one wave that owns it), token_eta is formed from its two addends;
 * the [B,H,seq,d] copies of xq, xk, xv that ttt_inner_inputs writes and ttt_linear_fwd reads are never made.
 *   xq,xk,xv [B,seq,H,d] io; lr_logits [B,seq,H] io; lr_bias [H]; token_idx, learnable_token_idx [mini_batch];
 *   rope_cos, rope_sin [npos, d/2] f32 or both NULL; pos_offset, pos_wrap as for ttt_inner_inputs, with pos_wrap
 *   either a divisor of mini_batch (positions repeat with the mini-batch: the reference's default, ttt.rs:186-189)
 *   or 0 (positions over the sequence, RopeGlobal).
 *   W0 .. b_ckpt as for ttt_linear_fwd (out [B,H,seq,d] io).
 *   xq_out, xk_out, xv_out [B,H,seq,d] io, lr_out [B,H,seq] io, token_eta_out [seq] f32: the operands as the
 *   kernel used them, i.e. exactly what ttt_inner_inputs would have written; ttt_linear_bwd takes them as its saved
 *   inputs.  Each may be NULL (not stored: inference).
 * Exists for bf16 I/O, head_dim 32 and 64, checkpoint formats TTT_CKPT_F32 and TTT_CKPT_PACKED, seq_stride 0;
 * ttt_linear_fwd_fused_inputs_supported says so beforehand (TTT_OK or the status the call would return; has_rope:
 * whether tables will be passed).  Results equal ttt_inner_inputs followed by ttt_linear_fwd on the same values
 * (same rounding of the rotated operands and of lr to the I/O type).
 */
int ttt_linear_fwd_fused_inputs_supported(const ttt_desc* desc, int pos_wrap, int has_rope);
int ttt_linear_fwd_fused_inputs(const ttt_desc* desc, const void* xq, const void* xk, const void* xv,
                                const void* lr_logits, const float* lr_bias, float base_lr, const float* token_idx,
                                const float* learnable_token_idx, const float* rope_cos, const float* rope_sin,
                                int pos_offset, int pos_wrap, const float* W0, const float* b0, const float* gamma,
                                const float* beta, void* out, float* W_out, float* b_out, float* W_ckpt, float* b_ckpt,
                                void* xq_out, void* xk_out, void* xv_out, void* lr_out, float* token_eta_out,
                                void* stream);

/*
 * TTT-MLP with n_hidden = 2, 3 or 4 hidden layers of width 4 d (d -> 4d -> ... -> 4d -> d, tanh-GELU between),
 * multi-stage forward: the fused counterpart of TTTMLP2 / TTTMLP3 / TTTMLP4::forward (rust/core/src/mlp2.rs:152-243,
 * mlp3.rs:162-279, mlp4.rs:186-324 looped as rust/core/src/inner.rs:25-50; the reference has no fused kernel for them).
 * W0, b0: host arrays of n_hidden + 1 device pointers, weight layer i = [H,in_i,out_i] or [B,H,in_i,out_i] and
 * [H,out_i] or [B,H,out_i] (state_per_batch selects; in_0 = out_last = d, every other side 4 d); W_out, b_out: the
 * same shapes per batch element, also the live state during the call (W_out[i] must not alias W0[i]).
 * Products are f32 for both I/O types.  head_dim 32 with 2 - 4 hidden layers, head_dim 64 with 2 (what fits the
 * LDS of a CU); ttt_mlpn_supported says so beforehand.  One hidden layer is ttt_mlp_fwd.  desc.seq_stride is
 * honoured (a window of a longer sequence in place).
 */
int ttt_mlpn_supported(const ttt_desc* desc, int n_hidden);
int ttt_mlpn_fwd(const ttt_desc* desc, int n_hidden, const void* xq, const void* xk, const void* xv,
                 const float* const* W0, const float* const* b0, const float* token_eta, const void* lr,
                 const float* gamma, const float* beta, void* out, float* const* W_out, float* const* b_out,
                 void* stream);

/*
 * TTT-Linear with an Adam inner optimiser, multi-stage forward.  The fused counterpart of TTTLinearAdam::forward
 * (rust/core/src/linear_adam.rs:183-236 looped as rust/core/src/inner.rs:25-50; the reference has no fused kernel for
 * it): the mini-batch of ttt_linear_fwd with the state update W -= XK^T (eta_last G), b -= colsum(eta_last G)
 * replaced by one Adam step on those gradients (adam_update, linear_adam.rs:76-128):
 *   m = beta1 m + (1 - beta1) g;  v = beta2 v + (1 - beta2) g^2;  t = step0 + mini-batches so far + 1;
 *   theta -= adam_lr (m / (1 - beta1^t)) / (sqrt(v / (1 - beta2^t)) + adam_eps).
 * xq .. beta, out, W_out, b_out as for ttt_linear_fwd (no checkpoints: forward only).  Moments are f32 in the layout of
 * the state, per batch element: Wm0, Wv0 [B,H,d,d], bm0, bv0 [B,H,d] enter (all four NULL: zero moments and step0 = 0,
 * TTTLinearAdam::init_state, linear_adam.rs:164-177), Wm_out .. bv_out leave; the step counter after the call is
 * step0 + seq / mini_batch.  State, moments and arithmetic are f32 for both I/O types (the reference keeps the first
 * moment in the backend's float type).  head_dim 32 and 64; ttt_linear_adam_supported says so beforehand.
 */
int ttt_linear_adam_supported(const ttt_desc* desc);
int ttt_linear_adam_fwd(const ttt_desc* desc, const void* xq, const void* xk, const void* xv, const float* W0,
                        const float* b0, const float* Wm0, const float* bm0, const float* Wv0, const float* bv0,
                        int step0, float beta1, float beta2, float adam_eps, float adam_lr, const float* token_eta,
                        const void* lr, const float* gamma, const float* beta, void* out, float* W_out, float* b_out,
                        float* Wm_out, float* bm_out, float* Wv_out, float* bv_out, void* stream);

/*
 * Self-test of a hardware fact the bf16 kernels rely on; no counterpart in the reference.  One wavefront computes
 * D = A1*B1 with one bf16 matrix instruction and D2 = A2*B2 + D with an instruction of the other shape (order 0:
 * 16x16x32 then 16x16x16 with D2 written over D; order 1: the reverse; orders 2, 3: the same two with D2 in other
 * registers), `gap` wait states apart (0, 4 or 5), on fixed small-integer operands:
 * A_p[i][k] = (7 i + 3 k + 5 p) mod 7 - 3 and B_p[k][j] = (5 j + 11 k + 3 p) mod 7 - 3 for product p (0 first, 1 second;
 * k < 32 or 16 by shape).  out: 256 floats, D2 row-major [16][16].  With five wait states the result is exact; closer
 * pairs are what the library's build refuses in compiler-generated code (MI355X returns wrong sums for them).
 * Enqueues one tiny kernel on `stream`.
 */
int ttt_selftest_mfma_mixed(int order, int gap, float* out, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* TTT_MI355X_H */
