/* flashpop_hip.h -- C ABI of libflashpop_hip.so: fused chunked retention and POP retention
 * on AMD MI355X (gfx950).
 *
 * The reference has no native ABI for this path: its "ABI" is a TileLang JIT kernel object
 * called from two torch.autograd.Functions.  Each entry point below replaces the kernel
 * launches inside one of those four methods; the citation names that method.
 *
 * Conventions common to all entry points
 *   - every tensor pointer is DEVICE memory, bf16 (2 bytes/element), contiguous, in the
 *     reference's layouts: q, k, dq, dk [B,T,H,dk]; v, o, d_o, dv [B,T,H,dv]; states
 *     [B,H,dk,dv]; block states [B, T/block_size, H, dk, dv]
 *   - head_decays is HOST memory: H doubles, gamma_h in (0, 1]
 *   - K is divided by sqrt(dk) inside (flash_pop/fused_retention/reference.py:57); Q is not scaled
 *   - dk, dv in {64, 128, 192, 256}; 1 <= H <= 512; T >= 1; B >= 1
 *   - the caller owns every buffer; the library allocates nothing and keeps no pointer
 *   - launches are asynchronous on `stream` (a hipStream_t, NULL = default stream)
 *   - returns 0 on success, a negative FP_ERR_* code otherwise; fp_last_error() then gives a
 *     message (thread-local).  No kernel is launched when an argument check fails.
 *   - the retention, POP and split entry points must not be recorded into a HIP graph: they return
 *     FP_ERR_LAUNCH when `stream` is capturing (instantiating a graph that holds their kernels has
 *     crashed the host process).  The decode step, the rotary embedding and the norm + gate entry
 *     points can be captured.
 *   - results are deterministic: no atomics, fixed reduction order
 */
#ifndef FLASHPOP_HIP_H
#define FLASHPOP_HIP_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FP_OK 0
#define FP_ERR_NULL_POINTER (-1)
#define FP_ERR_BAD_SHAPE (-2)
#define FP_ERR_UNSUPPORTED_DIM (-3)
#define FP_ERR_BAD_DECAY (-4)
#define FP_ERR_LAUNCH (-5)
#define FP_ERR_BAD_CONFIG (-6)

/* Replaces the kernel call in FusedChunkRetention.forward
 * (flash_pop/fused_retention/__init__.py:13-31).
 *   s0     initial state, may be NULL (zeros)
 *   o      out: retention output
 *   s_out  out: state after the last token, may be NULL */
int fp_retention_fwd(const void* q, const void* k, const void* v, const void* s0, const double* head_decays,
                     void* o, void* s_out, int B, int T, int H, int dk, int dv, void* stream);

/* Replaces the two kernel calls and four reductions in FusedChunkRetention.backward
 * (flash_pop/fused_retention/__init__.py:34-47).
 *   d_o      gradient of o
 *   d_s_out  gradient of the final state, may be NULL (zeros)
 *   dq, dk_, dv_  out: gradients of q, k (unscaled), v
 *   d_s0     out: gradient of the initial state, may be NULL (not wanted) */
int fp_retention_bwd(const void* q, const void* k, const void* v, const void* s0, const double* head_decays,
                     const void* d_o, const void* d_s_out, void* dq, void* dk_, void* dv_, void* d_s0, int B, int T,
                     int H, int dk, int dv, void* stream);

/* Forward and backward with checkpoints.  The backward needs the state at the start of every
 * chunk for dq and gets it by re-running the recurrence forward (as the reference's
 * fused_retention_bwd_dq does, fused_chunk_bwd.py:432-444), which walks against the reverse
 * recurrence of dk and dv and reads k, v and d_o a second time from HBM.  When the forward leaves
 * its state every `every` tokens, the backward takes the segments between those states from the
 * last to the first, beside the reverse walk, and the second read comes from the caches.  What
 * FusedChunkRetention saves for its backward (fused_retention/__init__.py:30) grows by these states.
 *   fp_retention_checkpoint_bytes  bytes of the checkpoint buffer that pays for this shape on the
 *                                  current device and, in *every, the interval in tokens; 0 when the
 *                                  shape is served as well without (then pass NULL below)
 *   checkpoints  [B, T / every, H, dk, dv] bf16: the state after tokens every - 1, 2 every - 1, ...;
 *                written by _fwd_ckpt, read by _bwd_ckpt.  NULL: same as fp_retention_fwd / _bwd.
 *   every        a multiple of 64
 * Results are those of fp_retention_fwd / fp_retention_bwd up to the rounding of the checkpoints
 * to bf16 (dq only). */
size_t fp_retention_checkpoint_bytes(int B, int T, int H, int dk, int dv, int* every);
int fp_retention_fwd_ckpt(const void* q, const void* k, const void* v, const void* s0, const double* head_decays, void* o,
                          void* s_out, void* checkpoints, int every, int B, int T, int H, int dk, int dv, void* stream);
int fp_retention_bwd_ckpt(const void* q, const void* k, const void* v, const void* s0, const double* head_decays,
                          const void* d_o, const void* d_s_out, const void* checkpoints, int every, void* dq, void* dk_,
                          void* dv_, void* d_s0, int B, int T, int H, int dk, int dv, void* stream);

/* Long sequences with few (batch, head) streams: one workgroup walks one stream, so B * H *
 * min(dk, dv) / 64 workgroups is all a call has, and a 256-CU device idles when that is small.
 * The _split variants cut every sequence into segments that run as separate sequences (a
 * state-only pass and a scan give each segment its starting state first); they need scratch
 * memory from the caller.  Same arguments, results and error behaviour as fp_retention_fwd /
 * fp_retention_bwd otherwise; segment states pass through bf16.  No counterpart in the
 * reference, whose kernels also walk a sequence serially (fused_chunk_fwd.py:95-187).
 *   fp_retention_workspace_bytes  scratch bytes the two calls need for this shape on the current
 *                                 device; 0 means they would not cut (and accept workspace = NULL)
 *   workspace                     device memory, 16-byte aligned, at least that many bytes; two calls
 *                                 that share it must be ordered by their stream.  After
 *                                 fp_retention_fwd_split it holds the state at the start of every
 *                                 segment, which the backward needs too:
 *   forward_states_kept           nonzero: `workspace` is the buffer fp_retention_fwd_split was given
 *                                 for the same q, k, v, s0 and decays and nothing has written to it
 *                                 since; the backward then skips recomputing those states (one pass
 *                                 over k and v).  0: the workspace holds nothing of use.
 *                                 Either way its contents are undefined after the backward. */
size_t fp_retention_workspace_bytes(int B, int T, int H, int dk, int dv);
int fp_retention_fwd_split(const void* q, const void* k, const void* v, const void* s0, const double* head_decays,
                           void* o, void* s_out, int B, int T, int H, int dk, int dv, void* workspace,
                           size_t workspace_bytes, void* stream);
int fp_retention_bwd_split(const void* q, const void* k, const void* v, const void* s0, const double* head_decays,
                           const void* d_o, const void* d_s_out, void* dq, void* dk_, void* dv_, void* d_s0, int B,
                           int T, int H, int dk, int dv, void* workspace, size_t workspace_bytes,
                           int forward_states_kept, void* stream);

/* fp_retention_fwd_split without a workspace argument and without any allocation.  It has no
 * counterpart in the reference; it is for callers that cannot allocate device memory at the call:
 * tight serving loops, harnesses that forbid hipMalloc.  The segment states live in an array inside
 * the library's code object (16 MiB per device, held from the first use of the library on that
 * device until the process ends).  Same results as fp_retention_fwd_split, bit for bit.  A shape
 * whose segment states need more than 16 MiB (fp_retention_workspace_bytes says how much: 64 KiB x
 * max(dk, dv) x compute units / 256, so 16 MiB at most on a device of 256 compute units) is rejected
 * with FP_ERR_BAD_SHAPE.  Every call on a device uses that device's one array: two calls that overlap
 * in time on one device (different streams or threads) race; calls on one stream are ordered and safe. */
int fp_retention_fwd_split_static(const void* q, const void* k, const void* v, const void* s0,
                                  const double* head_decays, void* o, void* s_out, int B, int T, int H, int dk, int dv,
                                  void* stream);

/* Replaces the kernel call in FlashPOPRetention.forward
 * (flash_pop/pop_retention/__init__.py:14-31).
 *   block_states  out: state after every FULL block of block_size tokens,
 *                 [B, T / block_size, H, dk, dv]; may be NULL only if T < block_size */
int fp_pop_retention_fwd(const void* q, const void* k, const void* v, const void* s0, const double* head_decays,
                         void* o, void* block_states, int B, int T, int H, int dk, int dv, int block_size,
                         void* stream);

/* Replaces the two kernel calls and four reductions in FlashPOPRetention.backward
 * (flash_pop/pop_retention/__init__.py:34-50).  block_size is passed explicitly (the
 * reference infers it as T / num_blocks, which is wrong when T % block_size != 0).
 *   d_block_states  gradient of block_states, may be NULL (zeros) */
int fp_pop_retention_bwd(const void* q, const void* k, const void* v, const void* s0, const double* head_decays,
                         const void* d_o, const void* d_block_states, void* dq, void* dk_, void* dv_, void* d_s0,
                         int B, int T, int H, int dk, int dv, int block_size, void* stream);

/* One POP layer step in a single walk over each sequence: the context retention and the N + 1
 * suffix retentions that POPDecoderLayer.pop_forward runs as two ops, pop_chunkwise and then
 * _suffixes_forward -> _retention_chunkwise (flash_pop/pop_retnet.py:107/113 and :152-171).
 * Suffix n of sequence b reads the state at token n * block_size (s0 for n = 0) straight from
 * the walk; block states are neither written nor read back, and the concatenation of
 * [s0, block states] (pop_retnet.py:163-165) does not happen.
 *   q_sfx, k_sfx  [B * (N + 1), sfx_len, H, dk], v_sfx, o_sfx [B * (N + 1), sfx_len, H, dv], block
 *                 index fastest, N = T / block_size, as the reference batches its suffixes
 *   s_out         out: state after the last full block, the reference's `last_state`
 *                 (pop_retnet.py:169); s0 (zeros if NULL) when T < block_size; may be NULL
 * T need not be a multiple of block_size: the tokens after the last block boundary are context like
 * any others (they see the state and each other) and no suffix follows them.  sfx_len >= 1; a suffix
 * longer than 64 tokens is walked in parts of 64, like a sequence of its own that starts from the
 * state at its boundary (dk and dv of 64 or 128 only). */
int fp_pop_fused_fwd(const void* q, const void* k, const void* v, const void* s0, const void* q_sfx, const void* k_sfx,
                     const void* v_sfx, const double* head_decays, void* o, void* o_sfx, void* s_out, int B, int T,
                     int H, int dk, int dv, int block_size, int sfx_len, void* stream);

/* Gradients of fp_pop_fused_fwd (what autograd derives for the reference's two ops plus the
 * concatenation between them).
 *   d_o, d_o_sfx  gradients of o and o_sfx
 *   d_s_out       gradient of s_out, may be NULL (zeros)
 *   dq .. dv_sfx  out: gradients of q, k, v and of the suffix tensors
 *   d_s0          out: gradient of s0 (context and suffix 0 together), may be NULL (not wanted) */
int fp_pop_fused_bwd(const void* q, const void* k, const void* v, const void* s0, const void* q_sfx, const void* k_sfx,
                     const void* v_sfx, const double* head_decays, const void* d_o, const void* d_o_sfx,
                     const void* d_s_out, void* dq, void* dk_, void* dv_, void* dq_sfx, void* dk_sfx, void* dv_sfx,
                     void* d_s0, int B, int T, int H, int dk, int dv, int block_size, int sfx_len, void* stream);

/* One recurrent (decode) step for all batch entries and heads in one launch; replaces the
 * einsums of retention_recurrent (flash_pop/retnet.py:79-101):
 *   S' = gamma_h S + (k / sqrt(dk))^T v,   o = q S'
 *   q, k [B,H,dk]; v, o [B,H,dv]; s_in (may be NULL: zeros), s_out [B,H,dk,dv]; s_out may be s_in
 * The state is read once and written once; arithmetic in fp32, storage bf16. */
int fp_retention_decode_step(const void* q, const void* k, const void* v, const void* s_in, const double* head_decays,
                             void* o, void* s_out, int B, int H, int dk, int dv, void* stream);

/* Rotary position embedding of q and k in one launch; replaces the elementwise chain of
 * XPos.__call__ / _theta_shift (flash_pop/xpos_emb.py:32-40, 120-126), which the layer applies
 * to q and k right before the retention op (flash_pop/retnet.py:273-278):
 *   out[2i]   = x[2i] cos(a_i) - x[2i+1] sin(a_i),   out[2i+1] = x[2i+1] cos(a_i) + x[2i] sin(a_i)
 *   a_i = float(position) * theta[i],  position of token t of sequence b = (start ? start[b] : start0) + t
 *   q, k [B,T,H,d] bf16 (k_in and k_out may both be NULL); out may alias in; d a multiple of 8
 *   theta  DEVICE, d/2 floats (the reference's 1 / 10000^linspace(0,1,d/2), xpos_emb.py:26-28)
 *   start  DEVICE, B int64 start positions (the reference's LongTensor start_idx, xpos_emb.py:57-63), or NULL
 *   inverse != 0 rotates by -a_i: the gradient of the op with respect to its input. */
int fp_rotary_qk(const void* q_in, const void* k_in, void* q_out, void* k_out, const float* theta, const long long* start,
                 long long start0, int B, int T, int H, int d, int inverse, void* stream);

/* GroupNorm over each head of the retention output, then the swish gate, in one pass; replaces
 * group_norm(retention.float()).to(dtype) * activation(g_proj(x)) in
 * MultiScaleRetention._retention_chunkwise (flash_pop/retnet.py:294-309; GroupNorm with one group
 * per head, no affine parameters, retnet.py:194-201; swish, retnet.py:29-30), same rounding points:
 *   n = bf16((r - mean_h) / sqrt(var_h + eps)),  out = bf16(n * bf16(g / (1 + exp(-g))))
 *   r [rows,H,dv] retention output, g [rows,H*dv] gate pre-activation, out [rows,H*dv]; bf16,
 *   16-byte aligned; statistics in fp32, biased variance; dv = 8 * 2^k <= 512.
 * The backward entry point returns d_r and d_g for a given d_out (all three shaped like r). */
int fp_gated_group_norm_fwd(const void* r, const void* g, void* out, long long rows, int H, int dv, double eps,
                            void* stream);
int fp_gated_group_norm_bwd(const void* r, const void* g, const void* d_out, void* d_r, void* d_g, long long rows, int H,
                            int dv, double eps, void* stream);

/* Measurement switch; no counterpart in the reference.  Where a shape can run both the fused backward
 * kernel and the pass-per-gradient backward, the library chooses by shape; this overrides it for the
 * whole process until called again (A/B timing, tests of the path not chosen).
 *   choice            0 by shape (default), 1 always the pass kernel (for the forward of sequences of at most 32
 *                     tokens too, which otherwise has a kernel of its own), 2 the fused kernel wherever it exists,
 *                     3 as 2 with the two workgroups of a stream paced so that they meet in the L2 (fewer bytes
 *                     fetched, a slower launch: kept for that comparison)
 *   checkpoint_every  tokens between the states fp_retention_checkpoint_bytes asks the forward to leave:
 *                     a multiple of 64, 0 for none, negative to leave the current setting (default 512)
 * The environment variables FLASHPOP_BWD (auto | passes | fused | paced) and FLASHPOP_CKPT give the initial
 * values; they are read once per process, and a value that is none of these makes every entry point
 * return FP_ERR_BAD_CONFIG.  Not synchronised with calls in flight on other threads: a forward and its
 * backward must run under the same setting. */
int fp_set_backward_choice(int choice, int checkpoint_every);

/* Message for the last nonzero return on this thread ("" if none). */
const char* fp_last_error(void);

/* ABI version: major * 1000 + minor. */
int fp_version(void);

#ifdef __cplusplus
}
#endif
#endif /* FLASHPOP_HIP_H */
