// Arguments of one "retention pass" launch, shared by host and device code.
//
// Every kernel launch of this library is one instance of the same recurrence over the
// tokens of each (batch, head) stream, in chunks of CH tokens of length L <= CH:
//
//   Y_i  = s_intra * sum_j m(i,j) (x_i . w_j) z_j  +  wread(i) * x_i R
//   R   <- gamma^L R + sum_j wkey(j) w_j^T z_j
//
// forward in time (reverse == 0):  m = gamma^(i-j) [i >= j],  wread(i) = s_read   * gamma^(i+1),
//                                  wkey(j) = s_update * gamma^(L-1-j)
// backward in time (reverse == 1): m = gamma^(j-i) [j >= i],  wread(i) = s_read   * gamma^(L-1-i),
//                                  wkey(j) = s_update * gamma^(j+1)
//
// X, W are [B, T, H, dA]; Z, Y are [B, T, H, dB]; R is a dA x dB matrix per (b, h) kept in
// fp32 registers for the whole sequence.  The retention forward and its three gradient
// passes are four choices of (X, W, Z, R); see flashpop_api.cpp.
#pragma once
#include <stdint.h>
#include <stddef.h>

namespace fpk {

constexpr int CH = 64;          // tokens per chunk
constexpr int BV = 64;          // columns of Z / Y / R owned by one workgroup
constexpr int MAX_HEADS = 512;   // per-head decays travel in the kernel arguments (2 KB of the 4 KB a launch may carry)

struct PassArgs {
  const uint16_t* X;
  const uint16_t* W;
  const uint16_t* Z;
  uint16_t* Y;
  const uint16_t* R0;    // initial R per (b, h), nullable (zeros)
  uint16_t* Rout;        // final R per (b, h), nullable
  uint16_t* Bout;        // R after every full block, [B, nblk, H, dk*dv], nullable (forward only)
  const uint16_t* Bin;   // added to R before the chunk that ends each full block, nullable (reverse only)
  // Suffix tensors, [B, nblk + 1, Ls, H, d] in the roles of X, W, Z, Y (all four or none; Ls > 0
  // selects the suffix walk).  Tokens after the last block boundary are walked like any others;
  // Rout (forward) and R0 (reverse) then belong to the state at that boundary, nblk * block.
  const uint16_t* Xs;
  const uint16_t* Ws;
  const uint16_t* Zs;
  uint16_t* Ys;
  long long rs_a, rs_n;  // element strides of R[a][n] inside one dk*dv state matrix
  int B, T, H, dA, dB;
  int nblk;              // number of full blocks (T / block), 0 if block == 0
  int block;             // block size in tokens; chunks never straddle a multiple of it (0: none)
  int reverse;
  int Ls;                // tokens per suffix (walked in parts of CH); 0: no suffixes
  int state_only;        // only R is wanted (Rout per sequence): X is not read, Y not written, no read-out
  int slots;             // workgroups per (head, column tile); workgroup `slot` walks the batch entries
                         // slot, slot + slots, ... one after another.  0: the launcher chooses.
  float s_intra, s_read, s_update;
  float log2g[MAX_HEADS];
};

// What can differ between passes that share a launch: the tensors, the walking direction and the
// three scales.  Everything else in PassArgs (shape, walk, decays) is common to them.
struct PassTensors {
  const uint16_t *X, *W, *Z;
  uint16_t* Y;
  const uint16_t* R0;
  uint16_t *Rout, *Bout;
  const uint16_t *Bin, *Xs, *Ws, *Zs;
  uint16_t* Ys;
  long long rs_a, rs_n;
  int reverse;
  float s_intra, s_read, s_update;
};
#if defined(__HIPCC__)
#define FPK_HOST_DEVICE __host__ __device__
#else
#define FPK_HOST_DEVICE
#endif
FPK_HOST_DEVICE inline PassTensors tensors_of(const PassArgs& a) {
  return PassTensors{a.X,  a.W,  a.Z,  a.Y,    a.R0,   a.Rout,    a.Bout,    a.Bin,    a.Xs,
                     a.Ws, a.Zs, a.Ys, a.rs_a, a.rs_n, a.reverse, a.s_intra, a.s_read, a.s_update};
}

constexpr int MAX_PASSES_PER_LAUNCH = 3;

// Arguments of the segment scan that stitches a sequence cut into S segments back together.
// U[b][s] is the state a segment contributes on its own (zero initial state); with g = gamma^Tseg
//   init[b][0] = R0[b] (zeros if null),  init[b][s] = g init[b][s-1] + U[b][s-1],
//   fin[b] = g init[b][S-1] + U[b][S-1]
// `reverse` runs the same recurrence from the last segment to the first (state gradients).
// All matrices are bf16, M = dk * dv elements each, laid out [B, S, H, M] (U, init) and [B, H, M].
struct ScanArgs {
  const uint16_t* U;
  const uint16_t* R0;   // nullable
  uint16_t* init;
  uint16_t* fin;        // nullable
  int B, S, H, M, Tseg, reverse;
  float log2g[MAX_HEADS];
};
// State-only pass for states of 128 rows (segment_contrib.h): U[b][h] = what sequence b adds to a
// zero state, sum_j weight(j) W[j]^T Z[j] with weight(j) = s_update gamma^(T - 1 - j) walking forward
// (`reverse` = 0) and s_update gamma^(j + 1) walking backward.  W [B,T,H,128], Z [B,T,H,dB],
// U [B,H,128,dB], bf16; T a multiple of CH, dB a multiple of 128.
struct ContribArgs {
  const uint16_t* W;
  const uint16_t* Z;
  uint16_t* U;
  int B, T, H, dB, reverse;
  float s_update;
  float log2g[MAX_HEADS];
};
// One recurrent (decode) step for every (batch, head):  S' = gamma S + (scale k)^T v,  o = q S'.
// q, k [B,H,dk]; v, o [B,H,dv]; S [B,H,dk,dv]; all bf16, fp32 arithmetic.  s_out may be s_in.
struct DecodeArgs {
  const uint16_t* q;
  const uint16_t* k;
  const uint16_t* v;
  const uint16_t* s_in;   // nullable (zeros)
  uint16_t* s_out;
  uint16_t* o;
  int B, H, dk, dv;
  float scale;
  float gamma[MAX_HEADS];
};
// The fused backward for dk, dv of 64 or 128 (retention_bwd_fused.h): per (batch, head) stream one workgroup
// walks backward for dk, dv and d_s0 and one walks forward for dq.
constexpr int FB_D = 128;                  // the widest head dimension it takes
constexpr int FB_THREADS = 512;
constexpr int PACE_SLOTS = 4096;          // streams whose two workgroups of the fused backward can be paced
constexpr int SS_ROWS = 32;                // longest sequence of the backward for many short sequences (short_seq.h), which takes
                                           // the same arguments: q .. dv, s0, ds0, B, T, H, the head dimensions, scale, log2g
struct FusedBwdArgs {
  const uint16_t *q, *k, *v, *dO;          // q, k [B,T,H,dk_dim]; v, dO [B,T,H,dv_dim]
  uint16_t *dq, *dk, *dv;
  const uint16_t* s0;                      // [B,H,dk_dim,dv_dim], nullable (zeros)
  const uint16_t* ds_out;                  // gradient of the final state, nullable (zeros)
  uint16_t* ds0;                           // gradient of s0, nullable (not wanted)
  // States that the forward pass left behind every `ckpt_every` tokens (a multiple of 64):
  // ckpt[b][m][h] is the state after token (m + 1) * ckpt_every - 1, m < T / ckpt_every.  With them
  // the dq workgroup takes the segments between them from the last to the first (forward inside a
  // segment), next to the reverse workgroup of its stream, so that what one of the two fetches
  // the other finds in the caches.  Null: one forward walk from s0.
  const uint16_t* ckpt;
  int ckpt_every;
  // Pacing of the two workgroups of a stream (a measurement switch, off unless want_pace; needs checkpoints): the
  // reverse workgroup leaves pace_base + the number of chunks it has asked for in pace[stream], and the dq
  // workgroup holds back a segment's first loads until the reverse walk has reached that segment's last chunk, so
  // that the two cross inside the segment and the second read of its k, v, dO rows finds them in the L2.  A hint
  // only: the wait is bounded, nothing else depends on the word.  Measured on a 256-unit device at B8 H16 T4096
  // d128: the launch fetches 10 % (512-token segments) to 19 % (128) fewer bytes and takes 3 % to 7 % longer,
  // because it waits for the reverse workgroup's chain of chunk steps, not for bytes.
  int want_pace;
  uint32_t* pace;                          // set by the launcher (its own words), null: none
  uint32_t pace_base;
  // POP suffixes (block > 0; none of the above checkpoints then): one suffix of Ls <= 64 tokens per
  // block boundary 0, block, ..., T, tensors [B * (T / block + 1), Ls, H, d] as in PassArgs; block a
  // multiple of 64 that divides T.  A suffix reads the state at its boundary without advancing it.
  const uint16_t *q_sfx, *k_sfx, *v_sfx, *dO_sfx;
  uint16_t *dq_sfx, *dk_sfx, *dv_sfx;
  int block, Ls;
  int fold;                                // suffixes of at most 16 tokens: folded into the chunks at their boundaries (FB_FOLD), set by the launcher
  // POP block states (no suffixes, no checkpoints then): d_blocks[b][m][h] is the gradient of the state after token
  // (m + 1) * blocks_every - 1, m < T / blocks_every; blocks_every a multiple of 64.  The reverse walk adds it to dS
  // where it crosses that boundary.
  const uint16_t* d_blocks;
  int blocks_every;
  int B, T, H;
  int dk_dim, dv_dim;                      // head dimensions: 64 or 128 each
  float scale;                             // dk^-1/2
  float log2g[MAX_HEADS];
};
// Forward for many short sequences (short_seq.h): T <= SS_ROWS.
struct ShortFwdArgs {
  const uint16_t *q, *k, *v;               // q, k [B,T,H,dk_dim]; v [B,T,H,dv_dim]
  const uint16_t* s0;                      // [B,H,dk_dim,dv_dim], nullable (zeros)
  uint16_t* o;                             // [B,T,H,dv_dim]
  uint16_t* s_out;                         // [B,H,dk_dim,dv_dim], nullable (not wanted)
  int B, T, H;
  int dk_dim, dv_dim;                      // head dimensions: 64 or 128 each
  float scale;                             // dk^-1/2
  float log2g[MAX_HEADS];
};
constexpr int DECODE_THREADS = 256;
constexpr int decode_lds_bytes(int dv) { return (DECODE_THREADS / (dv / 8)) * dv * 4; }

constexpr int SCAN_THREADS = 256;
constexpr int SCAN_VEC = 8;   // elements per thread

// Rotary position embedding of q and k in one launch.  Pairs (x[2i], x[2i+1]) of every head are
// rotated by the angle float(position) * theta[i], `sign` = -1 rotates back (the gradient).
// q, k [B, T, H, d] bf16 (k nullable); the position of token t of sequence b is
// (start ? start[b] : start0) + t.  Output may alias input.
struct RotaryArgs {
  const uint16_t* q_in;
  const uint16_t* k_in;    // nullable, together with k_out
  uint16_t* q_out;
  uint16_t* k_out;
  const float* theta;      // [d / 2], device
  const long long* start;  // [B], device, nullable
  long long start0;
  int B, T, H, d;
  float sign;
  int heads_per_thread;    // set by plan_rotary: all H, or fewer when there are too few tokens to fill the device
};

// Per-head normalisation of the retention output followed by the swish gate:
//   n = bf16((r - mean) / sqrt(var + eps))  over the dv values of one (row, head), biased variance
//   out = bf16(n * bf16(g / (1 + exp(-g))))
// r [rows, H, dv], g and out [rows, H * dv], bf16; statistics in fp32.  The backward launch
// (d_out given) writes d_r and d_g instead of out.
struct GatedNormArgs {
  const uint16_t* r;
  const uint16_t* g;
  const uint16_t* d_out;   // backward only
  uint16_t* out;           // forward only
  uint16_t* d_r;           // backward only
  uint16_t* d_g;           // backward only
  long long groups;        // rows * H
  int dv;
  float eps;
};
constexpr int LAYER_THREADS = 256;

}  // namespace fpk

// Launches the pass kernel on `stream` (a hipStream_t, or ignored by the CPU test harness).
// Returns 0 on success; on failure returns nonzero and *err points at a static message.
int fpk_launch_pass(const fpk::PassArgs& args, void* stream, const char** err);

// Launches n <= MAX_PASSES_PER_LAUNCH independent passes over the same shape in one grid (they
// must be the same walk of the same shape; tensors, direction and scales may differ).  A pass that
// would leave part of the chip idle on its own runs beside the others, and passes that read the
// same rows in the same direction have the workgroups of a stream run side by side, so that those
// rows come from HBM once.
int fpk_launch_passes(const fpk::PassArgs* const* passes, int n, void* stream, const char** err);

// Launches the fused backward (2 B H workgroups).  Same conventions as fpk_launch_pass.
int fpk_launch_bwd_fused(const fpk::FusedBwdArgs& args, void* stream, const char** err);

// Launches the backward for many short sequences (short_seq.h: T <= 32, no gradient of the final state).
int fpk_launch_short_bwd(const fpk::FusedBwdArgs& args, void* stream, const char** err);
int fpk_launch_short_fwd(const fpk::ShortFwdArgs& args, void* stream, const char** err);

// Launches the segment scan.  Same conventions as fpk_launch_pass.
int fpk_launch_scan(const fpk::ScanArgs& args, void* stream, const char** err);

// Launches the state-only pass for states of 128 rows (B H dB / 128 workgroups).  Same conventions.
int fpk_launch_contrib(const fpk::ContribArgs& args, void* stream, const char** err);

// Bytes of the library's own scratch array (one per device, see fpk_static_scratch).
namespace fpk {
constexpr size_t STATIC_SCRATCH_BYTES = 16u << 20;
}
// Address of the scratch array on the current device (device memory, 256-byte aligned,
// fpk::STATIC_SCRATCH_BYTES long); looked up on the first call on each device, never allocated.
int fpk_static_scratch(void** ptr, const char** err);

// Nonzero if `stream` is recording a HIP graph (the CPU test harness: a flag that its tests set).
int fpk_stream_is_capturing(void* stream);

// Compute units of the current device (what the launcher sizes its grids against).
int fpk_compute_units();

// Launches the decode-step kernel.  Same conventions as fpk_launch_pass.
int fpk_launch_decode(const fpk::DecodeArgs& args, void* stream, const char** err);

// Launch the rotary kernel / the gated per-head normalisation (forward if a.out, else backward).
int fpk_launch_rotary(const fpk::RotaryArgs& args, void* stream, const char** err);
int fpk_launch_gated_norm(const fpk::GatedNormArgs& args, void* stream, const char** err);
