// C-ABI layer: argument checks and the mapping of retention forward / backward onto
// launches of the one pass kernel.  No device code and no HIP calls here.
//
// With s = dk^-1/2, A = s (q k^T) . D and P = s (dO v^T) . D (D the causal decay mask):
//
//   pass   X    W    Z    Y    R (dA x dB)        walk      s_intra s_read s_update
//   fwd    q    k    v    o    S      dk x dv     forward   s       1      s
//   dq     dO   v    k    dq   S^T    dv x dk     forward   s       1      s
//   dk     v    dO   q    dk   dS^T   dv x dk     backward  s       s      1
//   dv     k    q    dO   dv   dS     dk x dv     backward  s       s      1
//
// The column dimension dB is split over workgroups, the contraction dimension dA never is,
// so no pass needs a cross-workgroup reduction.  The dq pass re-runs the state recurrence
// instead of reading stored chunk states; the dk and dv passes each carry dS.  The three gradient
// passes are independent of each other and share launches where they fit (run_gradients).
//
// The POP entry points add block states to these passes (written by fwd, their gradients read
// by dk and dv); the fused POP entry points add the suffix tensors in the same four roles; the
// split entry points run the passes on segments of the sequences after a state-only pass and a
// scan; the decode step and the two elementwise stages around the op (rotary embedding of q and
// k, per-head normalisation with the swish gate) are kernels of their own.
#include "../../include/flashpop_hip.h"

#include <atomic>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <cstdint>
#include <cstdlib>
#include <mutex>

#include "pass_args.h"

namespace {

thread_local char g_err[256] = "";

int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof g_err, fmt, ap);
  va_end(ap);
  return code;
}

bool dim_ok(int d) { return d == 64 || d == 128 || d == 192 || d == 256; }

// Two measurement switches, read from the environment once per process (the first entry point that
// looks) and changed afterwards only through fp_set_backward_choice:
//   FLASHPOP_BWD   auto | passes | fused | paced   which backward runs where both exist (paced: fused, its two
//                  workgroups per stream held together, see FusedBwdArgs::want_pace)
//   FLASHPOP_CKPT  tokens between the checkpoints that the forward leaves for the fused backward
//                  (a multiple of 64; 0: none; unset: 512)
// A value that is neither is an error of every entry point, not a silent default.
enum BwdChoice { BWD_AUTO = 0, BWD_PASSES = 1, BWD_FUSED = 2, BWD_FUSED_PACED = 3 };
constexpr int kDefaultCheckpointEvery = 8 * fpk::CH;
std::atomic<int> g_bwd_choice{BWD_AUTO}, g_ckpt_every{kDefaultCheckpointEvery};
std::once_flag g_env_once;
char g_env_error[160] = "";

void read_environment() {
  std::call_once(g_env_once, [] {
    if (const char* e = std::getenv("FLASHPOP_BWD")) {
      if (std::strcmp(e, "passes") == 0) g_bwd_choice = BWD_PASSES;
      else if (std::strcmp(e, "fused") == 0) g_bwd_choice = BWD_FUSED;
      else if (std::strcmp(e, "paced") == 0) g_bwd_choice = BWD_FUSED_PACED;
      else if (std::strcmp(e, "auto") != 0 && *e)
        std::snprintf(g_env_error, sizeof g_env_error, "FLASHPOP_BWD=%.40s: expected auto, passes, fused or paced", e);
    }
    if (const char* e = std::getenv("FLASHPOP_CKPT")) {
      char* end = nullptr;
      const long n = std::strtol(e, &end, 10);
      if (end == e || *end || n < 0 || n % fpk::CH != 0 || n > (1 << 24))
        std::snprintf(g_env_error, sizeof g_env_error, "FLASHPOP_CKPT=%.40s: expected a non-negative multiple of %d", e, fpk::CH);
      else g_ckpt_every = (int)n;
    }
  });
}

struct Shape {
  int B, T, H, dk, dv;
};

int check_shape(const Shape& s, const double* decays) {
  read_environment();
  if (g_env_error[0]) return fail(FP_ERR_BAD_CONFIG, "%s", g_env_error);
  if (!decays) return fail(FP_ERR_NULL_POINTER, "head_decays is NULL");
  if (s.B < 1 || s.T < 1 || s.H < 1) return fail(FP_ERR_BAD_SHAPE, "B, T, H must be >= 1 (got %d, %d, %d)", s.B, s.T, s.H);
  if (s.H > fpk::MAX_HEADS) return fail(FP_ERR_BAD_SHAPE, "H = %d exceeds the supported maximum %d", s.H, fpk::MAX_HEADS);
  if (!dim_ok(s.dk) || !dim_ok(s.dv))
    return fail(FP_ERR_UNSUPPORTED_DIM, "dk and dv must be 64, 128, 192 or 256 (got dk=%d, dv=%d)", s.dk, s.dv);
  // per-tensor element counts are indexed with size_t in the kernel; the grid is an int
  // the kernels address one (batch, head) stream with 32-bit byte offsets
  const long long span = 2LL * s.T * s.H * (s.dk > s.dv ? s.dk : s.dv);
  if (span >= (1LL << 32)) return fail(FP_ERR_BAD_SHAPE, "T * H * max(dk, dv) too large: one sequence must stay below 4 GiB");
  // ... and a row of a tensor by a 32-bit index
  if ((long long)s.B * s.T >= (1LL << 32)) return fail(FP_ERR_BAD_SHAPE, "B * T too large: a tensor must have fewer than 2^32 rows");
  const long long wgs = (long long)s.B * s.H * ((s.dk > s.dv ? s.dk : s.dv) / fpk::BV);
  if (wgs > 0x7fffffffLL) return fail(FP_ERR_BAD_SHAPE, "B * H too large");
  for (int h = 0; h < s.H; ++h) {
    if (!(decays[h] > 0.0) || !(decays[h] <= 1.0))
      return fail(FP_ERR_BAD_DECAY, "head_decays[%d] = %g is outside (0, 1]", h, decays[h]);
  }
  return FP_OK;
}

// The pass kernels must not be recorded into a HIP graph (instantiating a graph that holds them has
// crashed the host process); the entry points that launch them refuse a capturing stream.
int check_stream(void* stream, const char* what) {
  if (fpk_stream_is_capturing(stream))
    return fail(FP_ERR_LAUNCH, "%s: the stream is capturing a HIP graph; this entry point must be called eagerly", what);
  return FP_OK;
}

void fill_common(fpk::PassArgs& a, const Shape& s, const double* decays) {
  std::memset(&a, 0, sizeof a);
  a.B = s.B;
  a.T = s.T;
  a.H = s.H;
  // log2(gamma) from the double, so gammas that round to 1.0f keep their decay
  for (int h = 0; h < s.H; ++h) a.log2g[h] = (float)std::log2(decays[h]);
}

bool misaligned(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) != 0; }
const uint16_t* in(const void* p) { return static_cast<const uint16_t*>(p); }
uint16_t* out(void* p) { return static_cast<uint16_t*>(p); }

int run(const fpk::PassArgs& a, void* stream, const char* what) {
  const char* msg = "";
  if (fpk_launch_pass(a, stream, &msg) != 0) return fail(FP_ERR_LAUNCH, "%s pass: %s", what, msg);
  return FP_OK;
}

// Independent passes over the same shape may share a launch (fpk_launch_passes).
bool same_launch(const fpk::PassArgs& x, const fpk::PassArgs& y) {
  return x.dA == y.dA && x.dB == y.dB && x.block == y.block && x.nblk == y.nblk && x.Ls == y.Ls &&
         (x.Bin != nullptr || x.Bout != nullptr) == (y.Bin != nullptr || y.Bout != nullptr);
}

int run_together(const fpk::PassArgs* const* passes, int n, void* stream, const char* what) {
  const char* msg = "";
  if (fpk_launch_passes(passes, n, stream, &msg) != 0) return fail(FP_ERR_LAUNCH, "%s passes: %s", what, msg);
  return FP_OK;
}

// The three gradient passes do not depend on each other.  How they are grouped into launches:
//  - dk and dv read the same q and dO rows walking backward; with dk == dv they are the same
//    kernel with the same grid, and in one launch the workgroups of a stream in both passes run
//    side by side, so those rows come from HBM once;
//  - dq has the shape of the dk pass.  Where one pass alone leaves compute units idle it joins
//    that launch (it walks the other way, so nothing is shared but the chip);
//  - what does not fit together (different dk and dv; block states in dk and dv but not in dq)
//    is launched on its own.
int run_gradients(const fpk::PassArgs& dq, const fpk::PassArgs& dk, const fpk::PassArgs& dv, void* stream,
                  const char* what) {
  const long long alone = (long long)dk.B * dk.H * (dk.dB / fpk::BV);   // workgroups of one pass
  const bool fills = alone >= fpk_compute_units();
  const bool dq_dk = same_launch(dq, dk), dk_dv = same_launch(dk, dv);
  if (dq_dk && dk_dv && !fills) {
    const fpk::PassArgs* all[] = {&dk, &dv, &dq};
    return run_together(all, 3, stream, what);
  }
  if (dk_dv) {
    if (int rc = run(dq, stream, what)) return rc;
    const fpk::PassArgs* both[] = {&dk, &dv};
    return run_together(both, 2, stream, what);
  }
  if (dq_dk && !fills) {
    const fpk::PassArgs* both[] = {&dq, &dk};
    if (int rc = run_together(both, 2, stream, what)) return rc;
    return run(dv, stream, what);
  }
  if (int rc = run(dq, stream, what)) return rc;
  if (int rc = run(dk, stream, what)) return rc;
  return run(dv, stream, what);
}

// dk and dv alone (the split-sequence backward runs its dq earlier)
int run_dk_dv(const fpk::PassArgs& dk, const fpk::PassArgs& dv, void* stream, const char* what) {
  if (same_launch(dk, dv)) {
    const fpk::PassArgs* both[] = {&dk, &dv};
    return run_together(both, 2, stream, what);
  }
  if (int rc = run(dk, stream, what)) return rc;
  return run(dv, stream, what);
}

// R = S, dk x dv, rows contiguous in dv
void plain_state(fpk::PassArgs& a, const Shape& s) {
  a.dA = s.dk;
  a.dB = s.dv;
  a.rs_a = s.dv;
  a.rs_n = 1;
}
// R = S^T, dv x dk, read through the strides of S
void transposed_state(fpk::PassArgs& a, const Shape& s) {
  a.dA = s.dv;
  a.dB = s.dk;
  a.rs_a = 1;
  a.rs_n = s.dv;
}

// Sequences of at most fpk::SS_ROWS tokens with head dimensions of 64 or 128: the forward that takes a (sequence,
// head) pair per step (short_seq.h) instead of a 64-token item per pair and column tile.  Shares the switch of the
// backward (the pass kernel stays reachable for comparisons).
bool fused_dim(int d);
bool use_short_forward(const Shape& s) {
  if (s.T > fpk::SS_ROWS || !fused_dim(s.dk) || !fused_dim(s.dv)) return false;
  read_environment();
  return g_bwd_choice.load(std::memory_order_relaxed) != BWD_PASSES;
}

int forward_short(const Shape& s, const void* q, const void* k, const void* v, const void* s0, const double* decays, void* o,
                  void* s_out, void* stream) {
  fpk::ShortFwdArgs a;
  std::memset(&a, 0, sizeof a);
  a.q = in(q); a.k = in(k); a.v = in(v); a.s0 = in(s0);
  a.o = out(o); a.s_out = out(s_out);
  a.B = s.B; a.T = s.T; a.H = s.H;
  a.dk_dim = s.dk; a.dv_dim = s.dv;
  a.scale = 1.0f / std::sqrt((float)s.dk);
  for (int h = 0; h < s.H; ++h) a.log2g[h] = (float)std::log2(decays[h]);
  const char* msg = "";
  if (fpk_launch_short_fwd(a, stream, &msg) != 0) return fail(FP_ERR_LAUNCH, "short-sequence forward: %s", msg);
  return FP_OK;
}

int forward(const Shape& s, const void* q, const void* k, const void* v, const void* s0, const double* decays, void* o,
            void* s_out, void* block_states, int block, void* stream) {
  if (!block_states && block == 0 && use_short_forward(s)) return forward_short(s, q, k, v, s0, decays, o, s_out, stream);
  fpk::PassArgs a;
  fill_common(a, s, decays);
  const float sc = 1.0f / std::sqrt((float)s.dk);
  a.X = in(q); a.W = in(k); a.Z = in(v); a.Y = out(o);
  a.R0 = in(s0); a.Rout = out(s_out); a.Bout = out(block_states);
  plain_state(a, s);
  a.block = block;
  a.nblk = block > 0 ? s.T / block : 0;
  a.reverse = 0;
  a.s_intra = sc; a.s_read = 1.f; a.s_update = sc;
  return run(a, stream, "forward");
}

// The plain backward with dk and dv of 64 or 128 has a kernel of its own that reads q, k, v, dO once for dk
// and dv together (retention_bwd_fused.h); it runs two workgroups per (batch, head) stream, so it
// is chosen when there are enough streams for the device (below).  The backward choice (FLASHPOP_BWD,
// fp_set_backward_choice) overrides that (for A/B measurements).
bool fused_dim(int d) { return d == 64 || d == 128; }
// `d_blocks` with `block`: gradients of POP block states arrive; the kernel adds them on its way when the blocks are
// whole chunks.
bool use_fused_backward(const Shape& s, const void* d_blocks, bool pop_suffixes = false, int block = 0) {
  if (!fused_dim(s.dk) || !fused_dim(s.dv)) return false;
  if (d_blocks && (block <= 0 || block % fpk::CH != 0)) return false;
  read_environment();
  const int choice = g_bwd_choice.load(std::memory_order_relaxed);
  if (choice == BWD_PASSES) return false;
  if (choice >= BWD_FUSED) return true;   // whatever the length and the number of streams
  if (s.T < 8 * fpk::CH) return false;    // short sequences: the walk over many of them per workgroup serves better
  // Two workgroups per stream against column-tiled passes that fill the chip: the fused kernel needs enough streams.
  // Measured cross-overs on a 256-unit device (forward + backward at T = 2048 .. 4096; streams = B * H):
  //                 dk = dv = 128      dk 64, dv 128      dk 128, dv 64      dk = dv = 64
  //   plain         86  (3 s >= CU)    32  (8 s >= CU)    64  (4 s >= CU)    64  (4 s >= CU)
  //   POP suffixes  48  (16 s >= 3 CU) 32  (8 s >= CU)    32  (8 s >= CU)    96  (8 s >= 3 CU)
  // (d = 128, 64 streams: 0.33 ms fused against 0.30 ms in passes at T = 4096; with suffixes the passes pay for every
  // suffix as a stop of each of their four walks and this kernel does not: 48 streams, 64-token blocks, 0.44 against
  // 0.57 ms.  Narrower states make the fused kernel's chunk step cheaper sooner than they help the passes.)
  const long long streams = (long long)s.B * s.H, cu = fpk_compute_units();
  const bool wide = s.dk == fpk::FB_D && s.dv == fpk::FB_D, narrow = s.dk == 64 && s.dv == 64;
  if (pop_suffixes) return wide ? 16 * streams >= 3 * cu : narrow ? 8 * streams >= 3 * cu : 8 * streams >= cu;
  return wide ? 3 * streams >= cu : s.dk == 64 && s.dv == fpk::FB_D ? 8 * streams >= cu : 4 * streams >= cu;
}

// Tokens between the states that fp_retention_fwd_ckpt leaves for the backward (0: none wanted).
// Eight chunks: the checkpoints cost 1/16 of the forward's traffic, and the segment that the two
// workgroups of a stream share stays within reach of the caches.
int checkpoint_interval(const Shape& s) {
  read_environment();
  const int every = g_ckpt_every.load(std::memory_order_relaxed);
  if (every <= 0 || !use_fused_backward(s, nullptr) || s.T <= every) return 0;
  return every;
}

// Suffix tensors of one fused POP call, in the roles q, k, v / d_o (inputs) and o / dq, dk, dv (outputs)
struct Suffixes {
  const void *q, *k, *v;
  int len;
};
struct SuffixGrads {
  const void* d_o;
  void *dq, *dk, *dv;
  int block;
};

int backward_fused(const Shape& s, const void* q, const void* k, const void* v, const void* s0, const double* decays,
                   const void* d_o, const void* d_s_out, void* dq, void* dk_, void* dv_, void* d_s0, void* stream,
                   const void* ckpt = nullptr, int ckpt_every = 0, const Suffixes* sfx = nullptr,
                   const SuffixGrads* sg = nullptr, const void* d_blocks = nullptr, int blocks_every = 0) {
  fpk::FusedBwdArgs a;
  std::memset(&a, 0, sizeof a);
  a.d_blocks = in(d_blocks);
  a.blocks_every = d_blocks ? blocks_every : 0;
  a.ckpt = in(ckpt);
  a.ckpt_every = ckpt ? ckpt_every : 0;
  a.want_pace = g_bwd_choice.load(std::memory_order_relaxed) == BWD_FUSED_PACED;
  if (sfx) {
    a.q_sfx = in(sfx->q); a.k_sfx = in(sfx->k); a.v_sfx = in(sfx->v); a.dO_sfx = in(sg->d_o);
    a.dq_sfx = out(sg->dq); a.dk_sfx = out(sg->dk); a.dv_sfx = out(sg->dv);
    a.block = sg->block;
    a.Ls = sfx->len;
  }
  a.q = in(q); a.k = in(k); a.v = in(v); a.dO = in(d_o);
  a.dq = out(dq); a.dk = out(dk_); a.dv = out(dv_);
  a.s0 = in(s0); a.ds_out = in(d_s_out); a.ds0 = out(d_s0);
  a.B = s.B; a.T = s.T; a.H = s.H;
  a.dk_dim = s.dk; a.dv_dim = s.dv;
  a.scale = 1.0f / std::sqrt((float)s.dk);
  for (int h = 0; h < s.H; ++h) a.log2g[h] = (float)std::log2(decays[h]);
  const char* msg = "";
  if (fpk_launch_bwd_fused(a, stream, &msg) != 0) return fail(FP_ERR_LAUNCH, "fused backward: %s", msg);
  return FP_OK;
}

// Many short sequences that each read a state of their own and whose final states nobody differentiates (the
// suffix call of the reference's POP layer): one kernel that takes a (sequence, head) pair per step (short_seq.h)
// instead of a 64-token item per pass and pair.
bool use_short_backward(const Shape& s, const void* d_s_out, const void* d_blocks) {
  if (s.T > fpk::SS_ROWS || d_s_out || d_blocks || !fused_dim(s.dk) || !fused_dim(s.dv)) return false;
  read_environment();
  return g_bwd_choice.load(std::memory_order_relaxed) != BWD_PASSES;
}

int backward_short(const Shape& s, const void* q, const void* k, const void* v, const void* s0, const double* decays,
                   const void* d_o, void* dq, void* dk_, void* dv_, void* d_s0, void* stream) {
  fpk::FusedBwdArgs a;
  std::memset(&a, 0, sizeof a);
  a.q = in(q); a.k = in(k); a.v = in(v); a.dO = in(d_o);
  a.dq = out(dq); a.dk = out(dk_); a.dv = out(dv_);
  a.s0 = in(s0); a.ds0 = out(d_s0);
  a.B = s.B; a.T = s.T; a.H = s.H;
  a.dk_dim = s.dk; a.dv_dim = s.dv;
  a.scale = 1.0f / std::sqrt((float)s.dk);
  for (int h = 0; h < s.H; ++h) a.log2g[h] = (float)std::log2(decays[h]);
  const char* msg = "";
  if (fpk_launch_short_bwd(a, stream, &msg) != 0) return fail(FP_ERR_LAUNCH, "short-sequence backward: %s", msg);
  return FP_OK;
}

int backward(const Shape& s, const void* q, const void* k, const void* v, const void* s0, const double* decays,
             const void* d_o, const void* d_s_out, const void* d_blocks, int block, void* dq, void* dk_, void* dv_,
             void* d_s0, void* stream) {
  if (use_short_backward(s, d_s_out, d_blocks)) return backward_short(s, q, k, v, s0, decays, d_o, dq, dk_, dv_, d_s0, stream);
  if (use_fused_backward(s, d_blocks, false, block) && !(d_blocks && d_s_out))
    return backward_fused(s, q, k, v, s0, decays, d_o, d_s_out, dq, dk_, dv_, d_s0, stream, nullptr, 0, nullptr, nullptr,
                          d_blocks, block);
  const float sc = 1.0f / std::sqrt((float)s.dk);
  const int nblk = block > 0 ? s.T / block : 0;
  fpk::PassArgs g, a;

  fill_common(g, s, decays);   // dq
  g.X = in(d_o); g.W = in(v); g.Z = in(k); g.Y = out(dq);
  g.R0 = in(s0);
  transposed_state(g, s);
  g.reverse = 0;
  g.s_intra = sc; g.s_read = 1.f; g.s_update = sc;

  fill_common(a, s, decays);   // dk
  a.X = in(v); a.W = in(d_o); a.Z = in(q); a.Y = out(dk_);
  a.R0 = in(d_s_out); a.Bin = in(d_blocks);
  transposed_state(a, s);
  a.block = d_blocks ? block : 0; a.nblk = nblk;
  a.reverse = 1;
  a.s_intra = sc; a.s_read = sc; a.s_update = 1.f;

  fpk::PassArgs b;
  fill_common(b, s, decays);   // dv (+ d_s0)
  b.X = in(k); b.W = in(q); b.Z = in(d_o); b.Y = out(dv_);
  b.R0 = in(d_s_out); b.Bin = in(d_blocks); b.Rout = out(d_s0);
  plain_state(b, s);
  b.block = d_blocks ? block : 0; b.nblk = nblk;
  b.reverse = 1;
  b.s_intra = sc; b.s_read = sc; b.s_update = 1.f;
  return run_gradients(g, a, b, stream, "gradient");
}

// ---- long sequences, few streams: cut every sequence into segments ---------------------------
// One workgroup walks one (batch, head, column tile) stream from end to end, so B * H * tiles
// workgroups is all the parallelism a pass has.  When that leaves most of the chip idle, each
// sequence is cut into S equal segments that run as separate sequences:
//   1. a state-only pass gives the state each segment contributes on its own,
//   2. a scan over the S contributions gives the state at the start of every segment,
//   3. the ordinary pass runs on B * S sequences from those states.
// The backward does the same for S (needed by the dq pass; recomputed, not stored) and, walking
// backward, for dS.  Segment states pass through bf16 like POP block states do.

// Number of segments per sequence (1: do not cut) for a call whose narrowest pass has
// `tiles` column tiles per stream.  Cutting costs an extra state-only pass per recurrence, so it
// is done only when the uncut call would leave at least two thirds of the compute units idle.
int plan_segments(const Shape& s, int tiles) {
  constexpr int kMinChunks = 4;                 // shortest segment worth a workgroup of its own
  if (s.T % fpk::CH != 0) return 1;
  const int chunks = s.T / fpk::CH;
  const long long streams = (long long)s.B * s.H * tiles;
  const long long target = fpk_compute_units() / streams;   // segments that fill the chip once
  if (target < 3) return 1;
  int best = 1;
  for (int n = 2; n <= target && n <= chunks; ++n) {
    if (chunks % n == 0 && chunks / n >= kMinChunks) best = n;
  }
  return best;
}
// Forward and backward cut a sequence the same way (the backward's narrowest pass has the fewest
// column tiles and decides), so that the states the forward leaves at the start of every segment
// are the ones the backward's dq pass needs.
int plan_split(const Shape& s) { return plan_segments(s, (s.dk < s.dv ? s.dk : s.dv) / fpk::BV); }
int plan_forward(const Shape& s) { return plan_split(s); }
int plan_backward(const Shape& s) { return plan_split(s); }

size_t workspace_bytes(const Shape& s, int segments) {
  return segments > 1 ? 2 * sizeof(uint16_t) * (size_t)s.B * segments * s.H * s.dk * s.dv : 0;
}

struct Workspace {
  uint16_t* contrib;   // [B, S, H, dk, dv]: what each segment adds on its own
  uint16_t* start;     // [B, S, H, dk, dv]: state at the segment's first token (last, walking backward)
};

Workspace carve(void* workspace, const Shape& s, int segments) {
  uint16_t* base = static_cast<uint16_t*>(workspace);
  return Workspace{base, base + (size_t)s.B * segments * s.H * s.dk * s.dv};
}

int scan(const Shape& s, int segments, const double* decays, const Workspace& w, const void* r0, void* fin, int reverse,
         void* stream) {
  fpk::ScanArgs a;
  std::memset(&a, 0, sizeof a);
  a.U = w.contrib; a.R0 = in(r0); a.init = w.start; a.fin = out(fin);
  a.B = s.B; a.S = segments; a.H = s.H; a.M = s.dk * s.dv; a.Tseg = s.T / segments; a.reverse = reverse;
  for (int h = 0; h < s.H; ++h) a.log2g[h] = (float)std::log2(decays[h]);
  const char* msg = "";
  if (fpk_launch_scan(a, stream, &msg) != 0) return fail(FP_ERR_LAUNCH, "segment scan: %s", msg);
  return FP_OK;
}

// the B * S sequences of T / S tokens that the segments form (the same memory, reinterpreted)
Shape segment_shape(const Shape& s, int segments) { return Shape{s.B * segments, s.T / segments, s.H, s.dk, s.dv}; }

// State-only pass: contributions of the segments to S (forward walk over k, v) or to dS
// (backward walk over q, dO).
int contributions(const Shape& seg, const double* decays, const void* w_rows, const void* z_rows, int reverse,
                  const Workspace& w, void* stream) {
  const float sc = 1.0f / std::sqrt((float)seg.dk);
  if (seg.dk == fpk::FB_D && seg.dv % fpk::FB_D == 0) {   // the kernel that holds 128 x 128 of the state per workgroup
    fpk::ContribArgs c;
    std::memset(&c, 0, sizeof c);
    c.W = in(w_rows); c.Z = in(z_rows); c.U = w.contrib;
    c.B = seg.B; c.T = seg.T; c.H = seg.H; c.dB = seg.dv; c.reverse = reverse;
    c.s_update = reverse ? 1.f : sc;
    for (int h = 0; h < seg.H; ++h) c.log2g[h] = (float)std::log2(decays[h]);
    const char* msg = "";
    if (fpk_launch_contrib(c, stream, &msg) != 0) return fail(FP_ERR_LAUNCH, "%s: %s", reverse ? "dS contributions" : "S contributions", msg);
    return FP_OK;
  }
  fpk::PassArgs a;
  fill_common(a, seg, decays);
  a.X = in(w_rows);   // never read
  a.W = in(w_rows); a.Z = in(z_rows);
  a.Rout = w.contrib;
  plain_state(a, seg);
  a.reverse = reverse;
  a.state_only = 1;
  a.s_intra = sc; a.s_read = reverse ? sc : 1.f; a.s_update = reverse ? 1.f : sc;
  return run(a, stream, reverse ? "dS contributions" : "S contributions");
}

int forward_split(const Shape& s, int segments, const void* q, const void* k, const void* v, const void* s0,
                  const double* decays, void* o, void* s_out, void* workspace, void* stream) {
  const Shape seg = segment_shape(s, segments);
  const Workspace w = carve(workspace, s, segments);
  int rc;
  if ((rc = contributions(seg, decays, k, v, 0, w, stream)) != FP_OK) return rc;
  if ((rc = scan(s, segments, decays, w, s0, s_out, 0, stream)) != FP_OK) return rc;
  return forward(seg, q, k, v, w.start, decays, o, nullptr, nullptr, 0, stream);
}

int backward_split(const Shape& s, int segments, const void* q, const void* k, const void* v, const void* s0,
                   const double* decays, const void* d_o, const void* d_s_out, void* dq, void* dk_, void* dv_,
                   void* d_s0, void* workspace, bool states_kept, void* stream) {
  const Shape seg = segment_shape(s, segments);
  const Workspace w = carve(workspace, s, segments);
  const float sc = 1.0f / std::sqrt((float)s.dk);
  fpk::PassArgs a;
  int rc;

  // S at the start of every segment (unless the forward's are still there), then dq
  if (!states_kept) {
    if ((rc = contributions(seg, decays, k, v, 0, w, stream)) != FP_OK) return rc;
    if ((rc = scan(s, segments, decays, w, s0, nullptr, 0, stream)) != FP_OK) return rc;
  }
  fill_common(a, seg, decays);
  a.X = in(d_o); a.W = in(v); a.Z = in(k); a.Y = out(dq);
  a.R0 = w.start;
  transposed_state(a, seg);
  a.reverse = 0;
  a.s_intra = sc; a.s_read = 1.f; a.s_update = sc;
  if ((rc = run(a, stream, "dq")) != FP_OK) return rc;

  // dS at the end of every segment (the workspace is free again: the stream orders the passes), then dk and dv
  if ((rc = contributions(seg, decays, q, d_o, 1, w, stream)) != FP_OK) return rc;
  if ((rc = scan(s, segments, decays, w, d_s_out, d_s0, 1, stream)) != FP_OK) return rc;
  fill_common(a, seg, decays);
  a.X = in(v); a.W = in(d_o); a.Z = in(q); a.Y = out(dk_);
  a.R0 = w.start;
  transposed_state(a, seg);
  a.reverse = 1;
  a.s_intra = sc; a.s_read = sc; a.s_update = 1.f;

  fpk::PassArgs b;
  fill_common(b, seg, decays);
  b.X = in(k); b.W = in(q); b.Z = in(d_o); b.Y = out(dv_);
  b.R0 = w.start;
  plain_state(b, seg);
  b.reverse = 1;
  b.s_intra = sc; b.s_read = sc; b.s_update = 1.f;
  return run_dk_dv(a, b, stream, "dk / dv");
}

int check_workspace(const Shape& s, int segments, const void* workspace, size_t bytes) {
  if (segments <= 1) return FP_OK;
  if (!workspace) return fail(FP_ERR_NULL_POINTER, "workspace is NULL but fp_retention_workspace_bytes() is nonzero for this shape");
  if (bytes < workspace_bytes(s, segments))
    return fail(FP_ERR_BAD_SHAPE, "workspace of %zu bytes is smaller than the %zu that fp_retention_workspace_bytes() asks for",
                bytes, workspace_bytes(s, segments));
  if (reinterpret_cast<uintptr_t>(workspace) % 16 != 0) return fail(FP_ERR_BAD_SHAPE, "workspace must be 16-byte aligned");
  return FP_OK;
}

int check_fused(const Shape& s, int block, int sfx_len) {
  if (block < 1) return fail(FP_ERR_BAD_SHAPE, "block_size must be >= 1 (got %d)", block);
  if (sfx_len < 1) return fail(FP_ERR_BAD_SHAPE, "suffix length must be positive (got %d)", sfx_len);
  if (sfx_len > fpk::CH && (s.dk > 128 || s.dv > 128))
    return fail(FP_ERR_UNSUPPORTED_DIM, "suffixes longer than %d tokens need dk and dv of 64 or 128 (got %d, %d)", fpk::CH, s.dk, s.dv);
  if ((long long)s.B * (s.T / block + 1) * sfx_len >= (1LL << 32))
    return fail(FP_ERR_BAD_SHAPE, "too many suffix rows: B * (T / block_size + 1) * sfx_len must stay below 2^32");
  return FP_OK;
}

void suffix_walk(fpk::PassArgs& a, const Shape& s, int block, int sfx_len, const void* x, const void* w, const void* z,
                 void* y) {
  a.block = block;
  a.nblk = s.T / block;
  a.Ls = sfx_len;
  a.Xs = in(x); a.Ws = in(w); a.Zs = in(z); a.Ys = out(y);
}

int fused_forward(const Shape& s, const void* q, const void* k, const void* v, const void* s0, const Suffixes& x,
                  const double* decays, void* o, void* o_sfx, void* s_out, int block, void* stream) {
  fpk::PassArgs a;
  fill_common(a, s, decays);
  const float sc = 1.0f / std::sqrt((float)s.dk);
  a.X = in(q); a.W = in(k); a.Z = in(v); a.Y = out(o);
  a.R0 = in(s0); a.Rout = out(s_out);
  plain_state(a, s);
  suffix_walk(a, s, block, x.len, x.q, x.k, x.v, o_sfx);
  a.reverse = 0;
  a.s_intra = sc; a.s_read = 1.f; a.s_update = sc;
  return run(a, stream, "fused forward");
}

int fused_backward(const Shape& s, const void* q, const void* k, const void* v, const void* s0, const Suffixes& x,
                   const double* decays, const void* d_o, const void* d_o_sfx, const void* d_s_out, void* dq, void* dk_,
                   void* dv_, void* dq_sfx, void* dk_sfx, void* dv_sfx, void* d_s0, int block, void* stream) {
  // whole 64-token chunks per block, suffixes of one chunk at most: the kernel that carries dS once
  if (use_fused_backward(s, nullptr, true) && block % fpk::CH == 0 && s.T % block == 0 && x.len <= fpk::CH) {
    const SuffixGrads sg{d_o_sfx, dq_sfx, dk_sfx, dv_sfx, block};
    return backward_fused(s, q, k, v, s0, decays, d_o, d_s_out, dq, dk_, dv_, d_s0, stream, nullptr, 0, &x, &sg);
  }
  const float sc = 1.0f / std::sqrt((float)s.dk);
  fpk::PassArgs g, a;

  fill_common(g, s, decays);   // dq
  g.X = in(d_o); g.W = in(v); g.Z = in(k); g.Y = out(dq);
  g.R0 = in(s0);
  transposed_state(g, s);
  suffix_walk(g, s, block, x.len, d_o_sfx, x.v, x.k, dq_sfx);
  g.reverse = 0;
  g.s_intra = sc; g.s_read = 1.f; g.s_update = sc;

  fill_common(a, s, decays);   // dk
  a.X = in(v); a.W = in(d_o); a.Z = in(q); a.Y = out(dk_);
  a.R0 = in(d_s_out);
  transposed_state(a, s);
  suffix_walk(a, s, block, x.len, x.v, d_o_sfx, x.q, dk_sfx);
  a.reverse = 1;
  a.s_intra = sc; a.s_read = sc; a.s_update = 1.f;

  fpk::PassArgs b;
  fill_common(b, s, decays);   // dv (+ d_s0)
  b.X = in(k); b.W = in(q); b.Z = in(d_o); b.Y = out(dv_);
  b.R0 = in(d_s_out); b.Rout = out(d_s0);
  plain_state(b, s);
  suffix_walk(b, s, block, x.len, x.k, x.q, d_o_sfx, dv_sfx);
  b.reverse = 1;
  b.s_intra = sc; b.s_read = sc; b.s_update = 1.f;
  return run_gradients(g, a, b, stream, "fused gradient");
}

}  // namespace

extern "C" {

int fp_retention_fwd(const void* q, const void* k, const void* v, const void* s0, const double* head_decays, void* o,
                     void* s_out, int B, int T, int H, int dk, int dv, void* stream) {
  const Shape s{B, T, H, dk, dv};
  if (int rc = check_shape(s, head_decays)) return rc;
  if (int rc = check_stream(stream, "fp_retention_fwd")) return rc;
  if (!q || !k || !v || !o) return fail(FP_ERR_NULL_POINTER, "q, k, v and o must not be NULL");
  return forward(s, q, k, v, s0, head_decays, o, s_out, nullptr, 0, stream);
}

int fp_retention_bwd(const void* q, const void* k, const void* v, const void* s0, const double* head_decays,
                     const void* d_o, const void* d_s_out, void* dq, void* dk_, void* dv_, void* d_s0, int B, int T,
                     int H, int dk, int dv, void* stream) {
  const Shape s{B, T, H, dk, dv};
  if (int rc = check_shape(s, head_decays)) return rc;
  if (int rc = check_stream(stream, "fp_retention_bwd")) return rc;
  if (!q || !k || !v || !d_o || !dq || !dk_ || !dv_)
    return fail(FP_ERR_NULL_POINTER, "q, k, v, d_o, dq, dk and dv must not be NULL");
  return backward(s, q, k, v, s0, head_decays, d_o, d_s_out, nullptr, 0, dq, dk_, dv_, d_s0, stream);
}

size_t fp_retention_checkpoint_bytes(int B, int T, int H, int dk, int dv, int* every) {
  const Shape s{B, T, H, dk, dv};
  if (every) *every = 0;
  if (B < 1 || T < 1 || H < 1 || H > fpk::MAX_HEADS || !dim_ok(dk) || !dim_ok(dv)) return 0;
  const int n = checkpoint_interval(s);
  if (n <= 0) return 0;
  if (every) *every = n;
  return sizeof(uint16_t) * (size_t)B * (T / n) * H * dk * dv;
}

int fp_retention_fwd_ckpt(const void* q, const void* k, const void* v, const void* s0, const double* head_decays, void* o,
                          void* s_out, void* checkpoints, int every, int B, int T, int H, int dk, int dv, void* stream) {
  const Shape s{B, T, H, dk, dv};
  if (int rc = check_shape(s, head_decays)) return rc;
  if (int rc = check_stream(stream, "fp_retention_fwd_ckpt")) return rc;
  if (!q || !k || !v || !o) return fail(FP_ERR_NULL_POINTER, "q, k, v and o must not be NULL");
  if (!checkpoints || every <= 0) return forward(s, q, k, v, s0, head_decays, o, s_out, nullptr, 0, stream);
  if (every % fpk::CH != 0) return fail(FP_ERR_BAD_SHAPE, "the checkpoint interval must be a multiple of %d tokens (got %d)", fpk::CH, every);
  return forward(s, q, k, v, s0, head_decays, o, s_out, T / every > 0 ? checkpoints : nullptr, every, stream);
}

int fp_retention_bwd_ckpt(const void* q, const void* k, const void* v, const void* s0, const double* head_decays,
                          const void* d_o, const void* d_s_out, const void* checkpoints, int every, void* dq, void* dk_,
                          void* dv_, void* d_s0, int B, int T, int H, int dk, int dv, void* stream) {
  const Shape s{B, T, H, dk, dv};
  if (int rc = check_shape(s, head_decays)) return rc;
  if (int rc = check_stream(stream, "fp_retention_bwd_ckpt")) return rc;
  if (!q || !k || !v || !d_o || !dq || !dk_ || !dv_)
    return fail(FP_ERR_NULL_POINTER, "q, k, v, d_o, dq, dk and dv must not be NULL");
  if (checkpoints && (every <= 0 || every % fpk::CH != 0))
    return fail(FP_ERR_BAD_SHAPE, "the checkpoint interval must be a positive multiple of %d tokens (got %d)", fpk::CH, every);
  if (checkpoints && T / every > 0 && use_fused_backward(s, nullptr))
    return backward_fused(s, q, k, v, s0, head_decays, d_o, d_s_out, dq, dk_, dv_, d_s0, stream, checkpoints, every);
  return backward(s, q, k, v, s0, head_decays, d_o, d_s_out, nullptr, 0, dq, dk_, dv_, d_s0, stream);
}

size_t fp_retention_workspace_bytes(int B, int T, int H, int dk, int dv) {
  const Shape s{B, T, H, dk, dv};
  if (B < 1 || T < 1 || H < 1 || H > fpk::MAX_HEADS || !dim_ok(dk) || !dim_ok(dv)) return 0;
  const int fwd = plan_forward(s), bwd = plan_backward(s);
  return workspace_bytes(s, fwd > bwd ? fwd : bwd);
}

int fp_retention_fwd_split(const void* q, const void* k, const void* v, const void* s0, const double* head_decays,
                           void* o, void* s_out, int B, int T, int H, int dk, int dv, void* workspace,
                           size_t workspace_bytes_given, void* stream) {
  const Shape s{B, T, H, dk, dv};
  if (int rc = check_shape(s, head_decays)) return rc;
  if (int rc = check_stream(stream, "fp_retention_fwd_split")) return rc;
  if (!q || !k || !v || !o) return fail(FP_ERR_NULL_POINTER, "q, k, v and o must not be NULL");
  const int segments = plan_forward(s);
  if (int rc = check_workspace(s, segments, workspace, workspace_bytes_given)) return rc;
  if (segments <= 1) return forward(s, q, k, v, s0, head_decays, o, s_out, nullptr, 0, stream);
  return forward_split(s, segments, q, k, v, s0, head_decays, o, s_out, workspace, stream);
}

int fp_retention_fwd_split_static(const void* q, const void* k, const void* v, const void* s0,
                                  const double* head_decays, void* o, void* s_out, int B, int T, int H, int dk, int dv,
                                  void* stream) {
  const Shape s{B, T, H, dk, dv};
  if (int rc = check_shape(s, head_decays)) return rc;
  if (int rc = check_stream(stream, "fp_retention_fwd_split_static")) return rc;
  if (!q || !k || !v || !o) return fail(FP_ERR_NULL_POINTER, "q, k, v and o must not be NULL");
  const int segments = plan_forward(s);
  if (segments <= 1) return forward(s, q, k, v, s0, head_decays, o, s_out, nullptr, 0, stream);
  const size_t need = workspace_bytes(s, segments);
  if (need > fpk::STATIC_SCRATCH_BYTES)
    return fail(FP_ERR_BAD_SHAPE,
                "this shape needs %zu bytes of segment states, more than the %zu bytes of the library's own scratch: "
                "use fp_retention_fwd_split with a workspace",
                need, (size_t)fpk::STATIC_SCRATCH_BYTES);
  void* scratch_ptr = nullptr;
  const char* msg = "";
  if (fpk_static_scratch(&scratch_ptr, &msg) != 0) return fail(FP_ERR_LAUNCH, "%s", msg);
  // nothing in the scratch has to start at zero: the state-only pass writes every segment's
  // contribution and the scan every starting state before anything reads them
  return forward_split(s, segments, q, k, v, s0, head_decays, o, s_out, scratch_ptr, stream);
}

int fp_retention_bwd_split(const void* q, const void* k, const void* v, const void* s0, const double* head_decays,
                           const void* d_o, const void* d_s_out, void* dq, void* dk_, void* dv_, void* d_s0, int B,
                           int T, int H, int dk, int dv, void* workspace, size_t workspace_bytes_given,
                           int forward_states_kept, void* stream) {
  const Shape s{B, T, H, dk, dv};
  if (int rc = check_shape(s, head_decays)) return rc;
  if (int rc = check_stream(stream, "fp_retention_bwd_split")) return rc;
  if (!q || !k || !v || !d_o || !dq || !dk_ || !dv_)
    return fail(FP_ERR_NULL_POINTER, "q, k, v, d_o, dq, dk and dv must not be NULL");
  const int segments = plan_backward(s);
  if (int rc = check_workspace(s, segments, workspace, workspace_bytes_given)) return rc;
  if (segments <= 1) return backward(s, q, k, v, s0, head_decays, d_o, d_s_out, nullptr, 0, dq, dk_, dv_, d_s0, stream);
  return backward_split(s, segments, q, k, v, s0, head_decays, d_o, d_s_out, dq, dk_, dv_, d_s0, workspace,
                        forward_states_kept != 0, stream);
}

int fp_pop_retention_fwd(const void* q, const void* k, const void* v, const void* s0, const double* head_decays,
                         void* o, void* block_states, int B, int T, int H, int dk, int dv, int block_size,
                         void* stream) {
  const Shape s{B, T, H, dk, dv};
  if (int rc = check_shape(s, head_decays)) return rc;
  if (int rc = check_stream(stream, "fp_pop_retention_fwd")) return rc;
  if (block_size < 1) return fail(FP_ERR_BAD_SHAPE, "block_size must be >= 1 (got %d)", block_size);
  if (!q || !k || !v || !o) return fail(FP_ERR_NULL_POINTER, "q, k, v and o must not be NULL");
  if (!block_states && T / block_size > 0)
    return fail(FP_ERR_NULL_POINTER, "block_states is NULL but T / block_size = %d", T / block_size);
  return forward(s, q, k, v, s0, head_decays, o, nullptr, block_states, block_size, stream);
}

int fp_pop_retention_bwd(const void* q, const void* k, const void* v, const void* s0, const double* head_decays,
                         const void* d_o, const void* d_block_states, void* dq, void* dk_, void* dv_, void* d_s0,
                         int B, int T, int H, int dk, int dv, int block_size, void* stream) {
  const Shape s{B, T, H, dk, dv};
  if (int rc = check_shape(s, head_decays)) return rc;
  if (int rc = check_stream(stream, "fp_pop_retention_bwd")) return rc;
  if (block_size < 1) return fail(FP_ERR_BAD_SHAPE, "block_size must be >= 1 (got %d)", block_size);
  if (!q || !k || !v || !d_o || !dq || !dk_ || !dv_)
    return fail(FP_ERR_NULL_POINTER, "q, k, v, d_o, dq, dk and dv must not be NULL");
  const void* d_blocks = (T / block_size > 0) ? d_block_states : nullptr;
  return backward(s, q, k, v, s0, head_decays, d_o, nullptr, d_blocks, block_size, dq, dk_, dv_, d_s0, stream);
}

int fp_pop_fused_fwd(const void* q, const void* k, const void* v, const void* s0, const void* q_sfx, const void* k_sfx,
                     const void* v_sfx, const double* head_decays, void* o, void* o_sfx, void* s_out, int B, int T,
                     int H, int dk, int dv, int block_size, int sfx_len, void* stream) {
  const Shape s{B, T, H, dk, dv};
  if (int rc = check_shape(s, head_decays)) return rc;
  if (int rc = check_stream(stream, "fp_pop_fused_fwd")) return rc;
  if (int rc = check_fused(s, block_size, sfx_len)) return rc;
  if (!q || !k || !v || !o || !q_sfx || !k_sfx || !v_sfx || !o_sfx)
    return fail(FP_ERR_NULL_POINTER, "q, k, v, o and their suffix counterparts must not be NULL");
  return fused_forward(s, q, k, v, s0, Suffixes{q_sfx, k_sfx, v_sfx, sfx_len}, head_decays, o, o_sfx, s_out, block_size,
                       stream);
}

int fp_pop_fused_bwd(const void* q, const void* k, const void* v, const void* s0, const void* q_sfx, const void* k_sfx,
                     const void* v_sfx, const double* head_decays, const void* d_o, const void* d_o_sfx,
                     const void* d_s_out, void* dq, void* dk_, void* dv_, void* dq_sfx, void* dk_sfx, void* dv_sfx,
                     void* d_s0, int B, int T, int H, int dk, int dv, int block_size, int sfx_len, void* stream) {
  const Shape s{B, T, H, dk, dv};
  if (int rc = check_shape(s, head_decays)) return rc;
  if (int rc = check_stream(stream, "fp_pop_fused_bwd")) return rc;
  if (int rc = check_fused(s, block_size, sfx_len)) return rc;
  if (!q || !k || !v || !q_sfx || !k_sfx || !v_sfx || !d_o || !d_o_sfx || !dq || !dk_ || !dv_ || !dq_sfx || !dk_sfx ||
      !dv_sfx)
    return fail(FP_ERR_NULL_POINTER, "inputs, d_o, d_o_sfx and the six gradient outputs must not be NULL");
  return fused_backward(s, q, k, v, s0, Suffixes{q_sfx, k_sfx, v_sfx, sfx_len}, head_decays, d_o, d_o_sfx, d_s_out, dq,
                        dk_, dv_, dq_sfx, dk_sfx, dv_sfx, d_s0, block_size, stream);
}

int fp_retention_decode_step(const void* q, const void* k, const void* v, const void* s_in, const double* head_decays,
                             void* o, void* s_out, int B, int H, int dk, int dv, void* stream) {
  const Shape s{B, 1, H, dk, dv};
  if (int rc = check_shape(s, head_decays)) return rc;
  if (!q || !k || !v || !o || !s_out) return fail(FP_ERR_NULL_POINTER, "q, k, v, o and s_out must not be NULL");
  fpk::DecodeArgs a;
  std::memset(&a, 0, sizeof a);
  a.q = in(q); a.k = in(k); a.v = in(v); a.s_in = in(s_in); a.s_out = out(s_out); a.o = out(o);
  a.B = B; a.H = H; a.dk = dk; a.dv = dv;
  a.scale = 1.0f / std::sqrt((float)dk);
  for (int h = 0; h < H; ++h) a.gamma[h] = (float)head_decays[h];
  const char* msg = "";
  if (fpk_launch_decode(a, stream, &msg) != 0) return fail(FP_ERR_LAUNCH, "decode step: %s", msg);
  return FP_OK;
}

int fp_rotary_qk(const void* q_in, const void* k_in, void* q_out, void* k_out, const float* theta, const long long* start,
                 long long start0, int B, int T, int H, int d, int inverse, void* stream) {
  if (!q_in || !q_out || !theta) return fail(FP_ERR_NULL_POINTER, "q_in, q_out and theta must not be NULL");
  if ((k_in == nullptr) != (k_out == nullptr)) return fail(FP_ERR_NULL_POINTER, "k_in and k_out must both be given or both be NULL");
  if (B < 1 || T < 1 || H < 1) return fail(FP_ERR_BAD_SHAPE, "B, T, H must be >= 1 (got %d, %d, %d)", B, T, H);
  if (d < 8 || d % 8 != 0) return fail(FP_ERR_UNSUPPORTED_DIM, "the head dimension must be a multiple of 8 (got %d)", d);
  if (misaligned(q_in) || misaligned(k_in) || misaligned(q_out) || misaligned(k_out))
    return fail(FP_ERR_BAD_SHAPE, "q and k must be 16-byte aligned");
  fpk::RotaryArgs a;
  std::memset(&a, 0, sizeof a);
  a.q_in = in(q_in); a.k_in = in(k_in); a.q_out = out(q_out); a.k_out = out(k_out);
  a.theta = theta; a.start = start; a.start0 = start0;
  a.B = B; a.T = T; a.H = H; a.d = d;
  a.sign = inverse ? -1.f : 1.f;
  const char* msg = "";
  if (fpk_launch_rotary(a, stream, &msg) != 0) return fail(FP_ERR_LAUNCH, "%s", msg);
  return FP_OK;
}

namespace {

int gated_norm(const void* r, const void* g, const void* d_out, void* y, void* d_r, void* d_g, long long rows, int H,
               int dv, double eps, void* stream) {
  if (rows < 1 || H < 1) return fail(FP_ERR_BAD_SHAPE, "rows and H must be >= 1 (got %lld, %d)", rows, H);
  const int lanes = dv / 8;
  if (dv < 8 || dv % 8 != 0 || lanes > 64 || (lanes & (lanes - 1)) != 0)
    return fail(FP_ERR_UNSUPPORTED_DIM, "dv must be 8 times a power of two, at most 512 (got %d)", dv);
  if (!(eps >= 0.0)) return fail(FP_ERR_BAD_SHAPE, "eps must be non-negative (got %g)", eps);
  if (misaligned(r) || misaligned(g) || misaligned(d_out) || misaligned(y) || misaligned(d_r) || misaligned(d_g))
    return fail(FP_ERR_BAD_SHAPE, "tensors must be 16-byte aligned");
  fpk::GatedNormArgs a;
  std::memset(&a, 0, sizeof a);
  a.r = in(r); a.g = in(g); a.d_out = in(d_out); a.out = out(y); a.d_r = out(d_r); a.d_g = out(d_g);
  a.groups = rows * H;
  a.dv = dv;
  a.eps = (float)eps;
  const char* msg = "";
  if (fpk_launch_gated_norm(a, stream, &msg) != 0) return fail(FP_ERR_LAUNCH, "%s", msg);
  return FP_OK;
}

}  // namespace

int fp_gated_group_norm_fwd(const void* r, const void* g, void* out_, long long rows, int H, int dv, double eps,
                            void* stream) {
  if (!r || !g || !out_) return fail(FP_ERR_NULL_POINTER, "r, g and out must not be NULL");
  return gated_norm(r, g, nullptr, out_, nullptr, nullptr, rows, H, dv, eps, stream);
}

int fp_gated_group_norm_bwd(const void* r, const void* g, const void* d_out, void* d_r, void* d_g, long long rows, int H,
                            int dv, double eps, void* stream) {
  if (!r || !g || !d_out || !d_r || !d_g) return fail(FP_ERR_NULL_POINTER, "r, g, d_out, d_r and d_g must not be NULL");
  return gated_norm(r, g, d_out, nullptr, d_r, d_g, rows, H, dv, eps, stream);
}

int fp_set_backward_choice(int choice, int checkpoint_every) {
  read_environment();
  if (choice < BWD_AUTO || choice > BWD_FUSED_PACED)
    return fail(FP_ERR_BAD_CONFIG, "backward choice %d: expected 0 (by shape), 1 (passes), 2 (fused) or 3 (fused, paced)", choice);
  if (checkpoint_every >= 0 && checkpoint_every % fpk::CH != 0)
    return fail(FP_ERR_BAD_CONFIG, "the checkpoint interval must be a multiple of %d tokens (got %d)", fpk::CH, checkpoint_every);
  g_bwd_choice.store(choice, std::memory_order_relaxed);
  if (checkpoint_every >= 0) g_ckpt_every.store(checkpoint_every, std::memory_order_relaxed);
  return FP_OK;
}

const char* fp_last_error(void) { return g_err; }

int fp_version(void) { return 1008; }

}  // extern "C"
