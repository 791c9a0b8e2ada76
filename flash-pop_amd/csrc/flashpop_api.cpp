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
// instead of reading stored chunk states; the dk and dv passes each carry dS.
#include "../../include/flashpop_hip.h"

#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>

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

bool dim_ok(int d) { return d == 64 || d == 128 || d == 256; }

struct Shape {
  int B, T, H, dk, dv;
};

int check_shape(const Shape& s, const double* decays) {
  if (!decays) return fail(FP_ERR_NULL_POINTER, "head_decays is NULL");
  if (s.B < 1 || s.T < 1 || s.H < 1) return fail(FP_ERR_BAD_SHAPE, "B, T, H must be >= 1 (got %d, %d, %d)", s.B, s.T, s.H);
  if (s.H > fpk::MAX_HEADS) return fail(FP_ERR_BAD_SHAPE, "H = %d exceeds the supported maximum %d", s.H, fpk::MAX_HEADS);
  if (!dim_ok(s.dk) || !dim_ok(s.dv))
    return fail(FP_ERR_UNSUPPORTED_DIM, "dk and dv must be 64, 128 or 256 (got dk=%d, dv=%d)", s.dk, s.dv);
  // per-tensor element counts are indexed with size_t in the kernel; the grid is an int
  // the kernels address one (batch, head) stream with 32-bit byte offsets
  const long long span = 2LL * s.T * s.H * (s.dk > s.dv ? s.dk : s.dv);
  if (span >= (1LL << 32)) return fail(FP_ERR_BAD_SHAPE, "T * H * max(dk, dv) too large: one sequence must stay below 4 GiB");
  const long long wgs = (long long)s.B * s.H * ((s.dk > s.dv ? s.dk : s.dv) / fpk::BV);
  if (wgs > 0x7fffffffLL) return fail(FP_ERR_BAD_SHAPE, "B * H too large");
  for (int h = 0; h < s.H; ++h) {
    if (!(decays[h] > 0.0) || !(decays[h] <= 1.0))
      return fail(FP_ERR_BAD_DECAY, "head_decays[%d] = %g is outside (0, 1]", h, decays[h]);
  }
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

const uint16_t* in(const void* p) { return static_cast<const uint16_t*>(p); }
uint16_t* out(void* p) { return static_cast<uint16_t*>(p); }

int run(const fpk::PassArgs& a, void* stream, const char* what) {
  const char* msg = "";
  if (fpk_launch_pass(a, stream, &msg) != 0) return fail(FP_ERR_LAUNCH, "%s pass: %s", what, msg);
  return FP_OK;
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

int forward(const Shape& s, const void* q, const void* k, const void* v, const void* s0, const double* decays, void* o,
            void* s_out, void* block_states, int block, void* stream) {
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

int backward(const Shape& s, const void* q, const void* k, const void* v, const void* s0, const double* decays,
             const void* d_o, const void* d_s_out, const void* d_blocks, int block, void* dq, void* dk_, void* dv_,
             void* d_s0, void* stream) {
  const float sc = 1.0f / std::sqrt((float)s.dk);
  const int nblk = block > 0 ? s.T / block : 0;
  fpk::PassArgs a;
  int rc;

  fill_common(a, s, decays);   // dq
  a.X = in(d_o); a.W = in(v); a.Z = in(k); a.Y = out(dq);
  a.R0 = in(s0);
  transposed_state(a, s);
  a.reverse = 0;
  a.s_intra = sc; a.s_read = 1.f; a.s_update = sc;
  if ((rc = run(a, stream, "dq")) != FP_OK) return rc;

  fill_common(a, s, decays);   // dk
  a.X = in(v); a.W = in(d_o); a.Z = in(q); a.Y = out(dk_);
  a.R0 = in(d_s_out); a.Bin = in(d_blocks);
  transposed_state(a, s);
  a.block = d_blocks ? block : 0; a.nblk = nblk;
  a.reverse = 1;
  a.s_intra = sc; a.s_read = sc; a.s_update = 1.f;
  if ((rc = run(a, stream, "dk")) != FP_OK) return rc;

  fill_common(a, s, decays);   // dv (+ d_s0)
  a.X = in(k); a.W = in(q); a.Z = in(d_o); a.Y = out(dv_);
  a.R0 = in(d_s_out); a.Bin = in(d_blocks); a.Rout = out(d_s0);
  plain_state(a, s);
  a.block = d_blocks ? block : 0; a.nblk = nblk;
  a.reverse = 1;
  a.s_intra = sc; a.s_read = sc; a.s_update = 1.f;
  return run(a, stream, "dv");
}

// Suffix tensors of one fused POP call, in the roles q, k, v / d_o (inputs) and o / dq, dk, dv (outputs)
struct Suffixes {
  const void *q, *k, *v;
  int len;
};

int check_fused(const Shape& s, int block, int sfx_len) {
  if (block < 1) return fail(FP_ERR_BAD_SHAPE, "block_size must be >= 1 (got %d)", block);
  if (s.T % block != 0)
    return fail(FP_ERR_BAD_SHAPE, "the fused POP op needs T to be a multiple of block_size (got T=%d, block_size=%d)", s.T, block);
  if (sfx_len < 1 || sfx_len > fpk::CH)
    return fail(FP_ERR_BAD_SHAPE, "suffix length must be in 1..%d (got %d)", fpk::CH, sfx_len);
  if (s.dk > 128 || s.dv > 128)
    return fail(FP_ERR_UNSUPPORTED_DIM, "the fused POP op supports dk and dv of 64 or 128 (got dk=%d, dv=%d)", s.dk, s.dv);
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
  const float sc = 1.0f / std::sqrt((float)s.dk);
  fpk::PassArgs a;
  int rc;

  fill_common(a, s, decays);   // dq
  a.X = in(d_o); a.W = in(v); a.Z = in(k); a.Y = out(dq);
  a.R0 = in(s0);
  transposed_state(a, s);
  suffix_walk(a, s, block, x.len, d_o_sfx, x.v, x.k, dq_sfx);
  a.reverse = 0;
  a.s_intra = sc; a.s_read = 1.f; a.s_update = sc;
  if ((rc = run(a, stream, "fused dq")) != FP_OK) return rc;

  fill_common(a, s, decays);   // dk
  a.X = in(v); a.W = in(d_o); a.Z = in(q); a.Y = out(dk_);
  a.R0 = in(d_s_out);
  transposed_state(a, s);
  suffix_walk(a, s, block, x.len, x.v, d_o_sfx, x.q, dk_sfx);
  a.reverse = 1;
  a.s_intra = sc; a.s_read = sc; a.s_update = 1.f;
  if ((rc = run(a, stream, "fused dk")) != FP_OK) return rc;

  fill_common(a, s, decays);   // dv (+ d_s0)
  a.X = in(k); a.W = in(q); a.Z = in(d_o); a.Y = out(dv_);
  a.R0 = in(d_s_out); a.Rout = out(d_s0);
  plain_state(a, s);
  suffix_walk(a, s, block, x.len, x.k, x.q, d_o_sfx, dv_sfx);
  a.reverse = 1;
  a.s_intra = sc; a.s_read = sc; a.s_update = 1.f;
  return run(a, stream, "fused dv");
}

}  // namespace

extern "C" {

int fp_retention_fwd(const void* q, const void* k, const void* v, const void* s0, const double* head_decays, void* o,
                     void* s_out, int B, int T, int H, int dk, int dv, void* stream) {
  const Shape s{B, T, H, dk, dv};
  if (int rc = check_shape(s, head_decays)) return rc;
  if (!q || !k || !v || !o) return fail(FP_ERR_NULL_POINTER, "q, k, v and o must not be NULL");
  return forward(s, q, k, v, s0, head_decays, o, s_out, nullptr, 0, stream);
}

int fp_retention_bwd(const void* q, const void* k, const void* v, const void* s0, const double* head_decays,
                     const void* d_o, const void* d_s_out, void* dq, void* dk_, void* dv_, void* d_s0, int B, int T,
                     int H, int dk, int dv, void* stream) {
  const Shape s{B, T, H, dk, dv};
  if (int rc = check_shape(s, head_decays)) return rc;
  if (!q || !k || !v || !d_o || !dq || !dk_ || !dv_)
    return fail(FP_ERR_NULL_POINTER, "q, k, v, d_o, dq, dk and dv must not be NULL");
  return backward(s, q, k, v, s0, head_decays, d_o, d_s_out, nullptr, 0, dq, dk_, dv_, d_s0, stream);
}

int fp_pop_retention_fwd(const void* q, const void* k, const void* v, const void* s0, const double* head_decays,
                         void* o, void* block_states, int B, int T, int H, int dk, int dv, int block_size,
                         void* stream) {
  const Shape s{B, T, H, dk, dv};
  if (int rc = check_shape(s, head_decays)) return rc;
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
  if (int rc = check_fused(s, block_size, sfx_len)) return rc;
  if (!q || !k || !v || !q_sfx || !k_sfx || !v_sfx || !d_o || !d_o_sfx || !dq || !dk_ || !dv_ || !dq_sfx || !dk_sfx ||
      !dv_sfx)
    return fail(FP_ERR_NULL_POINTER, "inputs, d_o, d_o_sfx and the six gradient outputs must not be NULL");
  return fused_backward(s, q, k, v, s0, Suffixes{q_sfx, k_sfx, v_sfx, sfx_len}, head_decays, d_o, d_o_sfx, d_s_out, dq,
                        dk_, dv_, dq_sfx, dk_sfx, dv_sfx, d_s0, block_size, stream);
}

const char* fp_last_error(void) { return g_err; }

int fp_version(void) { return 1001; }

}  // extern "C"
