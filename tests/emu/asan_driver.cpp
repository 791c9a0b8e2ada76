// Runs every C entry point on the CPU thread harness with heap buffers of exactly the sizes the
// header documents, for AddressSanitizer / UBSan builds: any access of a kernel body outside a
// tensor, the workspace or the LDS block it was given aborts the run.  Test infrastructure only.
#include "../../include/flashpop_hip.h"

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>

namespace {

std::vector<void*> g_live;

uint16_t* buf(size_t n, bool fill = true) {
  uint16_t* p = static_cast<uint16_t*>(malloc(n * 2 + (n == 0)));
  for (size_t i = 0; i < n; ++i) p[i] = fill ? static_cast<uint16_t>(0x3c00 + (rand() & 0x1ff)) : 0;   // bf16 in [1, 2)
  g_live.push_back(p);
  return p;
}

int done(int rc, const char* what, int B, int T, int H, int dk, int dv, int extra) {
  for (void* p : g_live) free(p);
  g_live.clear();
  if (rc) {
    printf("FAILED %s: %s\n", what, fp_last_error());
  } else {
    printf("ok %s B%d T%d H%d dk%d dv%d (%d)\n", what, B, T, H, dk, dv, extra);
  }
  fflush(stdout);
  return rc;
}

// many short sequences with a state each and no gradient of the final state: the suffix call of the POP layer
int short_sequences(int B, int T, int H, int dk, int dv, bool state) {
  std::vector<double> dec(H, 0.97);
  const size_t nq = (size_t)B * T * H * dk, nv = (size_t)B * T * H * dv, ns = (size_t)B * H * dk * dv;
  uint16_t *q = buf(nq), *k = buf(nq), *v = buf(nv), *s = state ? buf(ns) : nullptr;
  uint16_t *dO = buf(nv), *dq = buf(nq, false), *dk_ = buf(nq, false), *dv_ = buf(nv, false), *ds0 = state ? buf(ns, false) : nullptr;
  uint16_t *o = buf(nv, false), *so = state ? buf(ns, false) : nullptr;   // the final state only for the pairs that have an initial one
  int rc = fp_retention_fwd(q, k, v, s, dec.data(), o, so, B, T, H, dk, dv, nullptr);
  if (!rc) rc = fp_retention_bwd(q, k, v, s, dec.data(), dO, nullptr, dq, dk_, dv_, ds0, B, T, H, dk, dv, nullptr);
  return done(rc, "short", B, T, H, dk, dv, state);
}

int plain(int B, int T, int H, int dk, int dv, bool split) {
  std::vector<double> dec(H, 0.97);
  const size_t nq = (size_t)B * T * H * dk, nv = (size_t)B * T * H * dv, ns = (size_t)B * H * dk * dv;
  uint16_t *q = buf(nq), *k = buf(nq), *v = buf(nv), *s = buf(ns), *o = buf(nv, false), *so = buf(ns, false);
  uint16_t *dO = buf(nv), *dS = buf(ns), *dq = buf(nq, false), *dk_ = buf(nq, false), *dv_ = buf(nv, false), *ds0 = buf(ns, false);
  int rc;
  if (split) {
    const size_t wb = fp_retention_workspace_bytes(B, T, H, dk, dv);
    void* ws = wb ? aligned_alloc(16, wb) : nullptr;
    rc = fp_retention_fwd_split(q, k, v, s, dec.data(), o, so, B, T, H, dk, dv, ws, wb, nullptr);
    if (!rc) rc = fp_retention_bwd_split(q, k, v, s, dec.data(), dO, dS, dq, dk_, dv_, ds0, B, T, H, dk, dv, ws, wb, 1, nullptr);
    if (!rc) rc = fp_retention_bwd_split(q, k, v, s, dec.data(), dO, dS, dq, dk_, dv_, ds0, B, T, H, dk, dv, ws, wb, 0, nullptr);
    free(ws);
    return done(rc, "split", B, T, H, dk, dv, (int)wb);
  }
  rc = fp_retention_fwd(q, k, v, s, dec.data(), o, so, B, T, H, dk, dv, nullptr);
  if (!rc && T <= 32) {   // short sequences have a forward kernel of their own: the pass kernel's turn
    fp_set_backward_choice(1, -1);
    rc = fp_retention_fwd(q, k, v, s, dec.data(), o, so, B, T, H, dk, dv, nullptr);
    fp_set_backward_choice(0, -1);
  }
  if (!rc) rc = fp_retention_bwd(q, k, v, s, dec.data(), dO, dS, dq, dk_, dv_, ds0, B, T, H, dk, dv, nullptr);
  return done(rc, "plain", B, T, H, dk, dv, 0);
}

int pop(int B, int T, int H, int dk, int dv, int block) {
  std::vector<double> dec(H, 0.97);
  const size_t nq = (size_t)B * T * H * dk, nv = (size_t)B * T * H * dv, ns = (size_t)B * H * dk * dv;
  const int nb = T / block;
  uint16_t *q = buf(nq), *k = buf(nq), *v = buf(nv), *s = buf(ns), *o = buf(nv, false), *dO = buf(nv);
  uint16_t *dq = buf(nq, false), *dk_ = buf(nq, false), *dv_ = buf(nv, false), *ds0 = buf(ns, false);
  uint16_t *bs = buf(nb * ns, false), *dbs = buf(nb * ns);
  int rc = fp_pop_retention_fwd(q, k, v, s, dec.data(), o, nb ? bs : nullptr, B, T, H, dk, dv, block, nullptr);
  if (!rc) rc = fp_pop_retention_bwd(q, k, v, s, dec.data(), dO, nb ? dbs : nullptr, dq, dk_, dv_, ds0, B, T, H, dk, dv, block, nullptr);
  return done(rc, "pop", B, T, H, dk, dv, block);
}

// forward with checkpoints every `every` tokens, then the backward that starts from them
int checkpointed(int B, int T, int H, int every, int dk = 128, int dv = 128) {
  std::vector<double> dec(H, 0.97);
  const size_t nq = (size_t)B * T * H * dk, nv = (size_t)B * T * H * dv, ns = (size_t)B * H * dk * dv,
               nc = (size_t)B * (T / every) * H * dk * dv;
  uint16_t *q = buf(nq), *k = buf(nq), *v = buf(nv), *s = buf(ns), *o = buf(nv, false), *so = buf(ns, false), *ck = buf(nc, false);
  uint16_t *dO = buf(nv), *dS = buf(ns), *dq = buf(nq, false), *dk_ = buf(nq, false), *dv_ = buf(nv, false), *ds0 = buf(ns, false);
  int rc = fp_retention_fwd_ckpt(q, k, v, s, dec.data(), o, so, ck, every, B, T, H, dk, dv, nullptr);
  if (!rc) rc = fp_retention_bwd_ckpt(q, k, v, s, dec.data(), dO, dS, ck, every, dq, dk_, dv_, ds0, B, T, H, dk, dv, nullptr);
  return done(rc, "checkpointed", B, T, H, dk, dv, every);
}

// nblk full blocks and `tail` < block tokens after them
int fused(int B, int nblk, int block, int ls, int H, int dk, int dv, int tail = 0) {
  std::vector<double> dec(H, 0.97);
  const int T = nblk * block + tail;
  const size_t nq = (size_t)B * T * H * dk, nv = (size_t)B * T * H * dv, ns = (size_t)B * H * dk * dv;
  const size_t sq = (size_t)B * (nblk + 1) * ls * H * dk, sv = (size_t)B * (nblk + 1) * ls * H * dv;
  uint16_t *q = buf(nq), *k = buf(nq), *v = buf(nv), *s = buf(ns), *qs = buf(sq), *ks = buf(sq), *vs = buf(sv);
  uint16_t *o = buf(nv, false), *os = buf(sv, false), *so = buf(ns, false), *dO = buf(nv), *dOs = buf(sv), *dS = buf(ns);
  uint16_t *dq = buf(nq, false), *dk_ = buf(nq, false), *dv_ = buf(nv, false), *dqs = buf(sq, false), *dks = buf(sq, false),
           *dvs = buf(sv, false), *ds0 = buf(ns, false);
  int rc = fp_pop_fused_fwd(q, k, v, s, qs, ks, vs, dec.data(), o, os, so, B, T, H, dk, dv, block, ls, nullptr);
  if (!rc) rc = fp_pop_fused_bwd(q, k, v, s, qs, ks, vs, dec.data(), dO, dOs, dS, dq, dk_, dv_, dqs, dks, dvs, ds0, B, T, H,
                                 dk, dv, block, ls, nullptr);
  return done(rc, "fused", B, T, H, dk, dv, ls);
}

int decode(int B, int H, int dk, int dv) {
  std::vector<double> dec(H, 0.97);
  const size_t ns = (size_t)B * H * dk * dv;
  uint16_t *q = buf((size_t)B * H * dk), *k = buf((size_t)B * H * dk), *v = buf((size_t)B * H * dv), *s = buf(ns);
  uint16_t *o = buf((size_t)B * H * dv, false), *so = buf(ns, false);
  int rc = fp_retention_decode_step(q, k, v, s, dec.data(), o, so, B, H, dk, dv, nullptr);
  if (!rc) rc = fp_retention_decode_step(q, k, v, so, dec.data(), o, so, B, H, dk, dv, nullptr);   // in place
  return done(rc, "decode", B, 1, H, dk, dv, 0);
}

int rotary(int B, int T, int H, int d, bool per_sequence) {
  const size_t n = (size_t)B * T * H * d;
  uint16_t *q = buf(n), *k = buf(n), *qo = buf(n, false), *ko = buf(n, false);
  std::vector<float> theta(d / 2);
  for (int i = 0; i < d / 2; ++i) theta[i] = 1.0f / (float)(i + 1);
  std::vector<long long> start(B);
  for (int b = 0; b < B; ++b) start[b] = 100 * b;
  int rc = fp_rotary_qk(q, k, qo, ko, theta.data(), per_sequence ? start.data() : nullptr, 7, B, T, H, d, 0, nullptr);
  if (!rc) rc = fp_rotary_qk(qo, nullptr, qo, nullptr, theta.data(), nullptr, 7, B, T, H, d, 1, nullptr);   // q only, in place
  return done(rc, "rotary", B, T, H, d, d, per_sequence);
}

int gated_norm(int rows, int H, int dv) {
  const size_t n = (size_t)rows * H * dv;
  uint16_t *r = buf(n), *g = buf(n), *d_out = buf(n), *out = buf(n, false), *d_r = buf(n, false), *d_g = buf(n, false);
  int rc = fp_gated_group_norm_fwd(r, g, out, rows, H, dv, 1e-6, nullptr);
  if (!rc) rc = fp_gated_group_norm_bwd(r, g, d_out, d_r, d_g, rows, H, dv, 1e-6, nullptr);
  return done(rc, "gated norm", rows, 1, H, dv, dv, 0);
}

}  // namespace

int main() {
  int rc = 0;
  rc |= plain(5, 16, 1, 128, 128, false);     // several short sequences per workgroup
  rc |= plain(3, 70, 2, 64, 64, false);       // ragged tails
  rc |= plain(2, 1, 1, 64, 64, false);        // single token
  rc |= plain(1, 65, 1, 64, 256, false);      // two visits per chunk, state read transposed
  rc |= plain(1, 130, 1, 256, 64, false);     // two visits per chunk, state as stored
  rc |= plain(1, 100, 1, 192, 192, false);    // three visits per chunk
  rc |= plain(1, 512, 1, 64, 128, true);      // cut into segments (state-only walk, scan)
  rc |= plain(1, 640, 1, 128, 256, true);     // ... with the state-only kernel for 128-wide keys, two workgroups per segment
  rc |= pop(1, 287, 1, 64, 128, 144);
  rc |= pop(2, 28, 1, 64, 64, 15);
  rc |= pop(1, 40, 1, 64, 64, 100);           // no full block
  rc |= pop(1, 96, 1, 256, 64, 32);           // block states with two visits per chunk
  rc |= fused(2, 2, 80, 5, 1, 64, 128);
  rc |= fused(1, 3, 24, 64, 1, 128, 64);
  rc |= fused(1, 2, 40, 9, 1, 64, 256);       // suffixes with two visits per chunk
  rc |= fused(1, 1, 80, 5, 1, 64, 128, 30);   // tokens after the last block boundary
  rc |= fused(1, 0, 90, 12, 1, 64, 64, 70);   // no full block
  rc |= fused(1, 2, 64, 100, 1, 128, 64);     // suffixes in two parts
  fp_set_backward_choice(2, -1);        // one short stream would not take this path by itself
  rc |= fused(1, 4, 64, 16, 1, 128, 128);     // backward in the kernel that carries dS once, suffixes as extra stops
  rc |= plain(1, 210, 1, 128, 128, false);    // the same kernel without suffixes, ragged last chunk
  rc |= checkpointed(1, 280, 1, 128);         // ... with the forward's checkpoints
  rc |= fused(1, 4, 64, 16, 1, 64, 128);      // the same kernels for 64-wide keys: folded suffixes,
  rc |= fused(1, 2, 128, 40, 1, 128, 64);     // 64-wide values with the suffixes as stops,
  rc |= plain(1, 210, 1, 64, 64, false);      // 64 x 64 states (half of the waves own a tile), ragged last chunk,
  rc |= checkpointed(1, 280, 1, 64, 64, 128);    // checkpoints of 64 x 128 states
  rc |= fused(1, 4, 64, 9, 1, 64, 64);        // folded suffixes of 9 tokens on 64 x 64 states
  rc |= pop(1, 256, 1, 128, 128, 64);         // gradients of block states added on the reverse walk of that kernel
  rc |= pop(1, 300, 1, 64, 128, 128);         // ... 64-wide keys, tokens after the last boundary
  fp_set_backward_choice(3, -1);
  rc |= checkpointed(1, 200, 2, 64, 128, 64);    // the two workgroups of a stream paced (pacing words written and polled)
  fp_set_backward_choice(0, -1);
  rc |= short_sequences(7, 16, 2, 128, 128, true);   // more pairs than workgroups, one k-step along the tokens
  rc |= short_sequences(2, 31, 1, 64, 128, true);    // two k-steps, 64-wide keys
  rc |= short_sequences(3, 5, 1, 128, 64, false);    // no state
  rc |= short_sequences(1, 32, 2, 64, 64, true);
  rc |= decode(2, 3, 64, 128);
  rc |= decode(1, 1, 256, 256);
  rc |= rotary(3, 11, 2, 64, true);           // last workgroup partly idle
  rc |= rotary(1, 5, 3, 8, false);
  rc |= gated_norm(7, 3, 64);                 // heads past the end in the last workgroup
  rc |= gated_norm(3, 1, 256);
  rc |= gated_norm(9, 5, 8);
  return rc;
}
