// The two elementwise stages that surround the retention op in a layer (see RotaryArgs and
// GatedNormArgs in pass_args.h), each as one pass over its tensors with 16-byte accesses:
//   rotary_qk         q and k rotated by position * theta, both tensors and all heads of a token
//                     sharing one set of sines and cosines per thread
//   gated_norm_fwd    per-head normalisation of the retention output times the swish gate
//   gated_norm_bwd    its gradients with respect to the retention output and the gate input
// Every tensor is read once and written once; the statistics of a head are reduced over the
// dv / 8 adjacent lanes that hold it with lane exchanges, so there is no LDS and no barrier.
#pragma once
#include "pass_args.h"
#include "lds_access.h"

namespace fpk {

// ------------------------------------------------------------------------------------------
// One thread: 8 adjacent features (4 rotation pairs) of one token, for p.heads_per_thread heads of
// q and k (all of them when there are plenty of tokens: the sines and cosines are then computed
// once per token; a single decode token is spread over more threads instead of more loop trips).
FP_DEVICE void rotary_qk(const RotaryArgs& p) {
  const int opr = p.d / 8;                                   // threads per token and head group
  const int hgroups = (p.H + p.heads_per_thread - 1) / p.heads_per_thread;
  const long long unit = (long long)fprt::block_index() * LAYER_THREADS + fprt::thread_index();
  const long long row = unit / (opr * hgroups);
  if (row >= (long long)p.B * p.T) return;
  const int oc = (int)(unit % opr);
  const int h_first = (int)((unit / opr) % hgroups) * p.heads_per_thread;
  const int h_end = h_first + p.heads_per_thread < p.H ? h_first + p.heads_per_thread : p.H;
  const int b = (int)(row / p.T), t = (int)(row % p.T);
  const float pos = (float)((p.start ? p.start[b] : p.start0) + t);
  float sn[4], cs[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    fprt::sincos_f32(pos * p.theta[4 * oc + j], sn[j], cs[j]);
    sn[j] *= p.sign;
  }
  const size_t at0 = (size_t)row * p.H * p.d + 8 * oc;
#pragma unroll
  for (int which = 0; which < 2; ++which) {
    const uint16_t* src = which ? p.k_in : p.q_in;
    uint16_t* dst = which ? p.k_out : p.q_out;
    if (!src) continue;
    // four heads at a time, their loads issued before the first is used
    for (int h0 = h_first; h0 < h_end; h0 += 4) {
      u32x4 v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        if (h0 + u < h_end) v[u] = ld128(src + at0 + (size_t)(h0 + u) * p.d);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        if (h0 + u >= h_end) break;
        u32x4 o;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float e = bf16_elem(v[u], 2 * j), d = bf16_elem(v[u], 2 * j + 1);
          o[j] = fprt::pack_bf16x2(e * cs[j] - d * sn[j], d * cs[j] + e * sn[j]);
        }
        st128(dst + at0 + (size_t)(h0 + u) * p.d, o);
      }
    }
  }
}

// ------------------------------------------------------------------------------------------
// sum over the `lanes` adjacent lanes (a power of two) that hold one head; every lane gets it
FP_DEVICE float head_sum(float v, int lanes) {
  for (int m = lanes >> 1; m >= 1; m >>= 1) v += fprt::lane_xor(v, m);
  return v;
}

struct HeadStats {
  float dev[8];   // r - mean
  float rstd;
};

// this thread's 8 values of r, centred, and the head's 1 / sqrt(var + eps)
FP_DEVICE HeadStats head_stats(u32x4 rv, int lanes, int dv, float eps) {
  HeadStats st;
  float s = 0.f;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    st.dev[e] = bf16_elem(rv, e);
    s += st.dev[e];
  }
  const float mean = head_sum(s, lanes) / (float)dv;
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    st.dev[e] -= mean;
    ss += st.dev[e] * st.dev[e];
  }
  st.rstd = fprt::rsqrt_f32(head_sum(ss, lanes) / (float)dv + eps);
  return st;
}

FP_DEVICE float round_bf16(float x) { return bf16_bits_to_float(float_to_bf16_bits(x)); }

// One thread: 8 adjacent values of one (row, head).  Threads past the last head take part in the
// lane exchanges with zeros and touch no memory.
FP_DEVICE void gated_norm_fwd(const GatedNormArgs& p) {
  const int lanes = p.dv / 8;
  const long long unit = (long long)fprt::block_index() * LAYER_THREADS + fprt::thread_index();
  const bool live = unit / lanes < p.groups;
  const size_t at = (size_t)unit * 8;
  const u32x4 zero = {0, 0, 0, 0};
  const u32x4 rv = live ? ld128(p.r + at) : zero;
  const u32x4 gv = live ? ld128(p.g + at) : zero;
  const HeadStats st = head_stats(rv, lanes, p.dv, p.eps);
  float y[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float g = bf16_elem(gv, e);
    const float gate = round_bf16(g * fprt::sigmoid_f32(g));
    y[e] = round_bf16(st.dev[e] * st.rstd) * gate;
  }
  u32x4 o;
#pragma unroll
  for (int e = 0; e < 4; ++e) o[e] = fprt::pack_bf16x2(y[2 * e], y[2 * e + 1]);
  if (live) st128(p.out + at, o);
}

// With n^ = (r - mean) rstd, s = swish(g), dn = d_out * s:
//   d_r = rstd (dn - mean(dn) - n^ mean(dn n^)),   d_g = d_out * n * swish'(g)
// where n is n^ rounded to bf16 as the forward used it and swish'(g) = sig (1 + g (1 - sig)).
FP_DEVICE void gated_norm_bwd(const GatedNormArgs& p) {
  const int lanes = p.dv / 8;
  const long long unit = (long long)fprt::block_index() * LAYER_THREADS + fprt::thread_index();
  const bool live = unit / lanes < p.groups;
  const size_t at = (size_t)unit * 8;
  const u32x4 zero = {0, 0, 0, 0};
  const u32x4 rv = live ? ld128(p.r + at) : zero;
  const u32x4 gv = live ? ld128(p.g + at) : zero;
  const u32x4 dv_ = live ? ld128(p.d_out + at) : zero;
  const HeadStats st = head_stats(rv, lanes, p.dv, p.eps);
  float nh[8], dn[8], dg[8];
  float s1 = 0.f, s2 = 0.f;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float g = bf16_elem(gv, e), dy = bf16_elem(dv_, e);
    const float sig = fprt::sigmoid_f32(g);
    nh[e] = st.dev[e] * st.rstd;
    dn[e] = dy * round_bf16(g * sig);
    dg[e] = dy * round_bf16(nh[e]) * (sig * (1.f + g * (1.f - sig)));
    s1 += dn[e];
    s2 += dn[e] * nh[e];
  }
  const float m1 = head_sum(s1, lanes) / (float)p.dv;
  const float m2 = head_sum(s2, lanes) / (float)p.dv;
  u32x4 o_r, o_g;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    o_r[e] = fprt::pack_bf16x2(st.rstd * (dn[2 * e] - m1 - nh[2 * e] * m2),
                               st.rstd * (dn[2 * e + 1] - m1 - nh[2 * e + 1] * m2));
    o_g[e] = fprt::pack_bf16x2(dg[2 * e], dg[2 * e + 1]);
  }
  if (live) {
    st128(p.d_r + at, o_r);
    st128(p.d_g + at, o_g);
  }
}

// ------------------------------------------------------------------------------------------
// Host side: argument checks and grid sizes, shared by the GPU launcher and the CPU test harness.
// Return nullptr if the launch is valid (and the number of workgroups in `blocks`), else the reason.
// (chooses a.heads_per_thread)
inline const char* plan_rotary(RotaryArgs& a, long long& blocks) {
  if (a.B < 1 || a.T < 1 || a.H < 1 || a.d < 8 || a.d % 8 != 0) return "rotary: B, T, H >= 1 and d a multiple of 8 expected";
  if (!a.q_in || !a.q_out || !a.theta || (a.k_in == nullptr) != (a.k_out == nullptr)) return "rotary: null pointer";
  if (a.sign != 1.f && a.sign != -1.f) return "rotary: sign must be +1 or -1";
  // fewer than two waves per compute unit's worth of token threads: one head per thread, so that a
  // decode step's few tokens do not walk all heads in a loop of dependent loads
  const long long token_threads = (long long)a.B * a.T * (a.d / 8);
  a.heads_per_thread = token_threads >= (1 << 15) ? a.H : 1;
  const long long units = token_threads * ((a.H + a.heads_per_thread - 1) / a.heads_per_thread);
  blocks = (units + LAYER_THREADS - 1) / LAYER_THREADS;
  return blocks > 0x7fffffffLL ? "rotary: too many tokens for one launch" : nullptr;
}

inline const char* plan_gated_norm(const GatedNormArgs& a, long long& blocks) {
  const int lanes = a.dv / 8;
  if (a.groups < 1 || a.dv < 8 || a.dv % 8 != 0 || lanes > 64 || (lanes & (lanes - 1)) != 0)
    return "gated norm: dv must be 8 times a power of two, at most 512";
  if (!(a.eps >= 0.f)) return "gated norm: eps must be non-negative";
  const bool fwd = a.out != nullptr;
  if (!a.r || !a.g || (fwd ? (a.d_out || a.d_r || a.d_g) : (!a.d_out || !a.d_r || !a.d_g)))
    return "gated norm: pointers of exactly one direction expected";
  const long long units = a.groups * lanes;
  blocks = (units + LAYER_THREADS - 1) / LAYER_THREADS;
  return blocks > 0x7fffffffLL ? "gated norm: too many rows for one launch" : nullptr;
}

}  // namespace fpk
