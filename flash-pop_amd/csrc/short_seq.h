// Plain retention for MANY SHORT sequences: at most 32 tokens each, head dimensions of 64 or 128, every sequence
// with an initial state of its own.  This is the suffix call of the reference's POP layer
// (flash_pop/pop_retnet.py:152-171: fused_chunk_retention on a batch of B * (N + 1) suffixes of Ls tokens, each
// seeded with a block state, the final states discarded), which the chunk kernels serve badly: a 16-token sequence
// costs them a whole 64-token item per pass and column tile, and the state traffic (a 32 KB state read and one
// written per sequence and head) dwarfs the few 4 KB tiles of token rows.
//
// Both kernels: one workgroup of 8 waves takes the (sequence, head) pairs m = block, block + grid, ... one after
// another, the next pair's rows and state on their way in registers meanwhile.  With T <= 32 a pair is one
// diagonal 32 x 32 score tile per product; with D[i][j] = scale gamma^(i - j) for j <= i (K is scaled inside
// `scale`) and every score tile rounded to bf16:
//
// forward (short_seq_fwd)
//   A = D . (q k^T),   o = A v + gamma^(i + 1) q S0,   S_out = gamma^T S0 + scale sum_j gamma^(T - 1 - j) k_j^T v_j
//   Per pair three barriers: tiles and S0 into LDS | the score tile (wave 0) and the tiles of S_out^T (all waves) |
//   waves 0..3 a 32-column slice of o (read-out of S0, then A) | everything leaves from staging tiles.
//
// backward (short_seq_bwd), no gradient arriving for the final state
//   A = D . (q k^T),  P = D . (dO v^T)
//   dv = A^T dO,   dk = P^T q,   dq = P k + gamma^(i + 1) dO S0^T,   d_s0 = sum_i gamma^(i + 1) q_i^T dO_i
//   (the state terms of dk and dv vanish with the gradient of the final state).
//   Per pair three barriers: tiles and S0 into LDS | the three score tiles (waves 0..2) | outputs: waves 0..3
//   a 32-column slice of dv and of dq (with the read-out of S0), waves 4..7 a slice of dk and the tiles of
//   d_s0^T | everything leaves from staging tiles with 16-byte stores.
// The tile layout and the operand helpers are those of retention_bwd_fused.h.
#pragma once
#include "pass_args.h"
#include "lds_access.h"
#include "retention_bwd_fused.h"

namespace fpk {

// q, k (dk wide), v, o (dv wide), 32 rows each; one score tile; the copy of S0 and the staging of S_out
constexpr int ss_fwd_lds_bytes(int dk, int dv) { return 2 * (SS_ROWS * (2 * (dk + 8) + 2 * (dv + 8)) + FB_XP + 2 * dk * (dv + 8)); }

template <int DK, int DV>
FP_DEVICE void short_seq_fwd(const ShortFwdArgs& p, char* lds) {
  using namespace fb;
  constexpr int LDK = DK + 8, LDV = DV + 8;
  constexpr int TK = SS_ROWS * LDK, TV = SS_ROWS * LDV;
  constexpr int KSK = DK / 16;
  constexpr int NTV = DV / 32, NT = (DK / 32) * NTV;         // 32 x 32 tiles of S_out^T, a row of NTV of them per 32 keys
  constexpr int TPW = (NT + 7) / 8;                          // ... per wave
  const int tid = fprt::thread_index(), wave = tid >> 6, lane = tid & 63, g = lane >> 5, c = lane & 31;
  uint16_t* const Qs = reinterpret_cast<uint16_t*>(lds);   // inputs: rows >= T are zero
  uint16_t* const Ks = Qs + TK;
  uint16_t* const Vs = Ks + TK;
  uint16_t* const OO = Vs + TV;                            // o [token][feature]
  uint16_t* const XP = OO + TV;                            // the score tile
  uint16_t* const S0 = XP + FB_XP;                         // the pair's initial state, [dk][dv] as stored
  uint16_t* const SN = S0 + DK * LDV;                      // its final state, [dk][dv]
  const uint32_t rowk = (uint32_t)p.H * DK * 2, rowv = (uint32_t)p.H * DV * 2;
  const int pairs = p.B * p.H, T = p.T;
  const bool two = T > 16;                                 // tokens 16 .. 31 exist: a second k-step along the tokens
  const bool state = p.s0 != nullptr, want_s = p.s_out != nullptr;
  const int rk = tid / (DK / 8), ck = tid % (DK / 8), rv = tid / (DV / 8), cv = tid % (DV / 8);
  const bool live_k = rk < SS_ROWS, live_v = rv < SS_ROWS;
  constexpr int SP = DK * (DV / 8) / FB_THREADS;           // 16-byte pieces of a state matrix per thread

  auto view = [&](const void* base, int m, int rows, int D) {
    const char* ptr = static_cast<const char*>(base) + ((size_t)(m / p.H) * T * p.H + (size_t)(m % p.H)) * D * 2;
    return fprt::make_buf(ptr, rows > 0 ? (uint32_t)(rows - 1) * ((uint32_t)p.H * D * 2) + D * 2 : 0u);
  };
  struct Rows {
    u32x4 q, k, v, s[SP];
  };
  auto load = [&](int m, Rows& r) {
    const int rows = m < pairs ? T : 0, mm = m < pairs ? m : 0;
    const int nk = live_k ? rows : 0, nv = live_v ? rows : 0;
    const uint32_t offk = (uint32_t)rk * rowk + ck * 16;
    r.q = fprt::buf_load128_nt(view(p.q, mm, nk, DK), offk);
    r.k = fprt::buf_load128_nt(view(p.k, mm, nk, DK), offk);
    r.v = fprt::buf_load128_nt(view(p.v, mm, nv, DV), (uint32_t)rv * rowv + cv * 16);
    const fprt::BufView sv = fprt::make_buf(state ? p.s0 + (size_t)mm * DK * DV : nullptr, state && m < pairs ? (uint32_t)(DK * DV * 2) : 0u);
#pragma unroll
    for (int u = 0; u < SP; ++u) r.s[u] = fprt::buf_load128_nt(sv, (uint32_t)(tid + FB_THREADS * u) * 16);
  };

  // the score tile: X = q (the token that reads), W = k (the token that is read), forward-walking
  const uint16_t* const s_xrow = Qs + at<LDK>(c, 8 * g);
  const uint16_t* const s_wrow = Ks + at<LDK>(score_row(c), 8 * g);
  const TrLane tr_acc_v = tr_lane<LDV>(lane, TR_ACC), tr_seq_v = tr_lane<LDV>(lane, TR_SEQ);
  const TrLane tr_nat_k = tr_lane<LDK>(lane, TR_NAT), tr_nat_v = tr_lane<LDV>(lane, TR_NAT);
  const int ct = wave & 3;   // this wave's 32-column slice of o

  Rows cur;
  load(fprt::block_index(), cur);
  for (int m = fprt::block_index(); m < pairs; m += fprt::grid_size()) {
    const float lg = p.log2g[m % p.H];
    if (live_k) {
      st128(Qs + at<LDK>(rk, 8 * ck), cur.q);
      st128(Ks + at<LDK>(rk, 8 * ck), cur.k);
    }
    if (live_v) st128(Vs + at<LDV>(rv, 8 * cv), cur.v);
    if (state) {
#pragma unroll
      for (int u = 0; u < SP; ++u) {
        const int pc = tid + FB_THREADS * u;
        st128(S0 + at<LDV>(pc / (DV / 8), 8 * (pc % (DV / 8))), cur.s[u]);
      }
    }
    load(m + fprt::grid_size(), cur);
    fprt::block_sync();

    if (wave == 0) {
      float mw[16];
      score_weights(p.scale, lg, true, false, c, g, mw);
      f32x16 sc = {0};
      u32x4 wf[KSK], xf[KSK];
#pragma unroll
      for (int t = 0; t < KSK; ++t) {
        wf[t] = frag_cols(s_wrow, t);
        xf[t] = frag_cols(s_xrow, t);
      }
      fprt::sched_fence();
#pragma unroll
      for (int t = 0; t < KSK; ++t) sc = fprt::mfma_32x32x16_bf16(wf[t], xf[t], sc);
      score_finish(sc, mw, true, false, c, g, XP, lane);
    }
    if (want_s) {
      // S_out^T[n][a] = gamma^T S0[a][n] + scale sum_j gamma^(T - 1 - j) v[j][n] k[j][a]   (rows j >= T are zero; their
      // weights are held at 1 so that a tiny gamma cannot turn them into inf)
      float wk0[8], wk1[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int d0 = T - 1 - nat_token(g, e), d1 = d0 - 16;
        wk0[e] = p.scale * fprt::exp2_approx((float)(d0 > 0 ? d0 : 0) * lg);
        wk1[e] = p.scale * fprt::exp2_approx((float)(d1 > 0 ? d1 : 0) * lg);
      }
      const float gT = fprt::exp2_approx((float)T * lg);
#pragma unroll
      for (int u = 0; u < TPW; ++u) {
        const int tile = wave + 8 * u;
        if (tile < NT) {
          const int nt = tile % NTV, at_ = tile / NTV;
          f32x16 acc = {0};
          if (state) {
            acc = get_state<LDV>(S0, 32 * at_ + c, 32 * nt, g);
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[r] *= gT;
          }
          acc = fprt::mfma_32x32x16_bf16(weigh(frag_rows<LDV>(Vs, tr_nat_v, 0, 32 * nt), wk0), frag_rows<LDK>(Ks, tr_nat_k, 0, 32 * at_), acc);
          if (two)
            acc = fprt::mfma_32x32x16_bf16(weigh(frag_rows<LDV>(Vs, tr_nat_v, 1, 32 * nt), wk1), frag_rows<LDK>(Ks, tr_nat_k, 1, 32 * at_), acc);
          // rows n = 32 nt + acc_row, column a = 32 at_ + c  ->  SN[a][n]
          put_output<LDV>(SN, 32 * at_ + c, 32 * nt, g, acc);
        }
      }
    }
    fprt::block_sync();

    if (wave < 4 && 32 * ct < DV) {
      // o^T[n][i] = gamma^(i + 1) sum_a S0[a][n] q[i][a]  +  sum_j v^T[n][j] A^T[j][i]
      f32x16 acc = {0};
      if (state) {
        u32x4 ra[KSK], xf[KSK];
#pragma unroll
        for (int t = 0; t < KSK; ++t) {
          ra[t] = frag_rows<LDV>(S0, tr_seq_v, t, 32 * ct);
          xf[t] = frag_cols(s_xrow, t);
        }
        fprt::sched_fence();
#pragma unroll
        for (int t = 0; t < KSK; ++t) acc = fprt::mfma_32x32x16_bf16(ra[t], xf[t], acc);
        const float wread = fprt::exp2_approx((float)(c + 1) * lg);
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[r] *= wread;
      }
      acc = fprt::mfma_32x32x16_bf16(frag_rows<LDV>(Vs, tr_acc_v, 0, 32 * ct), ld128(XP + lane * 8), acc);
      if (two) acc = fprt::mfma_32x32x16_bf16(frag_rows<LDV>(Vs, tr_acc_v, 1, 32 * ct), ld128(XP + 512 + lane * 8), acc);
      put_output<LDV>(OO, c, 32 * ct, g, acc);
    }
    fprt::block_sync();

    // rows < T leave; the final state leaves as it is stored
    if (live_v) fprt::buf_store128_nt(view(p.o, m, T, DV), (uint32_t)rv * rowv + cv * 16, ld128(OO + at<LDV>(rv, 8 * cv)));
    if (want_s) {
      const fprt::BufView sv = fprt::make_buf(p.s_out + (size_t)m * DK * DV, (uint32_t)(DK * DV * 2));
#pragma unroll
      for (int u = 0; u < SP; ++u) {
        const int pc = tid + FB_THREADS * u;
        fprt::buf_store128_nt(sv, (uint32_t)pc * 16, ld128(SN + at<LDV>(pc / (DV / 8), 8 * (pc % (DV / 8)))));
      }
    }
    // (the staging tiles are written again only behind the next pair's first barrier, which a thread reaches after its
    // reads from them above; the input tiles, the score tile and the copy of S0 were last read before the barrier above)
  }
}

// What the kernel assumes about its arguments; nullptr or a message for the caller.
inline const char* check_short_seq_fwd(const ShortFwdArgs& a) {
  if (a.B < 1 || a.T < 1 || a.T > SS_ROWS || a.H < 1 || a.H > MAX_HEADS || (long long)a.B * a.H > 0x7fffffffLL || !a.q || !a.k ||
      !a.v || !a.o)
    return "short-sequence forward: bad arguments";
  if (!fused_bwd_dims(a.dk_dim, a.dv_dim)) return "short-sequence forward: dk and dv of 64 or 128";
  return nullptr;
}

template <int N>
struct Pitch {
  static constexpr int value = N;
};
// q, k, dk, dq (dk wide) and v, dO, dv (dv wide), 32 rows each; three score tiles; the copy of S0 and the staging of d_s0
constexpr int ss_lds_bytes(int dk, int dv) { return 2 * (SS_ROWS * (4 * (dk + 8) + 3 * (dv + 8)) + 3 * FB_XP + 2 * dk * (dv + 8)); }

template <int DK, int DV>
FP_DEVICE void short_seq_bwd(const FusedBwdArgs& p, char* lds) {
  using namespace fb;
  constexpr int LDK = DK + 8, LDV = DV + 8;
  constexpr int TK = SS_ROWS * LDK, TV = SS_ROWS * LDV;
  constexpr int KSK = DK / 16, KSV = DV / 16;
  const int tid = fprt::thread_index(), wave = tid >> 6, lane = tid & 63, g = lane >> 5, c = lane & 31;
  uint16_t* const Qs = reinterpret_cast<uint16_t*>(lds);   // inputs: rows >= T are zero
  uint16_t* const Ks = Qs + TK;
  uint16_t* const Vs = Ks + TK;
  uint16_t* const Gs = Vs + TV;
  uint16_t* const ODV = Gs + TV;                           // outputs [token][feature]
  uint16_t* const ODK = ODV + TV;
  uint16_t* const ODQ = ODK + TK;
  uint16_t* const XP = ODQ + TK;                           // score tiles: 0 dv pass, 1 dk pass, 2 dq pass
  uint16_t* const S0 = XP + 3 * FB_XP;                     // the pair's initial state, [dk][dv] as stored
  uint16_t* const DS = S0 + DK * LDV;                      // d_s0, [dk][dv]
  const uint32_t rowk = (uint32_t)p.H * DK * 2, rowv = (uint32_t)p.H * DV * 2;
  const int pairs = p.B * p.H, T = p.T;
  const bool two = T > 16;                                 // tokens 16 .. 31 exist: a second k-step along the tokens
  const bool state = p.s0 != nullptr, want_ds = p.ds0 != nullptr;
  // this thread's 16-byte piece of the 32 rows of a tensor (a 64-wide tensor has pieces for half of the threads)
  const int rk = tid / (DK / 8), ck = tid % (DK / 8), rv = tid / (DV / 8), cv = tid % (DV / 8);
  const bool live_k = rk < SS_ROWS, live_v = rv < SS_ROWS;
  constexpr int SP = DK * (DV / 8) / FB_THREADS;           // 16-byte pieces of a state matrix per thread

  auto view = [&](const void* base, int m, int rows, int D) {
    const char* ptr = static_cast<const char*>(base) + ((size_t)(m / p.H) * T * p.H + (size_t)(m % p.H)) * D * 2;
    return fprt::make_buf(ptr, rows > 0 ? (uint32_t)(rows - 1) * ((uint32_t)p.H * D * 2) + D * 2 : 0u);
  };
  struct Rows {
    u32x4 q, k, v, d, s[SP];
  };
  auto load = [&](int m, Rows& r) {
    const int rows = m < pairs ? T : 0, mm = m < pairs ? m : 0;
    const int nk = live_k ? rows : 0, nv = live_v ? rows : 0;
    const uint32_t offk = (uint32_t)rk * rowk + ck * 16, offv = (uint32_t)rv * rowv + cv * 16;
    r.q = fprt::buf_load128_nt(view(p.q, mm, nk, DK), offk);
    r.k = fprt::buf_load128_nt(view(p.k, mm, nk, DK), offk);
    r.v = fprt::buf_load128_nt(view(p.v, mm, nv, DV), offv);
    r.d = fprt::buf_load128_nt(view(p.dO, mm, nv, DV), offv);
    const fprt::BufView sv = fprt::make_buf(state ? p.s0 + (size_t)mm * DK * DV : nullptr, state && m < pairs ? (uint32_t)(DK * DV * 2) : 0u);
#pragma unroll
    for (int u = 0; u < SP; ++u) r.s[u] = fprt::buf_load128_nt(sv, (uint32_t)(tid + FB_THREADS * u) * 16);
  };

  // score tile of waves 0..2: 0 dv pass (X = k, W = q, backward-walking), 1 dk pass (X = v, W = dO, backward), 2 dq pass
  // (X = dO, W = v, forward)
  const uint16_t* const s_xrow = wave == 0 ? Ks + at<LDK>(c, 8 * g) : wave == 1 ? Vs + at<LDV>(c, 8 * g) : Gs + at<LDV>(c, 8 * g);
  const uint16_t* const s_wrow = wave == 0   ? Qs + at<LDK>(score_row(c), 8 * g)
                                 : wave == 1 ? Gs + at<LDV>(score_row(c), 8 * g)
                                             : Vs + at<LDV>(score_row(c), 8 * g);
  const TrLane tr_acc_k = tr_lane<LDK>(lane, TR_ACC), tr_acc_v = tr_lane<LDV>(lane, TR_ACC);
  const TrLane tr_nat_k = tr_lane<LDK>(lane, TR_NAT), tr_nat_v = tr_lane<LDV>(lane, TR_NAT);
  const int ct = wave & 3;   // this wave's 32-column slice of its outputs

  Rows cur;
  load(fprt::block_index(), cur);
  for (int m = fprt::block_index(); m < pairs; m += fprt::grid_size()) {
    const float lg = p.log2g[m % p.H];
    if (live_k) {
      st128(Qs + at<LDK>(rk, 8 * ck), cur.q);
      st128(Ks + at<LDK>(rk, 8 * ck), cur.k);
    }
    if (live_v) {
      st128(Vs + at<LDV>(rv, 8 * cv), cur.v);
      st128(Gs + at<LDV>(rv, 8 * cv), cur.d);
    }
    if (state) {
#pragma unroll
      for (int u = 0; u < SP; ++u) {
        const int pc = tid + FB_THREADS * u;
        st128(S0 + at<LDV>(pc / (DV / 8), 8 * (pc % (DV / 8))), cur.s[u]);
      }
    }
    load(m + fprt::grid_size(), cur);
    fprt::block_sync();

    if (wave < 3) {
      float mw[16];
      score_weights(p.scale, lg, true, wave < 2, c, g, mw);
      f32x16 sc = {0};
      if (wave == 0) {
        u32x4 wf[KSK], xf[KSK];
#pragma unroll
        for (int t = 0; t < KSK; ++t) {
          wf[t] = frag_cols(s_wrow, t);
          xf[t] = frag_cols(s_xrow, t);
        }
        fprt::sched_fence();
#pragma unroll
        for (int t = 0; t < KSK; ++t) sc = fprt::mfma_32x32x16_bf16(wf[t], xf[t], sc);
      } else {
        u32x4 wf[KSV], xf[KSV];
#pragma unroll
        for (int t = 0; t < KSV; ++t) {
          wf[t] = frag_cols(s_wrow, t);
          xf[t] = frag_cols(s_xrow, t);
        }
        fprt::sched_fence();
#pragma unroll
        for (int t = 0; t < KSV; ++t) sc = fprt::mfma_32x32x16_bf16(wf[t], xf[t], sc);
      }
      score_finish(sc, mw, true, wave < 2, c, g, XP + wave * FB_XP, lane);
    }
    fprt::block_sync();

    // Y^T[n][i] = sum_j Z^T[n][j] P^T[j][i] over the tokens j in k-steps of 16
    auto product = [&](const uint16_t* Zs, auto tr, const TrLane& tl, const uint16_t* xp, f32x16& acc) {
      constexpr int LD = decltype(tr)::value;
      acc = fprt::mfma_32x32x16_bf16(frag_rows<LD>(Zs, tl, 0, 32 * ct), ld128(xp + lane * 8), acc);
      if (two) acc = fprt::mfma_32x32x16_bf16(frag_rows<LD>(Zs, tl, 1, 32 * ct), ld128(xp + 512 + lane * 8), acc);
    };
    using PitchK = Pitch<LDK>;
    using PitchV = Pitch<LDV>;
    if (wave < 4) {
      if (32 * ct < DV) {   // dv = A^T dO
        f32x16 acc = {0};
        product(Gs, PitchV{}, tr_acc_v, XP, acc);
        put_output<LDV>(ODV, c, 32 * ct, g, acc);
      }
      if (32 * ct < DK) {
        // dq^T[n][i] = gamma^(i + 1) sum_a S0[n][a] dO[i][a]  +  sum_j k^T[n][j] P^T[j][i]
        f32x16 acc = {0};
        if (state) {
          const uint16_t* const srow = S0 + at<LDV>(32 * ct + c, 8 * g);
          const uint16_t* const xrow = Gs + at<LDV>(c, 8 * g);
          u32x4 ra[KSV], xf[KSV];
#pragma unroll
          for (int t = 0; t < KSV; ++t) {
            ra[t] = frag_cols(srow, t);
            xf[t] = frag_cols(xrow, t);
          }
          fprt::sched_fence();
#pragma unroll
          for (int t = 0; t < KSV; ++t) acc = fprt::mfma_32x32x16_bf16(ra[t], xf[t], acc);
          const float wread = fprt::exp2_approx((float)(c + 1) * lg);
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[r] *= wread;
        }
        product(Ks, PitchK{}, tr_acc_k, XP + 2 * FB_XP, acc);
        put_output<LDK>(ODQ, c, 32 * ct, g, acc);
      }
    } else {
      if (32 * ct < DK) {   // dk = P^T q
        f32x16 acc = {0};
        product(Qs, PitchK{}, tr_acc_k, XP + FB_XP, acc);
        put_output<LDK>(ODK, c, 32 * ct, g, acc);
      }
      if (want_ds) {
        // d_s0^T[n][a] = sum_i gamma^(i + 1) dO[i][n] q[i][a]: this wave's rows n = 32 ct .. of d_s0^T, all of its columns
        if (32 * ct < DV) {
          float wk[8];
#pragma unroll
          for (int e = 0; e < 8; ++e) wk[e] = fprt::exp2_approx((float)(nat_token(g, e) + 1) * lg);
          const float g16 = fprt::exp2_approx(16.f * lg);
          const u32x4 wa0 = weigh(frag_rows<LDV>(Gs, tr_nat_v, 0, 32 * ct), wk);
#pragma unroll
          for (int e = 0; e < 8; ++e) wk[e] *= g16;
          const u32x4 wa1 = weigh(frag_rows<LDV>(Gs, tr_nat_v, 1, 32 * ct), wk);
#pragma unroll
          for (int at_ = 0; at_ < DK / 32; ++at_) {
            f32x16 acc = {0};
            acc = fprt::mfma_32x32x16_bf16(wa0, frag_rows<LDK>(Qs, tr_nat_k, 0, 32 * at_), acc);
            if (two) acc = fprt::mfma_32x32x16_bf16(wa1, frag_rows<LDK>(Qs, tr_nat_k, 1, 32 * at_), acc);
            // rows n = 32 ct + acc_row, column a = 32 at_ + c  ->  DS[a][n]
            put_output<LDV>(DS, 32 * at_ + c, 32 * ct, g, acc);
          }
        }
      }
    }
    fprt::block_sync();

    // rows < T leave; d_s0 leaves as it is stored
    if (live_v) fprt::buf_store128_nt(view(p.dv, m, T, DV), (uint32_t)rv * rowv + cv * 16, ld128(ODV + at<LDV>(rv, 8 * cv)));
    if (live_k) {
      const uint32_t off = (uint32_t)rk * rowk + ck * 16;
      fprt::buf_store128_nt(view(p.dk, m, T, DK), off, ld128(ODK + at<LDK>(rk, 8 * ck)));
      fprt::buf_store128_nt(view(p.dq, m, T, DK), off, ld128(ODQ + at<LDK>(rk, 8 * ck)));
    }
    if (want_ds) {
      const fprt::BufView dv_ = fprt::make_buf(p.ds0 + (size_t)m * DK * DV, (uint32_t)(DK * DV * 2));
#pragma unroll
      for (int u = 0; u < SP; ++u) {
        const int pc = tid + FB_THREADS * u;
        fprt::buf_store128_nt(dv_, (uint32_t)pc * 16, ld128(DS + at<LDV>(pc / (DV / 8), 8 * (pc % (DV / 8)))));
      }
    }
    // (the staging tiles are written again only behind the next pair's two barriers, the input tiles and the copy of
    // S0 were last read before the barrier above)
  }
}

// What the kernel assumes about its arguments; nullptr or a message for the caller.
inline const char* check_short_seq_bwd(const FusedBwdArgs& a) {
  if (a.B < 1 || a.T < 1 || a.T > SS_ROWS || a.H < 1 || a.H > MAX_HEADS || (long long)a.B * a.H > 0x7fffffffLL || !a.q || !a.k ||
      !a.v || !a.dO || !a.dq || !a.dk || !a.dv)
    return "short-sequence backward: bad arguments";
  if (!fused_bwd_dims(a.dk_dim, a.dv_dim)) return "short-sequence backward: dk and dv of 64 or 128";
  if (a.ds_out) return "short-sequence backward: not with a gradient of the final state";
  if (a.block > 0 || a.ckpt) return "short-sequence backward: no suffixes, no checkpoints";
  return nullptr;
}

}  // namespace fpk
