// The retention pass kernel body (see pass_args.h for the recurrence it evaluates).
//
// One workgroup of 4 wave64 owns one (batch, head) stream and one 64-column slice of
// Z / Y / R, and walks the sequence chunk by chunk.  R (dA x 64, fp32) lives in MFMA
// accumulators for the whole sequence; a bf16 copy is refreshed in LDS once per chunk
// as the operand of the state read-out.  Waves form a 2 x 2 grid: `ib` picks the 32
// chunk rows, `nb` the 32 output columns a wave produces.
//
// Per chunk:
//   scores^T = W X^T        (tokens j x tokens i, contraction over dA)       MFMA 32x32x16
//   P        = bf16(scores * s_intra * gamma^|i-j|), kept in registers: the accumulator
//              layout of scores^T is, lane for lane, the A-operand layout of P Z
//   Y        = wread * (X R) + P Z                                           MFMA
//   R        = gamma^L R + (wkey * W)^T Z                                    MFMA
// Products that contract over tokens need operands that are contiguous in the token
// index, so W (weighted) and Z are transposed on their way from registers into LDS.
//
// Written against the fprt primitives only, so the same body also runs under the CPU
// thread harness used by the tests.
#pragma once
#include "pass_args.h"

namespace fpk {

using fprt::f32x16;
using fprt::u32x2;
using fprt::u32x4;

typedef u32x4 __attribute__((may_alias, aligned(16))) u32x4_m;
typedef u32x2 __attribute__((may_alias, aligned(8))) u32x2_m;
typedef uint16_t __attribute__((may_alias)) u16_m;

FP_DEVICE u32x4 ld128(const uint16_t* p) { return *reinterpret_cast<const u32x4_m*>(p); }
FP_DEVICE u32x2 ld64(const uint16_t* p) { return *reinterpret_cast<const u32x2_m*>(p); }
FP_DEVICE void st128(uint16_t* p, u32x4 v) { *reinterpret_cast<u32x4_m*>(p) = v; }
FP_DEVICE void st64(uint16_t* p, u32x2 v) { *reinterpret_cast<u32x2_m*>(p) = v; }

FP_DEVICE float bf16_bits_to_float(uint32_t bits16) { return __builtin_bit_cast(float, bits16 << 16); }
// element e (0..7) of eight packed bf16
FP_DEVICE float bf16_elem(u32x4 v, int e) {
  uint32_t d = v[e >> 1];
  return __builtin_bit_cast(float, (e & 1) ? (d & 0xffff0000u) : (d << 16));
}
FP_DEVICE uint16_t float_to_bf16_bits(float x) { return (uint16_t)(fprt::pack_bf16x2(x, 0.f) & 0xffffu); }

// row of the 32x32 MFMA accumulator held in element r by a lane of half-wave g
FP_DEVICE int acc_row(int r, int g) { return 8 * (r >> 2) + 4 * g + (r & 3); }

template <int DA>
FP_DEVICE void retention_pass(const PassArgs& p, char* lds) {
  static_assert(DA % 64 == 0 && DA >= 64 && DA <= 256, "dA must be 64, 128, 192 or 256");
  constexpr int X_LD = DA + 8;    // bf16 elements per LDS row
  constexpr int WT_LD = CH + 4;
  constexpr int ZT_LD = CH + 4;
  constexpr int RT_LD = DA + 8;
  constexpr int YB_LD = BV + 8;
  constexpr int KS = DA / 16;     // MFMA k-steps over dA
  constexpr int FG = DA / 8;      // 16-byte pieces per X / W row
  constexpr int NUNIT = 16 * FG;  // load units (4 tokens x 8 features) per tile
  constexpr int NU = (NUNIT + NTHREADS - 1) / NTHREADS;
  constexpr int NAB = DA / 32;    // 32-row blocks of R
  constexpr int RU = NAB / 2;     // R blocks per wave

  uint16_t* XS = reinterpret_cast<uint16_t*>(lds);
  uint16_t* WS = XS + CH * X_LD;
  uint16_t* WT = WS + CH * X_LD;
  uint16_t* ZT = WT + DA * WT_LD;
  uint16_t* RT = ZT + BV * ZT_LD;
  uint16_t* YB = RT + BV * RT_LD;

  const int tid = fprt::thread_index();
  const int wave = tid >> 6, lane = tid & 63;
  const int ib = wave >> 1, nb = wave & 1;
  const int g = lane >> 5, c = lane & 31;

  // Workgroup -> (b, h, column tile).  Workgroups are dealt round-robin to the 8 XCDs;
  // undo that so that the column tiles of one stream, which read the same X and W, sit
  // behind the same L2.
  const int ntile = p.dB / BV;
  const int nwg = fprt::grid_size();
  int wg = fprt::block_index();
  if ((nwg & 7) == 0) wg = (wg & 7) * (nwg >> 3) + (wg >> 3);
  const int tile = wg % ntile;
  const int bh = wg / ntile;
  const int h = bh % p.H, b = bh / p.H;

  const int T = p.T, bs = p.block;
  const bool rev = p.reverse != 0;
  const float lg = p.log2g[h];
  const size_t rowA = (size_t)p.H * p.dA, rowB = (size_t)p.H * p.dB;
  const size_t streamA = ((size_t)b * T * p.H + h) * p.dA;
  const size_t streamB = ((size_t)b * T * p.H + h) * p.dB + (size_t)tile * BV;
  const uint16_t* Xg = p.X + streamA;
  const uint16_t* Wg = p.W + streamA;
  const uint16_t* Zg = p.Z + streamB;
  uint16_t* Yg = p.Y + streamB;
  const size_t mat = (size_t)p.dA * p.dB;   // elements of one state matrix

  // ---- chunk-invariant weights ------------------------------------------------------
  // Decay of the scores, for the diagonal tile (jb == ib) and the off-diagonal one.
  float mw_diag[16], mw_off[16];
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int jl = acc_row(r, g);
    const int d = rev ? (jl - c) : (c - jl);
    mw_diag[r] = d >= 0 ? p.s_intra * fprt::exp2_approx((float)d * lg) : 0.f;
    mw_off[r] = p.s_intra * fprt::exp2_approx((float)(32 + d) * lg);
  }
  // does this wave need the off-diagonal score tile?
  const bool need_off = rev ? (ib == 0) : (ib == 1);
  const int jb_off = 1 - ib;

  // ---- load-unit coordinates ---------------------------------------------------------
  int u_fg[NU], u_tg[NU];
  bool u_ok[NU];
#pragma unroll
  for (int u = 0; u < NU; ++u) {
    const int unit = tid + u * NTHREADS;
    u_ok[u] = unit < NUNIT;
    u_fg[u] = unit % FG;
    u_tg[u] = (unit / FG) & 15;
  }
  const int z_tg = tid >> 4, z_fq = tid & 15;

  u32x4 px[NU][4], pw[NU][4];
  u32x2 pz[4];
  const u32x4 zero4 = {0u, 0u, 0u, 0u};
  const u32x2 zero2 = {0u, 0u};

  auto prefetch = [&](int t0, int L) {
#pragma unroll
    for (int u = 0; u < NU; ++u) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int j = 4 * u_tg[u] + r;
        if (u_ok[u] && j < L) {
          const size_t off = (size_t)(t0 + j) * rowA + 8 * u_fg[u];
          px[u][r] = ld128(Xg + off);
          pw[u][r] = ld128(Wg + off);
        } else {
          px[u][r] = zero4;
          pw[u][r] = zero4;
        }
      }
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int j = 4 * z_tg + r;
      pz[r] = j < L ? ld64(Zg + (size_t)(t0 + j) * rowB + 4 * z_fq) : zero2;
    }
  };

  // chunk [t0, t0 + L) that follows position `pos` in walking order
  auto chunk_at = [&](int pos, int& t0, int& L) {
    if (!rev) {
      int end = pos + CH < T ? pos + CH : T;
      if (bs > 0) {
        const int nbnd = (pos / bs + 1) * bs;
        if (nbnd < end) end = nbnd;
      }
      t0 = pos;
      L = end - pos;
    } else {
      int start = pos - CH > 0 ? pos - CH : 0;
      if (bs > 0) {
        const int pbnd = ((pos - 1) / bs) * bs;
        if (pbnd > start) start = pbnd;
      }
      t0 = start;
      L = pos - start;
    }
  };

  // ---- state ---------------------------------------------------------------------------
  f32x16 racc[RU];
  const size_t n_glob = (size_t)tile * BV + 32 * nb + c;
  auto state_off = [&](int u, int r) -> size_t {
    const int a = 32 * (ib * RU + u) + acc_row(r, g);
    return (size_t)a * p.rs_a + n_glob * p.rs_n;
  };
#pragma unroll
  for (int u = 0; u < RU; ++u) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      racc[u][r] = p.R0 ? bf16_bits_to_float(p.R0[(size_t)bh * mat + state_off(u, r)]) : 0.f;
    }
  }

  // L-dependent weights, refreshed only when L changes
  int L_cached = -1;
  float wread[16], wkey[NU][4], gL = 1.f;
  auto refresh_weights = [&](int L) {
    if (L == L_cached) return;
    L_cached = L;
    gL = fprt::exp2_approx((float)L * lg);
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int i = 32 * ib + acc_row(r, g);
      int e = rev ? (L - 1 - i) : (i + 1);
      if (e < 0) e = 0;
      wread[r] = p.s_read * fprt::exp2_approx((float)e * lg);
    }
#pragma unroll
    for (int u = 0; u < NU; ++u) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int j = 4 * u_tg[u] + r;
        int e = rev ? (j + 1) : (L - 1 - j);
        if (e < 0) e = 0;
        wkey[u][r] = p.s_update * fprt::exp2_approx((float)e * lg);
      }
    }
  };

  // ---- walk the sequence ---------------------------------------------------------------
  int pos = rev ? T : 0;
  int t0, L;
  chunk_at(pos, t0, L);
  prefetch(t0, L);

  while (true) {
    const int t1 = t0 + L;
    refresh_weights(L);

    // block-state gradient joins R before the chunk that ends the block (reverse walk)
    if (p.Bin && bs > 0 && (t1 % bs) == 0) {
      const size_t base = (((size_t)b * p.nblk + (t1 / bs - 1)) * p.H + h) * mat;
#pragma unroll
      for (int u = 0; u < RU; ++u) {
#pragma unroll
        for (int r = 0; r < 16; ++r) racc[u][r] += bf16_bits_to_float(p.Bin[base + state_off(u, r)]);
      }
    }

    // -- registers -> LDS ------------------------------------------------------------
#pragma unroll
    for (int u = 0; u < NU; ++u) {
      if (u_ok[u]) {
        const int fg = u_fg[u], tg = u_tg[u];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          st128(XS + (4 * tg + r) * X_LD + 8 * fg, px[u][r]);
          st128(WS + (4 * tg + r) * X_LD + 8 * fg, pw[u][r]);
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          u32x2 d;
          d[0] = fprt::pack_bf16x2(bf16_elem(pw[u][0], e) * wkey[u][0], bf16_elem(pw[u][1], e) * wkey[u][1]);
          d[1] = fprt::pack_bf16x2(bf16_elem(pw[u][2], e) * wkey[u][2], bf16_elem(pw[u][3], e) * wkey[u][3]);
          st64(WT + (8 * fg + e) * WT_LD + 4 * tg, d);
        }
      }
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int w = e >> 1;
      u32x2 d;
      if (e & 1) {
        d[0] = (pz[0][w] >> 16) | (pz[1][w] & 0xffff0000u);
        d[1] = (pz[2][w] >> 16) | (pz[3][w] & 0xffff0000u);
      } else {
        d[0] = (pz[0][w] & 0xffffu) | (pz[1][w] << 16);
        d[1] = (pz[2][w] & 0xffffu) | (pz[3][w] << 16);
      }
      st64(ZT + (4 * z_fq + e) * ZT_LD + 4 * z_tg, d);
    }
#pragma unroll
    for (int u = 0; u < RU; ++u) {
      const int ab = ib * RU + u;
#pragma unroll
      for (int qd = 0; qd < 4; ++qd) {
        u32x2 d;
        d[0] = fprt::pack_bf16x2(racc[u][4 * qd], racc[u][4 * qd + 1]);
        d[1] = fprt::pack_bf16x2(racc[u][4 * qd + 2], racc[u][4 * qd + 3]);
        st64(RT + (32 * nb + c) * RT_LD + 32 * ab + 8 * qd + 4 * g, d);
      }
    }
    fprt::block_sync();

    // -- next chunk's global loads fly during this chunk's math ------------------------
    const int pos_next = rev ? t0 : t1;
    const bool more = rev ? (pos_next > 0) : (pos_next < T);
    int t0n = 0, Ln = 0;
    if (more) {
      chunk_at(pos_next, t0n, Ln);
      prefetch(t0n, Ln);
    }

    // -- scores and P --------------------------------------------------------------------
    u32x4 xf[KS];
#pragma unroll
    for (int t = 0; t < KS; ++t) xf[t] = ld128(XS + (32 * ib + c) * X_LD + 16 * t + 8 * g);

    u32x4 pf_diag[2], pf_off[2];
    {
      f32x16 sc = {0};
#pragma unroll
      for (int t = 0; t < KS; ++t) {
        const u32x4 wf = ld128(WS + (32 * ib + c) * X_LD + 16 * t + 8 * g);
        sc = fprt::mfma_32x32x16_bf16(wf, xf[t], sc);
      }
#pragma unroll
      for (int t = 0; t < 2; ++t) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          pf_diag[t][e] = fprt::pack_bf16x2(sc[8 * t + 2 * e] * mw_diag[8 * t + 2 * e],
                                            sc[8 * t + 2 * e + 1] * mw_diag[8 * t + 2 * e + 1]);
        }
      }
    }
    if (need_off) {
      f32x16 sc = {0};
#pragma unroll
      for (int t = 0; t < KS; ++t) {
        const u32x4 wf = ld128(WS + (32 * jb_off + c) * X_LD + 16 * t + 8 * g);
        sc = fprt::mfma_32x32x16_bf16(wf, xf[t], sc);
      }
#pragma unroll
      for (int t = 0; t < 2; ++t) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          pf_off[t][e] = fprt::pack_bf16x2(sc[8 * t + 2 * e] * mw_off[8 * t + 2 * e],
                                           sc[8 * t + 2 * e + 1] * mw_off[8 * t + 2 * e + 1]);
        }
      }
    }

    // -- Z fragments: k-step kt covers tokens 16 kt .. 16 kt + 15 in the order P has them ---
    u32x4 zf[4];
#pragma unroll
    for (int kt = 0; kt < 4; ++kt) {
      const uint16_t* zp = ZT + (32 * nb + c) * ZT_LD + 16 * kt + 4 * g;
      const u32x2 lo = ld64(zp), hi = ld64(zp + 8);
      zf[kt] = u32x4{lo[0], lo[1], hi[0], hi[1]};
    }

    // -- Y = wread * (X R) + P Z -------------------------------------------------------------
    f32x16 yacc = {0};
#pragma unroll
    for (int t = 0; t < KS; ++t) {
      const u32x4 rf = ld128(RT + (32 * nb + c) * RT_LD + 16 * t + 8 * g);
      yacc = fprt::mfma_32x32x16_bf16(xf[t], rf, yacc);
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) yacc[r] *= wread[r];
#pragma unroll
    for (int t = 0; t < 2; ++t) yacc = fprt::mfma_32x32x16_bf16(pf_diag[t], ib ? zf[2 + t] : zf[t], yacc);
    if (need_off) {
#pragma unroll
      for (int t = 0; t < 2; ++t) yacc = fprt::mfma_32x32x16_bf16(pf_off[t], ib ? zf[t] : zf[2 + t], yacc);
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      reinterpret_cast<u16_m*>(YB)[(32 * ib + acc_row(r, g)) * YB_LD + 32 * nb + c] = float_to_bf16_bits(yacc[r]);
    }

    // -- R = gamma^L R + (wkey W)^T Z -----------------------------------------------------------
#pragma unroll
    for (int u = 0; u < RU; ++u) {
      const int ab = ib * RU + u;
#pragma unroll
      for (int r = 0; r < 16; ++r) racc[u][r] *= gL;
#pragma unroll
      for (int kt = 0; kt < 4; ++kt) {
        const uint16_t* wp = WT + (32 * ab + c) * WT_LD + 16 * kt + 4 * g;
        const u32x2 lo = ld64(wp), hi = ld64(wp + 8);
        racc[u] = fprt::mfma_32x32x16_bf16(u32x4{lo[0], lo[1], hi[0], hi[1]}, zf[kt], racc[u]);
      }
    }

    // state after every full block (forward walk)
    if (p.Bout && bs > 0 && (t1 % bs) == 0) {
      uint16_t* dst = p.Bout + (((size_t)b * p.nblk + (t1 / bs - 1)) * p.H + h) * mat;
#pragma unroll
      for (int u = 0; u < RU; ++u) {
#pragma unroll
        for (int r = 0; r < 16; ++r) dst[state_off(u, r)] = float_to_bf16_bits(racc[u][r]);
      }
    }
    fprt::block_sync();

    // -- Y tile: LDS -> global, 32 bytes per thread, rows beyond L dropped -------------------
    {
      const int row = tid >> 2, col = (tid & 3) * 16;
      if (row < L) {
        const uint16_t* src = YB + row * YB_LD + col;
        uint16_t* dst = Yg + (size_t)(t0 + row) * rowB + col;
        st128(dst, ld128(src));
        st128(dst + 8, ld128(src + 8));
      }
    }

    if (!more) break;
    t0 = t0n;
    L = Ln;
  }

  if (p.Rout) {
    uint16_t* dst = p.Rout + (size_t)bh * mat;
#pragma unroll
    for (int u = 0; u < RU; ++u) {
#pragma unroll
      for (int r = 0; r < 16; ++r) dst[state_off(u, r)] = float_to_bf16_bits(racc[u][r]);
    }
  }
}

}  // namespace fpk
