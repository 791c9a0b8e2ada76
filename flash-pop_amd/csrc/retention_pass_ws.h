// Wave-specialised retention pass (see pass_args.h for the recurrence), dA = 64 or 128.
//
// One workgroup of 8 wave64 owns one (batch, head) stream and one 64-column slice of
// Z / Y / R.  Hardware places waves w and w + 4 on the same SIMD, so every SIMD runs one
// wave of each role:
//
//   readout waves (0..3)  scores^T = W X^T -> P (bf16, in registers) ; Y^T = wread (R X^T) + Z^T P^T
//                         -> Y tile into LDS.  2 x 2 grid: `ib` = 32 chunk rows, `nb` = 32 columns.
//   state waves   (4..7)  all global traffic (bounds-checked buffer loads one chunk ahead in
//                         registers, Y tile stores), the transposes of W and Z into LDS, the
//                         state update R = gamma^L R + (wkey W)^T Z in fp32 accumulators and its
//                         bf16 copy for the read-out.
//
// LDS tiles are double-buffered: while the readout waves work on chunk i from stage i & 1 the
// state waves finish chunk i's state update and fill stage (i + 1) & 1 with chunk i + 1.  One
// workgroup barrier per chunk.  The weighted, transposed W tile is private to the state wave
// that both writes and reads it, so it needs no second buffer and no barrier.
#pragma once
#include "pass_args.h"
#include "retention_pass.h"   // ld/st helpers, acc_row

namespace fpk {

constexpr int NTHREADS_WS = 512;

constexpr int lds_bytes_ws(int dA) {
  return 2 * (4 * CH * (dA + 8)        // X and W tiles, two stages
              + 2 * BV * (CH + 4)      // Z transposed, two stages
              + 2 * BV * (dA + 8)      // bf16 copy of R (transposed), two stages
              + 2 * CH * (BV + 8)      // Y staging, two stages
              + 4 * 32 * (CH + 4));    // weighted W transposed, one 32-row slab per state wave
}

template <int DA>
FP_DEVICE void retention_pass_ws(const PassArgs& p, char* lds) {
  static_assert(DA == 64 || DA == 128, "wave-specialised pass: dA must be 64 or 128");
  constexpr int X_LD = DA + 8;
  constexpr int T_LD = CH + 4;      // row length of the transposed tiles (tokens)
  constexpr int RT_LD = DA + 8;
  constexpr int YB_LD = BV + 8;
  constexpr int KS = DA / 16;       // MFMA k-steps over dA
  constexpr int FG = DA / 8;        // 16-byte pieces per X row
  constexpr int NXP = CH * FG / 256;  // X pieces per state thread
  constexpr int NAB = DA / 32;      // 32-row blocks of R: 2 or 4
  constexpr int NNW = NAB == 4 ? 2 : 1;   // 32-column blocks of R per state wave

  uint16_t* const XS = reinterpret_cast<uint16_t*>(lds);
  uint16_t* const WS = XS + 2 * CH * X_LD;
  uint16_t* const ZT = WS + 2 * CH * X_LD;
  uint16_t* const RT = ZT + 2 * BV * T_LD;
  uint16_t* const YB = RT + 2 * BV * RT_LD;
  uint16_t* const WT = YB + 2 * CH * YB_LD;

  const int tid = fprt::thread_index();
  const int wave = tid >> 6, lane = tid & 63;
  const bool state_role = wave >= 4;
  const int g = lane >> 5, c = lane & 31;

  const int ntile = p.dB / BV;
  const int nwg = fprt::grid_size();
  int wg = fprt::block_index();
  if ((nwg & 7) == 0) wg = (wg & 7) * (nwg >> 3) + (wg >> 3);   // column tiles of a stream share an XCD
  const int tile = wg % ntile;
  const int bh = wg / ntile;
  const int h = bh % p.H, b = bh / p.H;

  const int T = p.T, bs = p.block;
  const bool rev = p.reverse != 0;
  const float lg = p.log2g[h];

  // chunk [t0, t0 + L) that follows position `pos` in walking order; never straddles a block boundary
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
  auto next_pos = [&](int t0, int L) { return rev ? t0 : t0 + L; };
  auto has_more = [&](int pos) { return rev ? pos > 0 : pos < T; };

  int t0, L;
  chunk_at(rev ? T : 0, t0, L);

  if (!state_role) {
    // =============================== readout waves ===============================
    const int ib = wave >> 1, nb = wave & 1;
    float mw_diag[16], mw_off[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int jl = acc_row(r, g);
      const int d = rev ? (jl - c) : (c - jl);
      mw_diag[r] = d >= 0 ? p.s_intra * fprt::exp2_approx((float)d * lg) : 0.f;
      mw_off[r] = p.s_intra * fprt::exp2_approx((float)(32 + d) * lg);
    }
    const bool need_off = rev ? (ib == 0) : (ib == 1);
    const int i_row = 32 * ib + c;                 // this lane's chunk row (query index)
    const int x_off = i_row * X_LD + 8 * g;
    const int wd_off = (32 * ib + c) * X_LD + 8 * g;
    const int wo_off = (32 * (1 - ib) + c) * X_LD + 8 * g;
    const int r_off = (32 * nb + c) * RT_LD + 8 * g;
    const int z_off = (32 * nb + c) * T_LD + 4 * g;
    const int y_off = i_row * YB_LD + 32 * nb + 4 * g;
    const float wread_fwd = p.s_read * fprt::exp2_approx((float)(i_row + 1) * lg);

    fprt::block_sync();   // stage 0 is filled
    for (int it = 0;; ++it) {
      const int s = it & 1;
      const uint16_t* xs = XS + s * CH * X_LD;
      const uint16_t* ws = WS + s * CH * X_LD;
      const uint16_t* zt = ZT + s * BV * T_LD;
      const uint16_t* rt = RT + s * BV * RT_LD;
      uint16_t* yb = YB + s * CH * YB_LD;

      float wread = wread_fwd;
      if (rev) {
        int e = L - 1 - i_row;
        if (e < 0) e = 0;
        wread = p.s_read * fprt::exp2_approx((float)e * lg);
      }

      u32x4 xf[KS];
#pragma unroll
      for (int t = 0; t < KS; ++t) xf[t] = ld128(xs + x_off + 16 * t);

      // read-out of the carried state: Y^T[n][i] = sum_a R[a][n] X[i][a]
      f32x16 yacc = {0};
#pragma unroll
      for (int t = 0; t < KS; ++t) yacc = fprt::mfma_32x32x16_bf16(ld128(rt + r_off + 16 * t), xf[t], yacc);

      // scores^T tiles -> P fragments
      u32x4 pf_diag[2], pf_off[2];
      {
        f32x16 sc = {0};
#pragma unroll
        for (int t = 0; t < KS; ++t) sc = fprt::mfma_32x32x16_bf16(ld128(ws + wd_off + 16 * t), xf[t], sc);
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
        for (int t = 0; t < KS; ++t) sc = fprt::mfma_32x32x16_bf16(ld128(ws + wo_off + 16 * t), xf[t], sc);
#pragma unroll
        for (int t = 0; t < 2; ++t) {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            pf_off[t][e] = fprt::pack_bf16x2(sc[8 * t + 2 * e] * mw_off[8 * t + 2 * e],
                                             sc[8 * t + 2 * e + 1] * mw_off[8 * t + 2 * e + 1]);
          }
        }
      }

#pragma unroll
      for (int r = 0; r < 16; ++r) yacc[r] *= wread;

      // Y^T += Z^T P^T ; k-step kt covers tokens 16 kt .. 16 kt + 15 in the order P holds them
      auto zfrag = [&](int kt) {
        const u32x2 lo = ld64(zt + z_off + 16 * kt), hi = ld64(zt + z_off + 16 * kt + 8);
        return u32x4{lo[0], lo[1], hi[0], hi[1]};
      };
#pragma unroll
      for (int t = 0; t < 2; ++t) yacc = fprt::mfma_32x32x16_bf16(zfrag(2 * ib + t), pf_diag[t], yacc);
      if (need_off) {
#pragma unroll
        for (int t = 0; t < 2; ++t) yacc = fprt::mfma_32x32x16_bf16(zfrag(2 * (1 - ib) + t), pf_off[t], yacc);
      }

      // accumulator element r holds column n = 32 nb + 8 (r / 4) + 4 g + r % 4 of row i_row
#pragma unroll
      for (int qd = 0; qd < 4; ++qd) {
        u32x2 d;
        d[0] = fprt::pack_bf16x2(yacc[4 * qd], yacc[4 * qd + 1]);
        d[1] = fprt::pack_bf16x2(yacc[4 * qd + 2], yacc[4 * qd + 3]);
        st64(yb + y_off + 8 * qd, d);
      }

      fprt::block_sync();
      const int pos = next_pos(t0, L);
      if (!has_more(pos)) break;
      chunk_at(pos, t0, L);
    }
    return;
  }

  // ================================= state waves =================================
  const int sub = wave & 3;
  const int rt_id = tid - 256;                       // 0..255 within the role
  const int ablk = NAB == 4 ? sub : (sub >> 1);      // 32-row block of R this wave owns
  const int nb0 = NAB == 4 ? 0 : (sub & 1);          // first 32-column block it owns
  const bool ws_writer = NAB == 4 || (sub & 1) == 0; // one wave per row block fills the row-major W tile
  uint16_t* const wt = WT + sub * 32 * T_LD;

  const uint32_t rowA = (uint32_t)p.H * p.dA * 2, rowB = (uint32_t)p.H * p.dB * 2;   // bytes
  const size_t streamA = ((size_t)b * T * p.H + h) * p.dA;
  const size_t streamB = ((size_t)b * T * p.H + h) * p.dB + (size_t)tile * BV;
  const uint16_t* const Xg = p.X + streamA;
  const uint16_t* const Wg = p.W + streamA;
  const uint16_t* const Zg = p.Z + streamB;
  uint16_t* const Yg = p.Y + streamB;
  const size_t mat = (size_t)p.dA * p.dB;

  // per-thread load coordinates (bytes relative to the chunk's first row)
  uint32_t xg_off[NXP];
  int xs_off[NXP];
#pragma unroll
  for (int u = 0; u < NXP; ++u) {
    const int q = rt_id + 256 * u, row = q / FG, col = q % FG;
    xg_off[u] = row * rowA + col * 16;
    xs_off[u] = row * X_LD + col * 8;
  }
  const int w_fg = lane & 3, w_tg = lane >> 2;       // W unit: tokens 4 w_tg.., features 32 ablk + 8 w_fg..
  const uint32_t wg_off = (4 * w_tg) * rowA + (32 * ablk + 8 * w_fg) * 2;
  const int ws_off = (4 * w_tg) * X_LD + 32 * ablk + 8 * w_fg;
  const int wt_off = (8 * w_fg) * T_LD + 4 * w_tg;
  const int z_tg = rt_id >> 4, z_fq = rt_id & 15;    // Z unit: tokens 4 z_tg.., columns 4 z_fq..
  const uint32_t zg_off = (4 * z_tg) * rowB + z_fq * 8;
  const int zt_off = (4 * z_fq) * T_LD + 4 * z_tg;
  const int y_row = rt_id >> 2, y_col = (rt_id & 3) * 16;

  u32x4 px[NXP], pw[4];
  u32x2 pz[4];
  auto prefetch = [&](int ct0, int cL) {
    // bytes from the stream base up to the end of the chunk's last row: later rows read as zero
    const uint32_t endA = (uint32_t)(ct0 + cL - 1) * rowA + p.dA * 2;
    const uint32_t endB = (uint32_t)(ct0 + cL - 1) * rowB + BV * 2;
    const fprt::BufView xb = fprt::make_buf(Xg, endA), wb = fprt::make_buf(Wg, endA), zb = fprt::make_buf(Zg, endB);
    const uint32_t baseA = (uint32_t)ct0 * rowA, baseB = (uint32_t)ct0 * rowB;
#pragma unroll
    for (int u = 0; u < NXP; ++u) px[u] = fprt::buf_load128(xb, baseA + xg_off[u]);
#pragma unroll
    for (int r = 0; r < 4; ++r) pw[r] = fprt::buf_load128(wb, baseA + wg_off + r * rowA);
#pragma unroll
    for (int r = 0; r < 4; ++r) pz[r] = fprt::buf_load64(zb, baseB + zg_off + r * rowB);
  };

  // state tiles: racc[nn] is R[32 ablk + acc_row][32 (nb0 + nn) + c]
  f32x16 racc[NNW];
  auto state_off = [&](int nn, int r) -> size_t {
    const int a = 32 * ablk + acc_row(r, g);
    const size_t n = (size_t)tile * BV + 32 * (nb0 + nn) + c;
    return (size_t)a * p.rs_a + n * p.rs_n;
  };
#pragma unroll
  for (int nn = 0; nn < NNW; ++nn) {
#pragma unroll
    for (int r = 0; r < 16; ++r) racc[nn][r] = p.R0 ? bf16_bits_to_float(p.R0[(size_t)bh * mat + state_off(nn, r)]) : 0.f;
  }
  // gradient of the block state that ends at token t1 joins R before that chunk is read out
  auto inject = [&](int t1) {
    if (p.Bin && bs > 0 && (t1 % bs) == 0) {
      const size_t base = (((size_t)b * p.nblk + (t1 / bs - 1)) * p.H + h) * mat;
#pragma unroll
      for (int nn = 0; nn < NNW; ++nn) {
#pragma unroll
        for (int r = 0; r < 16; ++r) racc[nn][r] += bf16_bits_to_float(p.Bin[base + state_off(nn, r)]);
      }
    }
  };

  // registers (chunk of length cL) + R -> LDS stage s
  int Lk_cached = -1;
  float wkey[4];
  auto fill_stage = [&](int s, int cL) {
    if (cL != Lk_cached) {
      Lk_cached = cL;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int j = 4 * w_tg + r;
        int e = rev ? (j + 1) : (cL - 1 - j);
        if (e < 0) e = 0;
        wkey[r] = p.s_update * fprt::exp2_approx((float)e * lg);
      }
    }
    uint16_t* xs = XS + s * CH * X_LD;
    uint16_t* ws = WS + s * CH * X_LD;
    uint16_t* zt = ZT + s * BV * T_LD;
    uint16_t* rt = RT + s * BV * RT_LD;
#pragma unroll
    for (int nn = 0; nn < NNW; ++nn) {
#pragma unroll
      for (int qd = 0; qd < 4; ++qd) {
        u32x2 d;
        d[0] = fprt::pack_bf16x2(racc[nn][4 * qd], racc[nn][4 * qd + 1]);
        d[1] = fprt::pack_bf16x2(racc[nn][4 * qd + 2], racc[nn][4 * qd + 3]);
        st64(rt + (32 * (nb0 + nn) + c) * RT_LD + 32 * ablk + 8 * qd + 4 * g, d);
      }
    }
#pragma unroll
    for (int u = 0; u < NXP; ++u) st128(xs + xs_off[u], px[u]);
    if (ws_writer) {
#pragma unroll
      for (int r = 0; r < 4; ++r) st128(ws + ws_off + r * X_LD, pw[r]);
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      u32x2 d;
      d[0] = fprt::pack_bf16x2(bf16_elem(pw[0], e) * wkey[0], bf16_elem(pw[1], e) * wkey[1]);
      d[1] = fprt::pack_bf16x2(bf16_elem(pw[2], e) * wkey[2], bf16_elem(pw[3], e) * wkey[3]);
      st64(wt + wt_off + e * T_LD, d);
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
      st64(zt + zt_off + e * T_LD, d);
    }
  };

  // Y tile of chunk [ct0, ct0 + cL) from LDS stage s to global; rows beyond cL are dropped
  auto store_y = [&](int s, int ct0, int cL) {
    const uint32_t endB = (uint32_t)(ct0 + cL - 1) * rowB + BV * 2;
    const fprt::BufView yv = fprt::make_buf(Yg, endB);
    const uint16_t* src = YB + s * CH * YB_LD + y_row * YB_LD + y_col;
    const uint32_t off = (uint32_t)(ct0 + y_row) * rowB + y_col * 2;
    fprt::buf_store128(yv, off, ld128(src));
    fprt::buf_store128(yv, off + 16, ld128(src + 8));
  };

  // ---- prologue: chunk 0 into stage 0, chunk 1 into registers ------------------------
  prefetch(t0, L);
  inject(t0 + L);
  fill_stage(0, L);
  int t0n = 0, Ln = 0;
  bool more = has_more(next_pos(t0, L));
  if (more) {
    chunk_at(next_pos(t0, L), t0n, Ln);
    prefetch(t0n, Ln);
  }
  fprt::block_sync();

  int t0p = 0, Lp = 0;   // previous chunk, whose Y tile is still in LDS
  int Lg_cached = -1;
  float gL = 1.f;
  for (int it = 0;; ++it) {
    const int s = it & 1;
    if (it > 0) store_y(s ^ 1, t0p, Lp);

    // R = gamma^L R + (wkey W)^T Z for chunk `it`
    if (L != Lg_cached) {
      Lg_cached = L;
      gL = fprt::exp2_approx((float)L * lg);
    }
    const uint16_t* zt = ZT + s * BV * T_LD;
#pragma unroll
    for (int nn = 0; nn < NNW; ++nn) {
#pragma unroll
      for (int r = 0; r < 16; ++r) racc[nn][r] *= gL;
    }
#pragma unroll
    for (int kt = 0; kt < 4; ++kt) {
      const uint16_t* wp = wt + c * T_LD + 16 * kt + 4 * g;
      const u32x2 wlo = ld64(wp), whi = ld64(wp + 8);
      const u32x4 wf = {wlo[0], wlo[1], whi[0], whi[1]};
#pragma unroll
      for (int nn = 0; nn < NNW; ++nn) {
        const uint16_t* zp = zt + (32 * (nb0 + nn) + c) * T_LD + 16 * kt + 4 * g;
        const u32x2 zlo = ld64(zp), zhi = ld64(zp + 8);
        racc[nn] = fprt::mfma_32x32x16_bf16(wf, u32x4{zlo[0], zlo[1], zhi[0], zhi[1]}, racc[nn]);
      }
    }

    // state after every full block (forward walk)
    const int t1 = t0 + L;
    if (p.Bout && bs > 0 && (t1 % bs) == 0) {
      uint16_t* dst = p.Bout + (((size_t)b * p.nblk + (t1 / bs - 1)) * p.H + h) * mat;
#pragma unroll
      for (int nn = 0; nn < NNW; ++nn) {
#pragma unroll
        for (int r = 0; r < 16; ++r) dst[state_off(nn, r)] = float_to_bf16_bits(racc[nn][r]);
      }
    }

    t0p = t0;
    Lp = L;
    if (more) {
      inject(t0n + Ln);
      fill_stage(s ^ 1, Ln);
      t0 = t0n;
      L = Ln;
      more = has_more(next_pos(t0, L));
      if (more) {
        chunk_at(next_pos(t0, L), t0n, Ln);
        prefetch(t0n, Ln);
      }
      fprt::block_sync();
    } else {
      fprt::block_sync();
      store_y(s, t0p, Lp);
      break;
    }
  }

  if (p.Rout) {
    uint16_t* dst = p.Rout + (size_t)bh * mat;
#pragma unroll
    for (int nn = 0; nn < NNW; ++nn) {
#pragma unroll
      for (int r = 0; r < 16; ++r) dst[state_off(nn, r)] = float_to_bf16_bits(racc[nn][r]);
    }
  }
}

}  // namespace fpk
