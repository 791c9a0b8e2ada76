// Wave-specialised retention pass (see pass_args.h for the recurrence): dA = 64 or 128 per visit,
// dA = 256 in two visits per chunk, dA = 192 in three (NH below).
//
// One workgroup of 8 wave64 owns one (batch, head) stream and one 64-column slice of
// Z / Y / R.  Hardware places waves w and w + 4 on the same SIMD, so every SIMD runs one
// wave of each role:
//
//   readout waves (0..3)  scores^T = W X^T -> P (bf16) ; Y^T = wread (R X^T) + Z^T P^T -> Y tile
//                         into LDS.  2 x 2 grid: `ib` = 32 chunk rows, `nb` = 32 columns.  The
//                         rows of a block meet two 32 x 32 score tiles: the diagonal one, whose
//                         masked half is cleared after conversion, and one that lies wholly inside
//                         or wholly outside the decay window.  Every live tile is computed once,
//                         the diagonal one by the wave with nb = 0 and the other one by the wave
//                         with nb = 1, and handed to the partner wave of the row block through a
//                         2 KB LDS tile in operand layout (a barrier in the middle of the item).
//                         The loop has no data-dependent branches; it exists in three copies (two
//                         live tiles; one, made here; one, made by the partner).
//                         They also feed X and Z: bounds-checked buffer loads into registers, X
//                         copied and Z transposed into LDS one chunk ahead, and they store the Y
//                         tile of the previous chunk.
//   state waves   (4..7)  the W traffic (loads, row-major copy and the weighted transpose into
//                         LDS), the state update R = gamma^L R + (wkey W)^T Z in fp32
//                         accumulators and its bf16 copy for the read-out, block states.
// Each role has one set of load registers: as soon as chunk i + 1 has gone from it into LDS
// (during chunk i), the loads of chunk i + 2 are issued into it, in the shadow of the MFMAs; they
// have a whole chunk time to arrive.  (A second set, loaded a chunk earlier, was slower.)
// The split keeps the two roles' instruction streams about equally long.
//
// LDS tiles are double-buffered: while the readout waves work on chunk i from stage i & 1 the
// state waves finish chunk i's state update and fill stage (i + 1) & 1 with chunk i + 1.  One
// workgroup barrier ends a chunk and one in its middle publishes the P tiles.  The weighted,
// transposed W tile is private to the state wave that both writes and reads it, so it needs no
// second buffer and no barrier.
//
// Within a chunk the code is laid out in phases separated by scheduling fences: all LDS
// operands of a phase are requested first, the MFMAs that consume them follow back to back,
// and the vector work of one phase sits in the shadow of the next phase's MFMAs.
#pragma once
#include "pass_args.h"
#include "lds_access.h"

namespace fpk {

constexpr int NTHREADS_WS = 512;

constexpr int lds_bytes_ws(int dA) {
  return 2 * (4 * CH * (dA + 8)        // X and W tiles, two stages
              + 2 * BV * (CH + 4)      // Z transposed, two stages
              + 2 * BV * (dA + 8)      // bf16 copy of R (transposed), two stages
              + 2 * CH * (BV + 8)      // Y staging, two stages
              + 4 * 32 * (CH + 4)      // weighted W transposed, one 32-row slab per state wave
              + 3 * 32 * 32);          // P tiles handed between the readout waves of a row block
}

template <int H>
struct Half {
  static constexpr int value = H;
};

// Calls visit(part, it) for it = 0, 1, ... until it returns false, `part` being the visit's place in
// the cycle of NH visits per chunk as a type (Half<it % NH>; with one visit per chunk the two
// copies are the same code).  The LDS stage of a visit is it & 1, so a cycle of three is written
// out over six visits.
template <int NH, typename Visit>
FP_DEVICE void walk_visits(Visit&& visit) {
  if constexpr (NH == 3) {
    for (int it = 0;; it += 6) {
      if (!visit(Half<0>{}, it)) break;
      if (!visit(Half<1>{}, it + 1)) break;
      if (!visit(Half<2>{}, it + 2)) break;
      if (!visit(Half<0>{}, it + 3)) break;
      if (!visit(Half<1>{}, it + 4)) break;
      if (!visit(Half<2>{}, it + 5)) break;
    }
  } else {
    static_assert(NH == 1 || NH == 2, "one, two or three visits per chunk");
    for (int it = 0;; it += 2) {
      if (!visit(Half<0>{}, it)) break;
      if (!visit(Half<1>{}, it + 1)) break;
    }
  }
}

// two 8-byte LDS reads that form one MFMA operand: tokens 16 kt + 4 g + {0..3} and + 8
FP_DEVICE u32x4 ld_token_frag(const uint16_t* p) {
  const u32x2 lo = ld64(p), hi = ld64(p + 8);
  return u32x4{lo[0], lo[1], hi[0], hi[1]};
}

// Variants of the walk, one instantiation each so that the plain one stays lean:
// WALK_BLOCKS  the pass writes block states (Bout) or reads their gradients (Bin);
// WALK_MULTI   a workgroup walks several batch entries (p.slots < p.B), so that short sequences
//              keep the load pipeline full across sequence boundaries;
// WALK_SUFFIX  a suffix of p.Ls <= CH tokens hangs off every block boundary (positions 0, block,
//              ..., T; T is a multiple of the block size).  It is one more item of the walk, placed at
//              its boundary, with its own tensors: it reads the state at the boundary without
//              advancing it.  Walking forward its keys stay out of R and R is not decayed; walking
//              backward its read-out weight is 0 and what it adds to R (the gradient of the state
//              it read) is not decayed either.
// WALK_SUFFIX_ANY  the same for any T and any p.Ls: tokens after the last block boundary are
//              walked as context with no suffix behind them (Rout, forward, and R0, backward,
//              then belong to the state at that boundary), and a suffix of more than CH tokens
//              is walked in parts on a copy of the state.
// WALK_STATE   like WALK_MULTI, but only the final R of every sequence is wanted (p.state_only):
//              the readout waves feed Z and do nothing else, X is not read and Y not written.
enum Walk { WALK_PLAIN = 0, WALK_BLOCKS = 1, WALK_MULTI = 2, WALK_SUFFIX = 3, WALK_STATE = 4, WALK_SUFFIX_ANY = 5 };

// NH > 1 handles a contraction width of NH * DA (p.dA = 256 as 2 x 128, p.dA = 192 as 3 x 64) with the
// LDS footprint of DA: every chunk is visited NH times, once per part of the columns of X and W (of the rows of R).
// Scores and read-out are sums over the contraction index, so the readout waves simply keep
// accumulating across the two visits and convert, multiply by Z and store only after the second;
// the state waves carry one set of accumulators per half and update the half being visited.
template <int DA, int MODE, int NH = 1>
// `nwg` workgroups run this pass and this one is number `wg` of them (the launch may hold the
// workgroups of other passes as well).  `io` are the tensors, walking direction and scales of
// this pass, by value: in a launch of several passes they are chosen per workgroup, everything
// else in `p` is common to all of them.
FP_DEVICE void retention_pass_ws(const PassArgs& p, const PassTensors& io, char* lds, int wg, int nwg) {
  static_assert(DA == 64 || DA == 128, "wave-specialised pass: dA must be 64 or 128");
  static_assert(NH == 1 || MODE != WALK_MULTI, "two halves: not with several sequences per workgroup and a read-out");
  constexpr bool STATE = MODE == WALK_STATE;
  constexpr bool BLOCKS = MODE == WALK_BLOCKS, MULTI = MODE == WALK_MULTI || STATE;
  constexpr bool SFX_ANY = MODE == WALK_SUFFIX_ANY, SFX = MODE == WALK_SUFFIX || SFX_ANY;
  constexpr int X_LD = DA + 8;
  constexpr int T_LD = CH + 4;      // row length of the transposed tiles (tokens)
  constexpr int RT_LD = DA + 8;
  constexpr int YB_LD = BV + 8;
  constexpr int KS = DA / 16;       // MFMA k-steps over dA
  constexpr int FG = DA / 8;        // 16-byte pieces per X row
  constexpr int NXP = CH * FG / 256;  // X pieces per readout thread
  constexpr int NAB = DA / 32;      // 32-row blocks of R: 2 or 4
  constexpr int NNW = NAB == 4 ? 2 : 1;   // 32-column blocks of R per state wave

  uint16_t* const XS = reinterpret_cast<uint16_t*>(lds);
  uint16_t* const WS = XS + 2 * CH * X_LD;
  uint16_t* const ZT = WS + 2 * CH * X_LD;
  uint16_t* const RT = ZT + 2 * BV * T_LD;
  uint16_t* const YB = RT + 2 * BV * RT_LD;
  uint16_t* const WT = YB + 2 * CH * YB_LD;
  uint16_t* const PB = WT + 4 * 32 * T_LD;   // [diagonal tile of row block 0, of row block 1, the other tile][k-step][lane]

  const int tid = fprt::thread_index();
  const int wave = tid >> 6, lane = tid & 63;
  const bool state_role = wave >= 4;
  const int g = lane >> 5, c = lane & 31;

  const int ntile = p.dB / BV;
  const int tile = wg % ntile;
  const int h = (wg / ntile) % p.H;
  const int slot = (wg / ntile) / p.H;   // first batch entry of this workgroup

  const int T = p.T;
  const int bs = (BLOCKS || SFX) ? p.block : 0;   // only these walks cut chunks at block boundaries
  const bool rev = io.reverse != 0;
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

  // The walk: all chunks of batch entry `slot`, then of slot + slots, ... Both roles step
  // through the same list.
  struct Chunk {
    int b, t0, L;
    bool ok, first, last;   // exists / first item of its sequence / last item of its sequence
    bool sfx;               // a suffix (t0 is its block boundary) rather than a context chunk
    int n;                  // WALK_SUFFIX only: index of the suffix, or of the context chunk's block
    int part;               // WALK_SUFFIX only: which CH tokens of a suffix longer than a chunk (0 otherwise)
    int h;                  // NH = 2 only: which half of the contraction this visit covers
    uint32_t row;           // index of the item's first row among all rows of its tensor
  };
  const Chunk no_chunk = {0, 0, 0, false, false, false, false, 0, 0, 0, 0u};
  // A suffix of more than CH tokens is walked in parts of CH tokens (the last one shorter), in
  // walking order; between its parts the state moves on as between context chunks, on a copy.
  const int sfx_parts = SFX_ANY ? (p.Ls + CH - 1) / CH : 1;
  auto part_len = [&](int part) { return p.Ls - CH * part < CH ? p.Ls - CH * part : CH; };
  auto with_row = [&](Chunk ck) {
    ck.row = (SFX && ck.sfx) ? ((uint32_t)ck.b * (p.nblk + 1) + ck.n) * p.Ls + CH * ck.part : (uint32_t)ck.b * T + ck.t0;
    return ck;
  };
  // the part of suffix n at boundary `pos` that the walk meets first
  auto enter_suffix = [&](Chunk& ck, int n, int pos, bool ends_walk) {
    ck.sfx = true;
    ck.n = n;
    ck.t0 = pos;
    ck.part = rev ? sfx_parts - 1 : 0;
    ck.L = part_len(ck.part);
    ck.last = ends_walk && sfx_parts == 1;
  };
  auto first_chunk = [&](int b) {
    Chunk ck = {b, 0, 0, b < p.B, true, false, false, 0, 0};
    if (ck.ok) {
      if (SFX_ANY && rev && T > p.nblk * bs) {   // tokens after the last boundary: the walk back starts with them
        ck.n = p.nblk;
        ck.t0 = T - CH > p.nblk * bs ? T - CH : p.nblk * bs;
        ck.L = T - ck.t0;
      } else if (SFX) {   // the suffix at the first boundary met: position 0, or T walking backward
        enter_suffix(ck, rev ? p.nblk : 0, rev ? T : 0, false);
      } else {
        chunk_at(rev ? T : 0, ck.t0, ck.L);
        ck.last = !has_more(next_pos(ck.t0, ck.L));
      }
    }
    return with_row(ck);
  };
  auto chunk_after = [&](const Chunk& ck) {
    if (!ck.ok) return ck;
    if (NH > 1 && ck.h < NH - 1) {   // the same chunk again, next part of the contraction
      Chunk again = ck;
      again.h = ck.h + 1;
      again.first = false;
      return again;
    }
    if (ck.last) return MULTI ? first_chunk(ck.b + p.slots) : no_chunk;
    Chunk n = {ck.b, 0, 0, true, false, false, false, 0, 0};
    if (SFX_ANY && ck.sfx && (rev ? ck.part > 0 : ck.part < sfx_parts - 1)) {   // the next part of the same suffix
      n = ck;
      n.first = false;
      n.h = 0;
      n.part = rev ? ck.part - 1 : ck.part + 1;
      n.L = part_len(n.part);
      // the walk ends with the last part of the suffix at position T (forward) or 0 (backward)
      n.last = (rev ? n.part == 0 && ck.t0 == 0 : n.part == sfx_parts - 1 && ck.t0 == T);
      return with_row(n);
    }
    if (SFX) {
      // Block m spans [m bs, (m + 1) bs); the tokens after the last boundary, if any, form a
      // shorter block nblk that ends the walk without a suffix.  After a suffix comes the nearest
      // context chunk of the block that follows it in walking order; after the context chunk that
      // reaches the far boundary of its block comes that boundary's suffix.
      if (!rev) {
        const int m = ck.n, pos = ck.sfx ? ck.t0 : ck.t0 + ck.L, lim = (!SFX_ANY || (m + 1) * bs < T) ? (m + 1) * bs : T;
        if (!ck.sfx && pos == lim) {
          enter_suffix(n, m + 1, pos, pos == T);
        } else {
          n.n = m; n.t0 = pos; n.L = (pos + CH < lim ? pos + CH : lim) - pos;
          n.last = SFX_ANY && m == p.nblk && pos + n.L == T;
        }
      } else {
        const int m = ck.sfx ? ck.n - 1 : ck.n, pos = ck.t0, lo = m * bs;
        if (!ck.sfx && pos == lo) {
          enter_suffix(n, m, pos, pos == 0);
        } else {
          n.n = m; n.t0 = pos - CH > lo ? pos - CH : lo; n.L = pos - n.t0;
        }
      }
      return with_row(n);
    }
    chunk_at(next_pos(ck.t0, ck.L), n.t0, n.L);
    n.last = !has_more(next_pos(n.t0, n.L));
    return with_row(n);
  };

  const uint32_t rowA = (uint32_t)p.H * p.dA * 2, rowB = (uint32_t)p.H * p.dB * 2;   // row pitch in bytes
  // byte offset of the item's first row for head h in an [B,T,H,dA] tensor (suffixes:
  // [B, nblk + 1, Ls, H, dA]), resp. of this tile's columns in the dB-wide tensors: one 32 x 32 -> 64
  // bit multiply each (a tensor has fewer than 2^32 rows)
  const uint32_t headA = (uint32_t)h * p.dA * 2, headB = ((uint32_t)h * p.dB + (uint32_t)tile * BV) * 2;
  auto rowsA = [&](const Chunk& ck) { return (size_t)ck.row * rowA + headA + (NH > 1 ? ck.h * DA * 2 : 0); };
  auto rowsB = [&](const Chunk& ck) { return (size_t)ck.row * rowB + headB; };

  if (!state_role) {
    // =============================== readout waves ===============================
    const int ib = wave >> 1, nb = wave & 1;
    // The rows of block `ib` meet two 32-token score tiles: the "diagonal" one (tokens 32 ib ..),
    // half masked, and the "other" one (tokens 32 (1 - ib) ..), which lies either wholly inside
    // the decay window or wholly outside it.  Each live tile is computed once: the diagonal one
    // by the wave with nb = 0, the other one by the wave with nb = 1, and handed to the partner
    // wave of the row block through LDS (the accumulator layout of scores^T is, lane for lane,
    // the operand layout of the next product in both waves).  Masked scores are zeroed by
    // clearing their bits after the bf16 conversion, so that inf or nan in a masked operand
    // cannot leak through 0 * x.
    const bool other_live = rev ? (ib == 0) : (ib == 1);
    const bool makes_diag = nb == 0;
    float mw[16];          // decay weights of the tile this wave computes
    uint32_t keep[8];      // bits to keep after conversion (all of them off the diagonal)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int jl = acc_row(r, g);
      const int d = rev ? (jl - c) : (c - jl);          // distance inside the diagonal tile
      mw[r] = io.s_intra * fprt::exp2_approx((float)(makes_diag ? (d >= 0 ? d : 0) : 32 + d) * lg);
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int d0 = rev ? (acc_row(2 * e, g) - c) : (c - acc_row(2 * e, g));
      const int d1 = rev ? (acc_row(2 * e + 1, g) - c) : (c - acc_row(2 * e + 1, g));
      keep[e] = makes_diag ? ((d0 >= 0 ? 0x0000ffffu : 0u) | (d1 >= 0 ? 0xffff0000u : 0u)) : 0xffffffffu;
    }
    const int i_row = 32 * ib + c;                 // this lane's chunk row (query index)
    const int x_off = i_row * X_LD + 8 * g;
    const int w_off = (32 * (makes_diag ? ib : 1 - ib) + c) * X_LD + 8 * g;   // W rows of this wave's score tile
    uint16_t* const p_mine = PB + (makes_diag ? ib : 2) * 1024 + lane * 8;      // + 512 per k-step
    const uint16_t* const p_theirs = PB + (makes_diag ? 2 : ib) * 1024 + lane * 8;
    const int r_off = (32 * nb + c) * RT_LD + 8 * g;
    // Z^T fragments: the tokens of the tile this wave makes, and of the tile it is handed
    const int zm_off = (32 * nb + c) * T_LD + 4 * g + 32 * (makes_diag ? ib : 1 - ib);
    const int zh_off = (32 * nb + c) * T_LD + 4 * g + 32 * (makes_diag ? 1 - ib : ib);
    const int y_off = i_row * YB_LD + 32 * nb + 4 * g;
    const float wread_fwd = io.s_read * fprt::exp2_approx((float)(i_row + 1) * lg);

    // ---- feeding X, Z and draining Y: coordinates of this thread, bytes from the chunk's first row
    const char* const Xg = reinterpret_cast<const char*>(io.X);
    const char* const Zg = reinterpret_cast<const char*>(io.Z);
    char* const Yg = reinterpret_cast<char*>(io.Y);
    const char* const Xsg = reinterpret_cast<const char*>(io.Xs);
    const char* const Zsg = reinterpret_cast<const char*>(io.Zs);
    char* const Ysg = reinterpret_cast<char*>(io.Ys);
    uint32_t xg_off[NXP];
    int xs_off[NXP];
#pragma unroll
    for (int u = 0; u < NXP; ++u) {
      const int q = tid + 256 * u, row = q / FG, col = q % FG;
      xg_off[u] = row * rowA + col * 16;
      xs_off[u] = row * X_LD + col * 8;
    }
    const int z_tg = tid >> 4, z_fq = tid & 15;      // Z unit: tokens 4 z_tg.., columns 4 z_fq..
    uint32_t zg_off[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) zg_off[r] = (4 * z_tg + r) * rowB + z_fq * 8;
    const int zt_off = (4 * z_fq) * T_LD + 4 * z_tg;
    const int y_row = tid >> 2, y_col = (tid & 3) * 16;
    const uint32_t yg_off = y_row * rowB + y_col * 2;

    // Loads and stores are issued unconditionally (zero-length views when there is nothing to
    // do): exact wait counts.
    struct FeedRegs {
      u32x4 x[NXP];
      u32x2 z[4];
    };
    auto feed_load_x = [&](FeedRegs& fr, const Chunk& c2) {
      const bool live = c2.ok && !STATE;
      const uint32_t lenA = live ? (uint32_t)(c2.L - 1) * rowA + DA * 2 : 0u;
      const fprt::BufView xv = fprt::make_buf(((SFX && c2.sfx) ? Xsg : Xg) + (live ? rowsA(c2) : 0), lenA);
#pragma unroll
      for (int u = 0; u < NXP; ++u) fr.x[u] = fprt::buf_load128(xv, xg_off[u]);
    };
    auto feed_load_z = [&](FeedRegs& fr, const Chunk& c2) {
      const bool live = c2.ok;
      const uint32_t lenB = live ? (uint32_t)(c2.L - 1) * rowB + BV * 2 : 0u;
      const fprt::BufView zv = fprt::make_buf(((SFX && c2.sfx) ? Zsg : Zg) + (live ? rowsB(c2) : 0), lenB);
#pragma unroll
      for (int r = 0; r < 4; ++r) fr.z[r] = fprt::buf_load64(zv, zg_off[r]);
    };
    auto feed_store_x = [&](const FeedRegs& fr, int s) {
      uint16_t* xs = XS + s * CH * X_LD;
#pragma unroll
      for (int u = 0; u < NXP; ++u) st128(xs + xs_off[u], fr.x[u]);
    };
    auto feed_store_z = [&](const FeedRegs& fr, int s) {
      uint16_t* zt = ZT + s * BV * T_LD;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int w = e >> 1;
        u32x2 d;
        if (e & 1) {
          d[0] = (fr.z[0][w] >> 16) | (fr.z[1][w] & 0xffff0000u);
          d[1] = (fr.z[2][w] >> 16) | (fr.z[3][w] & 0xffff0000u);
        } else {
          d[0] = (fr.z[0][w] & 0xffffu) | (fr.z[1][w] << 16);
          d[1] = (fr.z[2][w] & 0xffffu) | (fr.z[3][w] << 16);
        }
        st64(zt + zt_off + e * T_LD, d);
      }
    };
    // Y tile of chunk c2 from LDS stage s to global; rows beyond its length are dropped
    auto drain_y = [&](const Chunk& c2, int s) {
      const uint16_t* src = YB + s * CH * YB_LD + y_row * YB_LD + y_col;
      const u32x4 v0 = ld128(src), v1 = ld128(src + 8);
      const bool live = c2.ok && !STATE;
      const fprt::BufView yv = fprt::make_buf(((SFX && c2.sfx) ? Ysg : Yg) + (live ? rowsB(c2) : 0),
                                              live ? (uint32_t)(c2.L - 1) * rowB + BV * 2 : 0u);
      // non-temporal: outputs are not read back by this launch and need not displace its inputs in the caches
      fprt::buf_store128_nt(yv, yg_off, v0);
      fprt::buf_store128_nt(yv, yg_off + 16, v1);
    };

    Chunk ck = first_chunk(slot), ck1 = chunk_after(ck), ckp = no_chunk;
    FeedRegs feed;
    feed_load_x(feed, ck);
    feed_load_z(feed, ck);
    feed_store_x(feed, 0);
    feed_store_z(feed, 0);
    feed_load_x(feed, ck1);
    feed_load_z(feed, ck1);
    fprt::block_sync();   // stage 0 is filled, item 1 is on its way

    // One item.  `feed` holds item it + 1 on entry; once its parts have gone into LDS they are
    // reloaded with item it + 2.  Returns false after the last item.  `half` is the parity of `it`
    // as a type: with NH = 2 the first visit of a chunk opens the accumulators and the second
    // closes them; with NH = 1 every visit does both.
    f32x16 yacc, sc;
    // `makes`: this wave computes a score tile.  `both`: the rows of this wave see two live tiles.
    auto iteration = [&](auto half, auto makes_c, auto both_c, int it) -> bool {
      constexpr int HF = decltype(half)::value;
      constexpr bool MAKES = decltype(makes_c)::value, BOTH = decltype(both_c)::value;
      constexpr bool opens = NH == 1 || HF == 0, closes = NH == 1 || HF == NH - 1;
      const int s = it & 1;
      const int L = ck.L;
      const Chunk ck2 = chunk_after(ck1);
      if (!STATE) drain_y(ckp, s ^ 1);
      const uint16_t* xs = XS + s * CH * X_LD;
      const uint16_t* ws = WS + s * CH * X_LD;
      const uint16_t* zt = ZT + s * BV * T_LD;
      const uint16_t* rt = RT + s * BV * RT_LD;
      uint16_t* yb = YB + s * CH * YB_LD;

      float wread = wread_fwd;
      if (rev) {
        int e = L - 1 - i_row;
        if (e < 0) e = 0;
        wread = io.s_read * fprt::exp2_approx((float)e * lg);
        // nothing downstream of a suffix reaches back into it: its last tokens meet a zero gradient state
        if (SFX && ck.sfx && ck.part == sfx_parts - 1) wread = 0.f;
      }

      if (STATE) {   // feed Z for the state waves, nothing else
        feed_store_z(feed, s ^ 1);
        feed_load_z(feed, ck2);
        fprt::block_sync();
        ckp = ck;
        ck = ck1;
        ck1 = ck2;
        return ck.ok;
      }
      // ---- phase 0: request X, R and the W rows of this wave's score tile
      u32x4 xf[KS], rf[KS], wf[KS], zm[2], zh[2];
#pragma unroll
      for (int t = 0; t < KS; ++t) {
        xf[t] = ld128(xs + x_off + 16 * t);
        rf[t] = ld128(rt + r_off + 16 * t);
      }
      if (MAKES) {
#pragma unroll
        for (int t = 0; t < KS; ++t) wf[t] = ld128(ws + w_off + 16 * t);
      }
      fprt::sched_fence();

      // ---- phase 1: read-out of the carried state, Y^T[n][i] = sum_a R[a][n] X[i][a]
      if (opens) yacc = f32x16{0};
#pragma unroll
      for (int t = 0; t < KS; ++t) yacc = fprt::mfma_32x32x16_bf16(rf[t], xf[t], yacc);
      fprt::sched_fence();

      // ---- phase 2: scores^T of this wave's tile; Z arrives meanwhile; X of chunk it + 1 goes
      // to the other stage
      if (closes) {
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          if (MAKES) zm[t] = ld_token_frag(zt + zm_off + 16 * t);
          if (BOTH || !MAKES) zh[t] = ld_token_frag(zt + zh_off + 16 * t);
        }
      }
      if (MAKES) {
        if (opens) sc = f32x16{0};
#pragma unroll
        for (int t = 0; t < KS; ++t) sc = fprt::mfma_32x32x16_bf16(wf[t], xf[t], sc);
      }
      feed_store_x(feed, s ^ 1);
      feed_load_x(feed, ck2);
      fprt::sched_fence();

      // ---- phase 3: the read-out is scaled, P converted and put where the partner wave finds
      // it, and Z of chunk it + 1 is transposed into the other stage.  Accumulator element
      // r = 8 t + e is token 16 t + 8 (e / 4) + 4 g + e % 4 of its tile, the order the Z
      // fragments are read in.
      u32x4 pm[2], pt[2];
      if (closes) {
#pragma unroll
        for (int r = 0; r < 16; ++r) yacc[r] *= wread;
        if (MAKES) {
#pragma unroll
          for (int t = 0; t < 2; ++t) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const int r = 8 * t + 2 * e;
              pm[t][e] = fprt::pack_bf16x2(sc[r] * mw[r], sc[r + 1] * mw[r + 1]) & keep[4 * t + e];
            }
            st128(p_mine + 512 * t, pm[t]);
          }
        }
      }
      feed_store_z(feed, s ^ 1);
      feed_load_z(feed, ck2);
      fprt::sched_fence();
      if (!closes) {   // first half of the contraction: nothing to finish yet
        fprt::block_sync();
        ckp = no_chunk;
        ck = ck1;
        ck1 = ck2;
        return true;
      }
      fprt::block_sync();   // every P tile of this chunk is in LDS

      // ---- phase 4: Y^T += Z^T P^T with the own tile from registers and the partner's from LDS.
      // A wave that made the diagonal tile gets the other one, and the other way round; a wave
      // that made nothing gets the diagonal one.
      if (BOTH || !MAKES) {
#pragma unroll
        for (int t = 0; t < 2; ++t) pt[t] = ld128(p_theirs + 512 * t);
      }
      if (MAKES) {
#pragma unroll
        for (int t = 0; t < 2; ++t) yacc = fprt::mfma_32x32x16_bf16(zm[t], pm[t], yacc);
      }
      if (BOTH || !MAKES) {
#pragma unroll
        for (int t = 0; t < 2; ++t) yacc = fprt::mfma_32x32x16_bf16(zh[t], pt[t], yacc);
      }
      fprt::sched_fence();

      // accumulator element r holds column n = 32 nb + 8 (r / 4) + 4 g + r % 4 of row i_row
#pragma unroll
      for (int qd = 0; qd < 4; ++qd) {
        u32x2 d;
        d[0] = fprt::pack_bf16x2(yacc[4 * qd], yacc[4 * qd + 1]);
        d[1] = fprt::pack_bf16x2(yacc[4 * qd + 2], yacc[4 * qd + 3]);
        st64(yb + y_off + 8 * qd, d);
      }

      fprt::block_sync();
      ckp = ck;
      ck = ck1;
      ck1 = ck2;
      if (!ck.ok) drain_y(ckp, s);   // the last Y tile
      return ck.ok;
    };
    // Three copies of the loop, chosen once per wave: two live tiles and this wave makes one of
    // them; one live tile made by this wave; one live tile made by the partner.
    if (other_live) {
      walk_visits<NH>([&](auto part, int it) { return iteration(part, Half<1>{}, Half<1>{}, it); });
    } else if (makes_diag) {
      walk_visits<NH>([&](auto part, int it) { return iteration(part, Half<1>{}, Half<0>{}, it); });
    } else {
      walk_visits<NH>([&](auto part, int it) { return iteration(part, Half<0>{}, Half<0>{}, it); });
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

  const char* const Wg = reinterpret_cast<const char*>(io.W);
  const char* const Wsg = reinterpret_cast<const char*>(io.Ws);
  const size_t mat = (size_t)p.dA * p.dB;

  // per-thread coordinates, bytes relative to the chunk's first row; they never change
  const int w_fg = lane & 3, w_tg = lane >> 2;       // W unit: tokens 4 w_tg.., features 32 ablk + 8 w_fg..
  uint32_t wg_off[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) wg_off[r] = (4 * w_tg + r) * rowA + (32 * ablk + 8 * w_fg) * 2;
  const int ws_off = (4 * w_tg) * X_LD + 32 * ablk + 8 * w_fg;
  const int wt_off = (8 * w_fg) * T_LD + 4 * w_tg;

  struct ChunkRegs {
    u32x4 w[4];
  };
  ChunkRegs wregs;
  // Loads are issued unconditionally so that the number of outstanding memory operations is the
  // same in every iteration; a chunk that does not exist gets zero-length views (no traffic).
  auto prefetch = [&](ChunkRegs& cr, const Chunk& ck) {
    // views that start at the chunk's first row and end with its last: later rows read as zero
    const bool live = ck.ok;
    const uint32_t lenA = live ? (uint32_t)(ck.L - 1) * rowA + DA * 2 : 0u;
    const fprt::BufView wb = fprt::make_buf(((SFX && ck.sfx) ? Wsg : Wg) + (live ? rowsA(ck) : 0), lenA);
#pragma unroll
    for (int r = 0; r < 4; ++r) cr.w[r] = fprt::buf_load128(wb, wg_off[r]);
  };

  // state tiles: racc[hf][nn] is R[DA hf + 32 ablk + acc_row][32 (nb0 + nn) + c]
  f32x16 racc[NH][NNW];
#pragma unroll
  for (int hf = 0; hf < NH; ++hf) {
#pragma unroll
    for (int nn = 0; nn < NNW; ++nn) racc[hf][nn] = f32x16{0};
  }

  // ---- this wave's tile of a state matrix <-> global memory --------------------------------
  // Global accesses are 16 bytes per lane along the contiguous direction of the matrix; the
  // change to and from the accumulator layout goes through the part of an R staging buffer that
  // only this wave writes (rows 32 nb0 .., columns 32 ablk ..), so no barrier is involved.  In
  // the staging area the tile is kept in the order of the global matrix: for R = S that is
  // [a][n] (one accumulator element per 2-byte access), for R = S^T it is [n][a], which is also
  // the natural order of the staging buffer (four accumulator elements per 8-byte access).
  const bool tposed = io.rs_a == 1;
  constexpr int NP = 2 * NNW;                    // 16-byte pieces per lane
  constexpr int NCOL = 32 * NNW;                 // tile columns
  struct TileRegs {
    u32x4 v[NP];
  };
  uint32_t tile_goff[NP];                        // byte offsets inside one state matrix (< 256 KiB)
  int tile_soff[NP];                             // element offsets inside one staging stage
  auto stage_elem = [&](int e) { return (32 * nb0 + e / 32) * RT_LD + 32 * ablk + e % 32; };
  // accumulator element (nn, r) in the staging area: one per-lane base plus constants
  const int dl_base = tposed ? (32 * nb0 + c) * RT_LD + 32 * ablk + 4 * g
                             : (32 * nb0 + NNW * 4 * g) * RT_LD + 32 * ablk + c;
  auto dl_plain = [&](int nn, int r) { return dl_base + (NNW * (8 * (r >> 2) + (r & 3)) + nn) * RT_LD; };
  auto dl_tposed = [&](int nn, int qd) { return dl_base + 32 * nn * RT_LD + 8 * qd; };
#pragma unroll
  for (int u = 0; u < NP; ++u) {
    const int q = lane + 64 * u;
    if (!tposed) {
      const int a_l = q / (4 * NNW), piece = q % (4 * NNW);
      tile_goff[u] = 2u * (uint32_t)((32 * ablk + a_l) * (int)io.rs_a + tile * BV + 32 * nb0 + 8 * piece);
      tile_soff[u] = stage_elem(a_l * NCOL + 8 * piece);
    } else {
      const int n_l = q / 4, piece = q % 4;
      tile_goff[u] = 2u * (uint32_t)((tile * BV + 32 * nb0 + n_l) * (int)io.rs_n + 32 * ablk + 8 * piece);
      tile_soff[u] = stage_elem(n_l * 32 + 8 * piece);
    }
  }
  // byte offset of half hf of the rows of R inside a state matrix
  const uint32_t half_stride = 2u * DA * (uint32_t)(tposed ? 1 : io.rs_a);
  // issue the global loads of a tile; `src` null or !live -> zeros without memory traffic
  auto tile_load = [&](TileRegs& tr, const uint16_t* src, bool live, int hf) {
    const fprt::BufView view = fprt::make_buf(src, (src && live) ? (uint32_t)(mat * 2) : 0u);
#pragma unroll
    for (int u = 0; u < NP; ++u) tr.v[u] = fprt::buf_load128(view, tile_goff[u] + hf * half_stride);
  };
  // R (+)= loaded tile, through stage s
  auto tile_accumulate = [&](const TileRegs& tr, int s, bool add, f32x16 (&racc)[NNW]) {
    uint16_t* st = RT + s * BV * RT_LD;
#pragma unroll
    for (int u = 0; u < NP; ++u) st128(st + tile_soff[u], tr.v[u]);
    fprt::wave_sync();
#pragma unroll
    for (int nn = 0; nn < NNW; ++nn) {
      if (!tposed) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float x = bf16_bits_to_float(reinterpret_cast<const u16_m*>(st)[dl_plain(nn, r)]);
          racc[nn][r] = add ? racc[nn][r] + x : x;
        }
      } else {
#pragma unroll
        for (int qd = 0; qd < 4; ++qd) {
          const u32x2 d = ld64(st + dl_tposed(nn, qd));
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            const uint32_t w = d[k >> 1];
            const float x = __builtin_bit_cast(float, (k & 1) ? (w & 0xffff0000u) : (w << 16));
            racc[nn][4 * qd + k] = add ? racc[nn][4 * qd + k] + x : x;
          }
        }
      }
    }
    fprt::wave_sync();   // the staging area is reused right after
  };
  // bf16(R) -> global matrix at dst, through stage s
  auto tile_store = [&](uint16_t* dst, int s, const f32x16 (&racc)[NNW], int hf) {
    uint16_t* st = RT + s * BV * RT_LD;
#pragma unroll
    for (int nn = 0; nn < NNW; ++nn) {
      if (!tposed) {
#pragma unroll
        for (int r = 0; r < 16; ++r)
          reinterpret_cast<u16_m*>(st)[dl_plain(nn, r)] = float_to_bf16_bits(racc[nn][r]);
      } else {
#pragma unroll
        for (int qd = 0; qd < 4; ++qd) {
          u32x2 d;
          d[0] = fprt::pack_bf16x2(racc[nn][4 * qd], racc[nn][4 * qd + 1]);
          d[1] = fprt::pack_bf16x2(racc[nn][4 * qd + 2], racc[nn][4 * qd + 3]);
          st64(st + dl_tposed(nn, qd), d);
        }
      }
    }
    fprt::wave_sync();
    const fprt::BufView view = fprt::make_buf(dst, (uint32_t)(mat * 2));
#pragma unroll
    for (int u = 0; u < NP; ++u) fprt::buf_store128(view, tile_goff[u] + hf * half_stride, ld128(st + tile_soff[u]));
    fprt::wave_sync();   // the staging area is reused right after
  };
  // block-state matrix of the block that ends at token t1 (its gradient in a reverse pass)
  auto block_matrix = [&](const uint16_t* base, int b, int t1) {
    const int m = bs > 0 ? t1 / bs - 1 : 0;   // bs is a compile-time 0 in the walks that never get here
    return base + (((size_t)b * p.nblk + m) * p.H + h) * mat;
  };
  auto state_matrix = [&](const uint16_t* base, int b) { return base + ((size_t)b * p.H + h) * mat; };
  auto ends_block = [&](int t1) { return bs > 0 && (t1 % bs) == 0; };

  // bf16 copy of R -> LDS stage s
  auto write_rt = [&](int s, const f32x16 (&racc)[NNW]) {
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
  };

  // A loaded W chunk goes to LDS: the weighted W^T slab is formed in registers and written at
  // once (short live ranges), the row-major W tile of stage s is a copy.
  int Lk_cached = -1;
  float wkey[4];
  auto store_transposed = [&](const ChunkRegs& cr, const Chunk& ck) {
    // walking forward, a suffix's keys never enter the state (only, on a copy, the state that its own later parts read)
    if (SFX && ck.sfx && !rev && ck.part == sfx_parts - 1) return;
    if (ck.L != Lk_cached) {
      Lk_cached = ck.L;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int j = 4 * w_tg + r;
        int e = rev ? (j + 1) : (ck.L - 1 - j);
        if (e < 0) e = 0;
        wkey[r] = io.s_update * fprt::exp2_approx((float)e * lg);
      }
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      u32x2 d;
      d[0] = fprt::pack_bf16x2(bf16_elem(cr.w[0], e) * wkey[0], bf16_elem(cr.w[1], e) * wkey[1]);
      d[1] = fprt::pack_bf16x2(bf16_elem(cr.w[2], e) * wkey[2], bf16_elem(cr.w[3], e) * wkey[3]);
      st64(wt + wt_off + e * T_LD, d);
    }
  };
  auto store_rowmajor = [&](const ChunkRegs& cr, int s) {
    uint16_t* ws = WS + s * CH * X_LD;
    if (ws_writer && !STATE) {
#pragma unroll
      for (int r = 0; r < 4; ++r) st128(ws + ws_off + r * X_LD, cr.w[r]);
    }
  };

  // Suffix walk, backward, with tokens after the last block boundary: R0 is the gradient of the
  // state at that boundary, not at the end of the sequence.  The walk starts from zero and R0 joins
  // when the boundary is reached, the way block-state gradients do.
  const bool r0_late = SFX_ANY && rev && io.R0 && T > p.nblk * bs;
  const bool r0_first = io.R0 && !r0_late;
  // ---- prologue: chunk 0 into stage 0, chunk 1 in flight ----------------------------------
  Chunk cur = first_chunk(slot), nxt = chunk_after(cur);
  prefetch(wregs, cur);
#pragma unroll
  for (int hf = 0; hf < NH; ++hf) {
    // initial R, plus the gradient of the last block state if the first chunk of a reverse pass ends a block
    TileRegs t_init, t_inj;
    tile_load(t_init, r0_first ? state_matrix(io.R0, cur.b) : nullptr, true, hf);
    const bool inj = BLOCKS && io.Bin && ends_block(cur.t0 + cur.L);
    tile_load(t_inj, inj ? block_matrix(io.Bin, cur.b, cur.t0 + cur.L) : nullptr, inj, hf);
    if (r0_first) tile_accumulate(t_init, 0, false, racc[hf]);
    if (inj) tile_accumulate(t_inj, 0, true, racc[hf]);
  }
  write_rt(0, racc[0]);
  store_transposed(wregs, cur);
  store_rowmajor(wregs, 0);
  prefetch(wregs, nxt);
  fprt::block_sync();

  int Lg_cached = -1;
  float gL = 1.f;
  // suffix walk: R while a suffix in several parts works on its copy (one visit per chunk only:
  // with two, a second set of both halves does not fit the register file)
  f32x16 saved[NNW];
  // One iteration: `wregs` holds the W rows of item it + 1 on entry and is reloaded with item
  // it + 2 once they have gone into LDS.  Returns false after the last item.  `half` is the parity
  // of `it` as a type; with NH = 2 it is the half of R this visit updates.
  auto iteration = [&](auto half, int it) -> bool {
    constexpr int HF = NH > 1 ? decltype(half)::value : 0;
    constexpr bool closes = HF == NH - 1;   // the chunk is complete after this visit
    f32x16 (&racc_h)[NNW] = racc[HF];
    const int s = it & 1;
    const Chunk nn = chunk_after(nxt);
    // gradient of the block state that the next chunk ends (reverse pass); an empty view otherwise
    // (suffix walk: the gradient of the state at the last boundary, when the next item is that boundary's suffix)
    const bool inj = closes && nxt.ok && (BLOCKS ? io.Bin && ends_block(nxt.t0 + nxt.L) : r0_late && nxt.sfx && nxt.n == p.nblk && nxt.part == sfx_parts - 1);
    TileRegs t_inj[NH];
    if ((BLOCKS || SFX_ANY) && closes) {
      const uint16_t* const src = !inj ? nullptr : BLOCKS ? block_matrix(io.Bin, nxt.b, nxt.t0 + nxt.L) : state_matrix(io.R0, nxt.b);
#pragma unroll
      for (int hf = 0; hf < NH; ++hf) tile_load(t_inj[hf], src, inj, hf);
    }
    // initial state of the next sequence, if the next chunk starts one
    const bool fresh = MULTI && nxt.ok && nxt.first;
    TileRegs t_init;
    if (MULTI) tile_load(t_init, (fresh && io.R0) ? state_matrix(io.R0, nxt.b) : nullptr, fresh, 0);

    // A suffix carries tokens only in its first k-steps, and none that enter the state when
    // walking forward: the other k-steps are skipped (uniform branches).
    // A suffix in several parts works on a copy of the state: R is put aside when the walk
    // enters the suffix and comes back when it leaves.  Forward, the copy advances through all
    // parts but the last; backward, it starts from zero and what it holds in the end (the
    // gradient of the state the suffix read) is added to R.
    const bool sfx_item = SFX && cur.sfx;
    const bool sfx_multi = SFX_ANY && NH == 1 && sfx_item && sfx_parts > 1;
    const bool enters = sfx_multi && cur.part == (rev ? sfx_parts - 1 : 0);
    const bool leaves_sfx = sfx_multi && cur.part == (rev ? 0 : sfx_parts - 1);
    const bool advances = !sfx_item || rev || cur.part < sfx_parts - 1;
    const bool decays = !sfx_item || (sfx_multi && (rev ? !enters : advances));
    const int nk = !sfx_item ? 4 : rev ? (cur.L + 15) >> 4 : advances ? 4 : 0;

    // ---- phase 0: request the operands of the state update (this wave's whole W^T slab, the
    // first half of Z^T); decay R while they arrive
    const int gkey = decays ? cur.L : 0;   // a suffix in one part does not advance the state
    if (gkey != Lg_cached) {
      Lg_cached = gkey;
      gL = fprt::exp2_approx((float)gkey * lg);
    }
    const uint16_t* zt = ZT + s * BV * T_LD;
    u32x4 wf[4], zlo[NNW][2], zhi[NNW][2];
#pragma unroll
    for (int kt = 0; kt < 4; ++kt) {
      if (kt < nk) wf[kt] = ld_token_frag(wt + c * T_LD + 16 * kt + 4 * g);
    }
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
      if (kt < nk) {
#pragma unroll
        for (int nq = 0; nq < NNW; ++nq) zlo[nq][kt] = ld_token_frag(zt + (32 * (nb0 + nq) + c) * T_LD + 16 * kt + 4 * g);
      }
    }
    if (SFX_ANY && enters) {
#pragma unroll
      for (int nq = 0; nq < NNW; ++nq) {
        saved[nq] = racc_h[nq];
        if (rev) racc_h[nq] = f32x16{0};
      }
    }
    if (decays) {
#pragma unroll
      for (int nq = 0; nq < NNW; ++nq) {
#pragma unroll
        for (int r = 0; r < 16; ++r) racc_h[nq][r] *= gL;
      }
    }
    fprt::sched_fence();

    // ---- phase 1: first half of R = gamma^L R + (wkey W)^T Z; in its shadow the rest of Z^T is
    // requested and the W of chunk it + 1 (zeros if there is none) is transposed.  The W^T slab is overwritten only after all of it was read.
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
      if (kt < nk) {
#pragma unroll
        for (int nq = 0; nq < NNW; ++nq) racc_h[nq] = fprt::mfma_32x32x16_bf16(wf[kt], zlo[nq][kt], racc_h[nq]);
      }
    }
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
      if (2 + kt < nk) {
#pragma unroll
        for (int nq = 0; nq < NNW; ++nq)
          zhi[nq][kt] = ld_token_frag(zt + (32 * (nb0 + nq) + c) * T_LD + 16 * (2 + kt) + 4 * g);
      }
    }
    store_transposed(wregs, nxt);
    fprt::sched_fence();
    if (!STATE && closes) fprt::block_sync();   // the readout waves hand their P tiles to each other here

    // ---- phase 2: second half of the state update; the row-major copies go out in its shadow
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
      if (2 + kt < nk) {
#pragma unroll
        for (int nq = 0; nq < NNW; ++nq) racc_h[nq] = fprt::mfma_32x32x16_bf16(wf[2 + kt], zhi[nq][kt], racc_h[nq]);
      }
    }
    store_rowmajor(wregs, s ^ 1);
    prefetch(wregs, nn);
    fprt::sched_fence();

    // ---- phase 3: the state after a full block or at the end of a sequence leaves, the gradient
    // of the next block state joins (reverse walk) or the next sequence's initial state takes
    // over, and the bf16 copy for the next chunk's read-out is written.  All of them use this
    // wave's part of the other stage's R buffer, in this order.
    const int t1 = cur.t0 + cur.L;
    if (SFX_ANY && leaves_sfx) {
#pragma unroll
      for (int nq = 0; nq < NNW; ++nq) {
#pragma unroll
        for (int r = 0; r < 16; ++r) racc_h[nq][r] = rev ? racc_h[nq][r] + saved[nq][r] : saved[nq][r];
      }
    }
    if (closes) {
#pragma unroll
      for (int hf = 0; hf < NH; ++hf) {
        if (BLOCKS && io.Bout && ends_block(t1))
          tile_store(const_cast<uint16_t*>(block_matrix(io.Bout, cur.b, t1)), s ^ 1, racc[hf], hf);
        // the state that leaves: after the last item; walking forward with suffixes, the one that the
        // suffix at the last block boundary reads (tokens after that boundary are not in it)
        const bool leaves = (SFX && !rev) ? cur.sfx && cur.n == p.nblk && cur.part == sfx_parts - 1 : cur.last;
        if (leaves && io.Rout) tile_store(const_cast<uint16_t*>(state_matrix(io.Rout, cur.b)), s ^ 1, racc[hf], hf);
      }
    }
    if (nxt.ok) {
      if (MULTI && fresh) {
        if (io.R0) {
          tile_accumulate(t_init, s ^ 1, false, racc[0]);
        } else {
#pragma unroll
          for (int nq = 0; nq < NNW; ++nq) racc[0][nq] = f32x16{0};
        }
      }
      if ((BLOCKS || SFX_ANY) && closes && inj) {
#pragma unroll
        for (int hf = 0; hf < NH; ++hf) tile_accumulate(t_inj[hf], s ^ 1, true, racc[hf]);
      }
      // the next visit reads the other half (NH = 2), which this visit did not touch
      if (!STATE) write_rt(s ^ 1, racc[(HF + 1) % NH]);
    }
    fprt::block_sync();
    if (!nxt.ok) return false;
    cur = nxt;
    nxt = nn;
    return true;
  };
  walk_visits<NH>([&](auto part, int it) { return iteration(part, it); });
}

}  // namespace fpk
