// Fused retention backward for dk, dv in {64, 128}: two workgroups per (batch, head) stream, each
// covering the full width of its tensors, in one launch.
//
//   "reverse" workgroup   walks the chunks from the last to the first and carries dS once.  It is
//                         the dk pass and the dv pass of pass_args.h side by side:
//                           pass 0 (dv):  X = k,  W = q,   Z = dO,  R = dS     (dk x dv)
//                           pass 1 (dk):  X = v,  W = dO,  Z = q,   R = dS^T   (dv x dk)
//                         W of one pass is Z of the other, so the state update
//                         dS <- gamma^L dS + sum_j gamma^(j+1) q_j^T dO_j is done once and q, k, v,
//                         dO are read once.
//   "forward" workgroup   the dq pass (X = dO, W = v, Z = k, R = S^T), walking forward and
//                         re-running the state recurrence from s0, or, with the states that the
//                         forward pass left every few chunks, from those checkpoints: segment by
//                         segment from the last to the first, close to the reverse workgroup of
//                         its stream, so that rows read twice are read close together in time.
//
// With POP suffixes a suffix is one more stop of either walk at its block boundary, with tensors of
// its own: it reads the state there and leaves it as it is (FB_STOPS).  Suffixes of at most 16 tokens
// are not stops (FB_FOLD): the two things that tie a suffix to the carried states become part of the
// chunk that starts at its boundary, and the rest is done by a second, small kernel (suffix_intra_bwd).
//
// Outputs are stored, and q (which only the reverse workgroup reads) is loaded, with the
// non-temporal hint: kept out of the caches they leave room for k, v and dO, which both workgroups
// of a stream read.
//
// Both kinds keep the four (three) 64 x d input tiles of a chunk row-major in LDS, single
// buffered; the next chunk waits in registers.  Operands that run along the features of a tile are
// 16-byte row reads, operands that run along its tokens come from the same tile through the
// transposing LDS read, so no transposed copy is ever written.  Rows are padded by 8 elements
// (a pitch of 136 or 72 elements: 4 banks more than a multiple of 32): 16 consecutive rows of a row
// read, and the 4 rows r, r + 4, r + 8, r + 12 that the lanes of a transposing read address, fall on
// different banks, and every address is a per-lane base plus a compile-time offset.  Transposing
// reads therefore take the tokens of a k-step in a strided order (below), which products with two
// such operands are free to do; score tiles are computed with their rows permuted to match.
//
// Per chunk (reverse workgroup; the forward one is the same without the second pass):
//   scores    three live 32 x 32 tiles per pass, one wave each, scaled by the decay, masked,
//             rounded to bf16 and put into LDS in operand layout
//   -- barrier --
//   outputs   wave (pass, rt) owns rows 32 rt .. of Y^T for both 32-token halves (a 64-wide output has
//             two such waves; the other two of the pass only make score tiles and update the state):
//             Y^T = wread (R^T X^T) + Z^T P^T, written to a staging tile
//   update    every wave owns one or two 32 x 32 tiles of dS: decay, += (wkey W)^T Z
//   -- barrier --
//   the bf16 copy of dS, the next chunk's tiles and the staged outputs move
//   -- barrier --
#pragma once
#include "pass_args.h"
#include "lds_access.h"

namespace fpk {

// geometry of a row-major LDS tile of 64 tokens x D features and of the workgroup's sweep over it
template <int D>
struct FbTile {
  static_assert(D == 64 || D == 128, "tiles of 64 or 128 features");
  static constexpr int LD = D + 8;                 // row pitch, elements
  static constexpr int ELEMS = CH * LD;
  static constexpr int PPR = D / 8;                // 16-byte pieces per row
  static constexpr int ROWS = FB_THREADS / PPR;    // rows that one sweep of the 512 threads covers
  static constexpr int NU = CH / ROWS;             // sweeps per tile = pieces per thread
};
constexpr int FB_LD = FbTile<FB_D>::LD;     // the 128-wide tile (what the state-only kernel of segment_contrib.h uses too)
constexpr int FB_TILE = FbTile<FB_D>::ELEMS;
constexpr int FB_XP = 32 * 32;              // elements of one score tile in operand layout
// How POP suffixes take part in the walks:
//   FB_PLAIN  none
//   FB_STOPS  a suffix is one more stop of either walk (Ls <= 64)
//   FB_FOLD   suffixes of at most 16 tokens: only what couples a suffix to the carried states is done here, as part of
//             the chunk that starts at its boundary (the reverse workgroup adds sum_j gamma^(j+1) q_s[j]^T dO_s[j] to
//             dS as one more k-step of that chunk's update, the forward workgroup reads the state out for dO_s beside
//             the chunk's own read-out and writes that part of dq_s); what stays inside a suffix (dk_s, dv_s and the
//             rest of dq_s) is the work of suffix_intra_bwd, which runs afterwards.  Both walks take one more, empty,
//             chunk at T for the suffix there.
//   FB_BLOCKS no suffixes, but gradients of the states at block boundaries (the POP operator's block states) join dS
//             on the way: the reverse workgroup adds d_blocks[m] when its walk crosses the boundary behind block m
enum FbMode { FB_PLAIN = 0, FB_STOPS = 1, FB_FOLD = 2, FB_BLOCKS = 3 };
constexpr int FB_SFX_ROWS = 16;                         // longest suffix of FB_FOLD
// LDS of a launch (the larger of its two kinds of workgroup), bytes.
//   reverse: q, dO, k, v tiles; bf16 copy of dS; staging tiles for dv and dk; six score tiles;
//            FB_FOLD: 16 rows each of q_s and dO_s
//   forward: dO, v, k tiles; bf16 copy of S; staging tile for dq; three score tiles;
//            FB_FOLD: 32 rows for dO_s and two staging tiles of 32 rows for dq_s
constexpr int fb_lds_bytes(int dk, int dv, int mode) {
  const int ldk = dk + 8, ldv = dv + 8;
  const int reverse = 2 * CH * (ldk + ldv) + dv * ldk + CH * (ldv + ldk) + 6 * FB_XP + (mode == FB_FOLD ? FB_SFX_ROWS * (ldk + ldv) : 0);
  const int forward = CH * (2 * ldv + ldk) + dk * ldv + CH * ldk + 3 * FB_XP + (mode == FB_FOLD ? 2 * FB_SFX_ROWS * (ldv + 2 * ldk) : 0);
  return 2 * (reverse > forward ? reverse : forward);
}

namespace fb {

// element offset of (row, col) in a tile of pitch LD
template <int LD>
FP_DEVICE int at(int row, int col) { return row * LD + col; }
FP_DEVICE int at(int row, int col) { return at<FB_LD>(row, col); }

// Operand that runs along the columns of a tile: columns 16 t + 8 g .. + 7 of the lane's row.
// `rowp` points at column 8 g of that row.
FP_DEVICE u32x4 frag_cols(const uint16_t* rowp, int t) { return ld128(rowp + 16 * t); }

// Operands that run along the rows (tokens) of a tile come from two transposing reads.  A lane
// serves column cbase + lane % 32 and supplies the address of 4 columns of one row per read; the
// rows that the four lanes 4 q + i of a group of 16 address become elements 0..3 of every lane
// of the group.  Which rows of k-step t (rows 16 t .. 16 t + 15) a lane of half-wave g gets:
//   TR_NAT  e < 4: 16 t + 2 g + 4 e,          e >= 4: 16 t + 2 g + 1 + 4 (e - 4)
//           for products whose other operand is read the same way (any order serves)
//   TR_ACC  e < 4: 16 t + g + 4 e,            e >= 4: 16 t + 2 + g + 4 (e - 4)
//           the order in which a converted score tile (rows permuted by score_row) holds its tokens
//   TR_SEQ  16 t + 8 g + e
//           the order of a column-wise operand (rows four apart are what keeps the other two off
//           the same banks; this one pays for consecutive rows)
enum TrOrder { TR_NAT, TR_ACC, TR_SEQ };
struct TrLane {
  int lo, hi;   // element offsets of the two reads from (row 16 t, column cbase)
};
template <int LD>
FP_DEVICE TrLane tr_lane(int lane, TrOrder order) {
  const int g = lane >> 5, q = (lane & 15) >> 2;
  const int col = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
  const int r_lo = order == TR_NAT ? 2 * g + 4 * q : order == TR_ACC ? g + 4 * q : 8 * g + q;
  const int r_hi = order == TR_NAT ? r_lo + 1 : order == TR_ACC ? r_lo + 2 : r_lo + 4;
  return TrLane{r_lo * LD + col, r_hi * LD + col};
}
FP_DEVICE TrLane tr_lane(int lane, TrOrder order) { return tr_lane<FB_LD>(lane, order); }
// token (within its k-step) of element e of a TR_NAT operand
FP_DEVICE int nat_token(int g, int e) { return 2 * g + 4 * (e & 3) + (e >> 2); }
// row of the score tile that accumulator row m stands for: within each group of 16, m = 8 h + 4 g + e
// holds token 4 e + 2 h + g, so that a TR_ACC operand meets the converted tile element for element
FP_DEVICE int score_row(int m) { return (m & 16) + 4 * (m & 3) + 2 * ((m >> 3) & 1) + ((m >> 2) & 1); }

template <int LD>
FP_DEVICE u32x4 frag_rows(const uint16_t* tile, const TrLane& tl, int t, int cbase) {
  const uint16_t* p = tile + 16 * t * LD + cbase;
  const u32x2 lo = fprt::lds_read_tr16_b64(p + tl.lo);
  const u32x2 hi = fprt::lds_read_tr16_b64(p + tl.hi);
  return u32x4{lo[0], lo[1], hi[0], hi[1]};
}
FP_DEVICE u32x4 frag_rows(const uint16_t* tile, const TrLane& tl, int t, int cbase) { return frag_rows<FB_LD>(tile, tl, t, cbase); }

// eight packed bf16 times eight weights
FP_DEVICE u32x4 weigh(u32x4 v, const float (&w)[8]) {
  u32x4 o;
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    const float lo = __builtin_bit_cast(float, v[d] << 16) * w[2 * d];
    const float hi = __builtin_bit_cast(float, v[d] & 0xffff0000u) * w[2 * d + 1];
    o[d] = fprt::pack_bf16x2(lo, hi);
  }
  return o;
}

// What a workgroup of either kind shares: coordinates and the walk.
struct Common {
  int tid, wave, lane, g, c;
  int b, h, H;
  int T, nch;
  float lg;
  // POP suffixes (SFX instantiations): block = tokens per block (a multiple of CH that divides T),
  // Ls <= CH tokens per suffix, nblk = T / block, spb = chunks per block
  int block, Ls, nblk, spb;
};

// One stop of a walk: a chunk of the sequence or, with POP suffixes, the suffix that hangs off a
// block boundary.  `row` is its first row among all rows of its tensors ([B * T] rows; suffixes:
// [B * (nblk + 1) * Ls] rows); L = 0 stands for "beyond the walk".
struct Item {
  uint32_t row;
  int L;
  bool sfx;
};
FP_DEVICE Item chunk_item(const Common& k, int ci) {
  if (ci < 0 || ci >= k.nch) return Item{0u, 0, false};
  const int t0 = ci * CH;
  return Item{(uint32_t)k.b * k.T + t0, k.T - t0 < CH ? k.T - t0 : CH, false};
}
FP_DEVICE Item suffix_item(const Common& k, int n) { return Item{((uint32_t)k.b * (k.nblk + 1) + n) * k.Ls, k.Ls, true}; }
// Walking backward with suffixes: the suffix at T, then per block (from the last) its chunks
// from the last to the first and the suffix at its lower boundary.
FP_DEVICE Item item_backward(const Common& k, int it) {
  if (k.block == 0) return chunk_item(k, k.nch - 1 - it);
  if (it <= 0) return it == 0 ? suffix_item(k, k.nblk) : Item{0u, 0, false};
  const int j = it - 1, blk = k.nblk - 1 - j / (k.spb + 1), r = j % (k.spb + 1);
  if (blk < 0) return Item{0u, 0, false};
  return r < k.spb ? chunk_item(k, (blk + 1) * k.spb - 1 - r) : suffix_item(k, blk);
}
// Walking forward with suffixes: per block the suffix at its lower boundary and its chunks, then the suffix at T.
FP_DEVICE Item item_forward(const Common& k, int it) {
  if (k.block == 0) return chunk_item(k, it);
  const int blk = it / (k.spb + 1), r = it % (k.spb + 1);
  if (it < 0 || blk > k.nblk || (blk == k.nblk && r > 0)) return Item{0u, 0, false};
  return r == 0 ? suffix_item(k, blk) : chunk_item(k, blk * k.spb + r - 1);
}
FP_DEVICE int item_count(const Common& k) { return k.block == 0 ? k.nch : 1 + k.nblk * (k.spb + 1); }

FP_DEVICE Common make_common(const FusedBwdArgs& p, int stream) {
  Common k;
  k.tid = fprt::thread_index();
  k.wave = k.tid >> 6;
  k.lane = k.tid & 63;
  k.g = k.lane >> 5;
  k.c = k.lane & 31;
  k.H = p.H;
  k.h = stream % p.H;
  k.b = stream / p.H;
  k.T = p.T;
  k.nch = (p.T + CH - 1) / CH;
  k.lg = p.log2g[k.h];
  k.block = p.block;
  k.Ls = p.Ls;
  k.nblk = p.block > 0 ? p.T / p.block : 0;
  k.spb = p.block / CH;
  return k;
}

// view of the rows of an item in one tensor of D features per head (`ctx` for chunks, `sfx` for
// suffixes) for this stream; rows past the item read as zero and are dropped on stores
template <int D>
FP_DEVICE fprt::BufView item_view(const Common& k, const void* ctx, const void* sfx, const Item& it) {
  const uint32_t rowp = (uint32_t)k.H * D * 2;   // bytes between consecutive tokens
  const char* ptr = static_cast<const char*>(it.sfx ? sfx : ctx) + (size_t)it.row * rowp + (size_t)k.h * D * 2;
  return fprt::make_buf(ptr, it.L > 0 ? (uint32_t)(it.L - 1) * rowp + D * 2 : 0u);
}

// registers <- the rows of an item in one tensor.  ONCE: the tensor is read by nobody else (non-temporal load)
template <int D, bool ONCE = false>
FP_DEVICE void load_tile(const Common& k, const void* ctx, const void* sfx, const Item& it, u32x4 (&pf)[FbTile<D>::NU]) {
  using G = FbTile<D>;
  const fprt::BufView v = item_view<D>(k, ctx, sfx, it);
  const uint32_t rowp = (uint32_t)k.H * D * 2;
  const int row0 = k.tid / G::PPR, piece = k.tid % G::PPR;
#pragma unroll
  for (int u = 0; u < G::NU; ++u) {
    const uint32_t off = (uint32_t)(row0 + G::ROWS * u) * rowp + piece * 16;
    pf[u] = ONCE ? fprt::buf_load128_nt(v, off) : fprt::buf_load128(v, off);
  }
}
template <int D>
FP_DEVICE void stage_tile(const Common& k, uint16_t* tile, const u32x4 (&pf)[FbTile<D>::NU]) {
  using G = FbTile<D>;
  const int row0 = k.tid / G::PPR, piece = k.tid % G::PPR;
#pragma unroll
  for (int u = 0; u < G::NU; ++u) st128(tile + at<G::LD>(row0 + G::ROWS * u, 8 * piece), pf[u]);
}
// staging tile ([token][feature]) -> rows of an item in `dst` (chunks) or `dst_sfx` (suffixes)
template <int D>
FP_DEVICE void drain_tile(const Common& k, const uint16_t* tile, void* dst, void* dst_sfx, const Item& it) {
  using G = FbTile<D>;
  const fprt::BufView v = item_view<D>(k, dst, dst_sfx, it);
  const uint32_t rowp = (uint32_t)k.H * D * 2;
  const int row0 = k.tid / G::PPR, piece = k.tid % G::PPR;
#pragma unroll
  for (int u = 0; u < G::NU; ++u) {
    const int row = row0 + G::ROWS * u;
    // non-temporal: the gradients are not read back here, and kept out of the caches they leave
    // room for the rows that the other workgroup of the stream is about to read a second time
    fprt::buf_store128_nt(v, (uint32_t)row * rowp + piece * 16, ld128(tile + at<G::LD>(row, 8 * piece)));
  }
}

// 32 x 32 accumulator (rows n = nbase + acc_row(r, g), column token i) -> staging tile [i][n]
template <int LD>
FP_DEVICE void put_output(uint16_t* tile, int i, int nbase, int g, const f32x16& acc) {
#pragma unroll
  for (int qd = 0; qd < 4; ++qd) {
    u32x2 d;
    d[0] = fprt::pack_bf16x2(acc[4 * qd], acc[4 * qd + 1]);
    d[1] = fprt::pack_bf16x2(acc[4 * qd + 2], acc[4 * qd + 3]);
    st64(tile + at<LD>(i, nbase + 8 * qd + 4 * g), d);
  }
}

// The bf16 copy of a state matrix R (rows a, columns n) lives in LDS as Rt[n][a].
// accumulator tile (rows a = abase + acc_row, column n) -> Rt
template <int LD>
FP_DEVICE void put_state(uint16_t* Rt, int n, int abase, int g, const f32x16& acc) { put_output<LD>(Rt, n, abase, g, acc); }
FP_DEVICE void put_state(uint16_t* Rt, int n, int abase, int g, const f32x16& acc) { put_output<FB_LD>(Rt, n, abase, g, acc); }
template <int LD>
FP_DEVICE f32x16 get_state(const uint16_t* Rt, int n, int abase, int g) {
  f32x16 acc;
#pragma unroll
  for (int qd = 0; qd < 4; ++qd) {
    const u32x2 d = ld64(Rt + at<LD>(n, abase + 8 * qd + 4 * g));
    acc[4 * qd] = __builtin_bit_cast(float, d[0] << 16);
    acc[4 * qd + 1] = __builtin_bit_cast(float, d[0] & 0xffff0000u);
    acc[4 * qd + 2] = __builtin_bit_cast(float, d[1] << 16);
    acc[4 * qd + 3] = __builtin_bit_cast(float, d[1] & 0xffff0000u);
  }
  return acc;
}
// Global state matrix S [DK][DV] (dv contiguous) <-> its LDS copy, by all threads of the workgroup.
//   BY_DK = true   the copy is indexed [dk][dv], pitch DV + 8 (forward workgroup: R^T = S)
//   BY_DK = false  the copy is indexed [dv][dk], pitch DK + 8 (reverse workgroup: R^T = dS^T)
template <int DK, int DV, bool BY_DK>
FP_DEVICE void load_state(const Common& k, uint16_t* Rt, const uint16_t* src) {
  constexpr int PPR = DV / 8, PER = DK * PPR / FB_THREADS;
  const fprt::BufView v = fprt::make_buf(src, src ? (uint32_t)(DK * DV * 2) : 0u);   // null: zeros
#pragma unroll
  for (int u = 0; u < PER; ++u) {
    const int pc = k.tid + FB_THREADS * u, major = pc / PPR, minor = (pc % PPR) * 8;
    const u32x4 d = fprt::buf_load128(v, (uint32_t)pc * 16);
    if (BY_DK) {
      st128(Rt + at<DV + 8>(major, minor), d);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e)
        reinterpret_cast<u16_m*>(Rt)[at<DK + 8>(minor + e, major)] = (uint16_t)((e & 1) ? d[e >> 1] >> 16 : d[e >> 1] & 0xffffu);
    }
  }
}
template <int DK, int DV, bool BY_DK>
FP_DEVICE void store_state(const Common& k, const uint16_t* Rt, uint16_t* dst) {
  constexpr int PPR = DV / 8, PER = DK * PPR / FB_THREADS;
  const fprt::BufView v = fprt::make_buf(dst, (uint32_t)(DK * DV * 2));
#pragma unroll
  for (int u = 0; u < PER; ++u) {
    const int pc = k.tid + FB_THREADS * u, major = pc / PPR, minor = (pc % PPR) * 8;
    u32x4 d;
    if (BY_DK) {
      d = ld128(Rt + at<DV + 8>(major, minor));
    } else {
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const uint32_t lo = reinterpret_cast<const u16_m*>(Rt)[at<DK + 8>(minor + 2 * w, major)];
        const uint32_t hi = reinterpret_cast<const u16_m*>(Rt)[at<DK + 8>(minor + 2 * w + 1, major)];
        d[w] = lo | (hi << 16);
      }
    }
    fprt::buf_store128(v, (uint32_t)pc * 16, d);
  }
}

// One 32 x 32 score tile D[m][i] = sum_a W[j(m)][a] X[i][a] with j(m) = 32 jb + score_row(m) and
// i = 32 ib + column: after the products, decay, mask, bf16, into `xp` in operand layout (two k-steps
// of 512 elements).  `mw`: decay weights of this lane's accumulator elements.  Element r stands for W
// token score_const(r) + g and X token c; on the diagonal it is live if the W token is not before
// (`reverse`) / not after the X token, and dead entries are cleared whatever the product was
// (so that inf or nan from a masked token cannot leak).
FP_DEVICE int score_const(int r) { return 16 * (r >> 3) + 4 * (r & 3) + 2 * ((r >> 2) & 1); }
FP_DEVICE void score_finish(const f32x16& sc, const float (&mw)[16], bool diagonal, bool reverse, int c, int g,
                            uint16_t* xp, int lane) {
  const int x = reverse ? c - g : g - c;   // live: score_const(r) >= x (reverse) / -score_const(r) >= x
  float v[16];
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const bool live = !diagonal || (reverse ? score_const(r) >= x : -score_const(r) >= x);
    v[r] = live ? sc[r] * mw[r] : 0.f;
  }
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    u32x4 pm;
#pragma unroll
    for (int e = 0; e < 4; ++e) pm[e] = fprt::pack_bf16x2(v[8 * t + 2 * e], v[8 * t + 2 * e + 1]);
    st128(xp + 512 * t + lane * 8, pm);
  }
}

// Decay weights of this lane's accumulator elements of a score tile: s_intra gamma^distance, the
// distance being |W token - X token| inside a diagonal tile (0 for dead entries) and 32 more in the
// tile off the diagonal.
FP_DEVICE void score_weights(float s_intra, float lg, bool diagonal, bool reverse, int c, int g, float (&mw)[16]) {
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int jl = score_const(r) + g;
    const int d = reverse ? jl - c : c - jl;
    mw[r] = s_intra * fprt::exp2_approx((float)(diagonal ? (d >= 0 ? d : 0) : 32 + d) * lg);
  }
}

}  // namespace fb

// ---------------------------------------------------------------------------------------------
// reverse workgroup: dk, dv, d_s0
// PASS: 0 for waves 0..3 (dv), 1 for waves 4..7 (dk); the two copies meet at the same barriers.
//
// Per chunk, three stretches separated by workgroup barriers:
//   1  what reads X (k or v): the score tile of this wave and the read-out of dS for its two output
//      tiles, in one loop over the k-steps that shares the X operands; P goes to LDS
//   2  Y^T += Z^T P^T and the outputs go to their staging tile; the state update; the k and v
//      tiles of the next chunk replace the ones nobody reads any more; the new copy of dS
//   3  the q and dO tiles of the next chunk
// The outputs leave for global memory at the start of the next chunk's first stretch.
//
// SFX: POP suffixes hang off the block boundaries (item_backward).  Nothing downstream of a suffix
// reaches back into it, so it reads no dS (no read-out), and what it adds to dS, the gradient of
// the state it read, is not decayed.
template <int DK, int DV, int PASS, int MODE>
FP_DEVICE void fused_bwd_reverse(const FusedBwdArgs& p, char* lds, int stream) {
  using namespace fb;
  using GK = FbTile<DK>;
  using GV = FbTile<DV>;
  constexpr int LDK = GK::LD, LDV = GV::LD;
  constexpr bool SFX = MODE == FB_STOPS, FOLD = MODE == FB_FOLD, BLOCKS = MODE == FB_BLOCKS;
  static_assert(CH * (LDK + LDV) >= DK * LDV, "a block state's gradient fits where the k and v tiles are");
  const Common k = make_common(p, stream);
  uint16_t* const Qs = reinterpret_cast<uint16_t*>(lds);   // q  [64][LDK]
  uint16_t* const Gs = Qs + GK::ELEMS;                     // dO [64][LDV]
  uint16_t* const Ks = Gs + GV::ELEMS;                     // k  [64][LDK]
  uint16_t* const Vs = Ks + GK::ELEMS;                     // v  [64][LDV]
  uint16_t* const Rt = Vs + GV::ELEMS;                     // bf16(dS) as Rt[n = dv][a = dk]
  uint16_t* const OUTV = Rt + DV * LDK;                    // staging: dv [64][LDV]
  uint16_t* const OUTK = OUTV + GV::ELEMS;                 //          dk [64][LDK]
  uint16_t* const XP = OUTK + GK::ELEMS;                   // score tiles [pass][tile][k-step][lane]
  uint16_t* const QS = XP + 6 * FB_XP;                     // FOLD: 16 rows of q_s, then 16 rows of dO_s
  uint16_t* const GS = QS + FB_SFX_ROWS * LDK;

  // this pass: X and W are DX wide (the contraction of scores and read-out), Z and Y are DZ wide
  constexpr int pass = PASS;
  constexpr int DX = pass ? DV : DK, DZ = pass ? DK : DV;
  constexpr int LDX = DX + 8, LDZ = DZ + 8;
  constexpr int KS = DX / 16;          // k-steps of the contraction
  constexpr int NCT = DZ / 32;         // waves of this pass that own output rows
  const int rt = k.wave & 3, g = k.g, c = k.c, lane = k.lane;
  const uint16_t* const Xs = pass ? Vs : Ks;
  const uint16_t* const Ws = pass ? Gs : Qs;
  const uint16_t* const Zs = pass ? Qs : Gs;
  uint16_t* const out = pass ? OUTK : OUTV;
  uint16_t* const xp_pass = XP + pass * 3 * FB_XP;
  const float lg = k.lg;
  const bool has_out = NCT >= 4 || rt < NCT;

  // score tile of this wave (rt < 3): (jb, ib) = (0,0), (1,0), (1,1); live entries have j >= i
  const bool scores = rt < 3;
  const int s_jb = rt == 0 ? 0 : 1, s_ib = rt == 2 ? 1 : 0;
  float mw[16];
  score_weights(p.scale, lg, s_jb == s_ib, true, c, g, mw);
  const uint16_t* const s_wrow = Ws + at<LDX>(32 * s_jb + score_row(c), 8 * g);

  const TrLane tr_acc = tr_lane<LDZ>(lane, TR_ACC), tr_seq = tr_lane<LDK>(lane, TR_SEQ);
  const TrLane tr_nat_k = tr_lane<LDK>(lane, TR_NAT), tr_nat_v = tr_lane<LDV>(lane, TR_NAT);
  // state tiles of this wave: rows a = 32 at_ .. of dk, columns n = 32 (nt0 + u) .. of dv, u < TPW
  constexpr int NRT = DK / 32, NCTS = DV / 32;
  constexpr int TPW = NRT * NCTS >= 8 ? NRT * NCTS / 8 : 1;
  const int at_ = k.wave % NRT, nt0 = (k.wave / NRT) * TPW;
  const bool owns = NRT * NCTS >= 8 || nt0 < NCTS;   // 64 x 64: four tiles, waves 0..3
  // weights of the state update: wkey(j) = gamma^(j + 1) for the tokens of k-step 0
  float wk0[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) wk0[e] = fprt::exp2_approx((float)(nat_token(g, e) + 1) * lg);
  const float g16 = fprt::exp2_approx(16.f * lg);
  // read-out weights of a full chunk and its decay
  const float wread_full0 = p.scale * fprt::exp2_approx((float)(CH - 1 - c) * lg);
  const float wread_full1 = p.scale * fprt::exp2_approx((float)(CH - 1 - 32 - c) * lg);
  const float gL_full = fprt::exp2_approx((float)CH * lg);

  // FOLD: the chunks from the one past the end (empty; it carries the suffix at T) down to the first
  auto item_of = [&](int it) { return FOLD ? chunk_item(k, k.nch - it) : item_backward(k, it); };
  const int nitems = FOLD ? k.nch + 1 : item_count(k);
  // FOLD: the suffix that hangs off the first token of the chunk visited it-th (L = 0: none), and this thread's
  // 16 bytes of its q_s (threads 0..255) or dO_s rows (threads 256..511)
  auto suffix_of = [&](int it) {
    const int t0 = (k.nch - it) * CH;
    return it >= 0 && it < nitems && t0 % k.block == 0 ? suffix_item(k, t0 / k.block) : Item{0u, 0, false};
  };
  const bool sfx_q = k.tid < 256;
  const int sfx_i = k.tid & 255;
  const int sfx_row = sfx_q ? sfx_i / GK::PPR : sfx_i / GV::PPR, sfx_piece = sfx_q ? sfx_i % GK::PPR : sfx_i % GV::PPR;
  auto load_suffix = [&](int it) {
    Item sx = suffix_of(it);
    if (sfx_row >= FB_SFX_ROWS) sx.L = 0;
    sx.sfx = true;
    if (sfx_q) return fprt::buf_load128(item_view<DK>(k, nullptr, p.q_sfx, sx), (uint32_t)sfx_row * ((uint32_t)k.H * DK * 2) + sfx_piece * 16);
    return fprt::buf_load128(item_view<DV>(k, nullptr, p.dO_sfx, sx), (uint32_t)sfx_row * ((uint32_t)k.H * DV * 2) + sfx_piece * 16);
  };
  auto stage_suffix = [&](u32x4 v) {
    if (sfx_row >= FB_SFX_ROWS) return;
    if (sfx_q) st128(QS + at<LDK>(sfx_row, 8 * sfx_piece), v);
    else st128(GS + at<LDV>(sfx_row, 8 * sfx_piece), v);
  };
  // BLOCKS: the gradient of the block state at token t0 > 0 (the state that the chunk before t0 leaves), or nullptr
  const int nblocks = BLOCKS ? k.T / p.blocks_every : 0;
  auto block_grad = [&](int t0) -> const uint16_t* {
    if (!BLOCKS || t0 <= 0 || t0 % p.blocks_every != 0 || t0 / p.blocks_every > nblocks) return nullptr;
    return p.d_blocks + (((size_t)k.b * nblocks + (t0 / p.blocks_every - 1)) * p.H + k.h) * DK * DV;
  };
  constexpr int BP = DK * (DV / 8) / FB_THREADS;   // 16-byte pieces of a state matrix per thread
  Item cur = item_of(0), nxt = item_of(1), prev = cur;
  u32x4 pf_q[GK::NU], pf_g[GV::NU], pf_k[GK::NU], pf_v[GV::NU], pf_s = {0, 0, 0, 0};
  load_tile<DK, true>(k, p.q, p.q_sfx, cur, pf_q);   // q: read by this workgroup only
  load_tile<DV>(k, p.dO, p.dO_sfx, cur, pf_g);
  load_tile<DK>(k, p.k, p.k_sfx, cur, pf_k);
  load_tile<DV>(k, p.v, p.v_sfx, cur, pf_v);
  if constexpr (FOLD) pf_s = load_suffix(0);
  // the gradient that the walk starts from: that of the final state, or (BLOCKS) of a block that ends with the sequence
  load_state<DK, DV, false>(k, Rt, BLOCKS ? block_grad(k.T) : p.ds_out ? p.ds_out + (size_t)stream * DK * DV : nullptr);
  stage_tile<DK>(k, Qs, pf_q);
  stage_tile<DV>(k, Gs, pf_g);
  stage_tile<DK>(k, Ks, pf_k);
  stage_tile<DV>(k, Vs, pf_v);
  if constexpr (FOLD) stage_suffix(pf_s);
  load_tile<DK, true>(k, p.q, p.q_sfx, nxt, pf_q);
  load_tile<DV>(k, p.dO, p.dO_sfx, nxt, pf_g);
  load_tile<DK>(k, p.k, p.k_sfx, nxt, pf_k);
  load_tile<DV>(k, p.v, p.v_sfx, nxt, pf_v);
  fprt::block_sync();
  f32x16 racc[TPW];
#pragma unroll
  for (int u = 0; u < TPW; ++u) racc[u] = owns ? get_state<LDK>(Rt, 32 * (nt0 + u) + c, 32 * at_, g) : f32x16{0};

  const uint16_t* const xrow0 = Xs + at<LDX>(c, 8 * g);
  const uint16_t* const xrow1 = Xs + at<LDX>(32 + c, 8 * g);
  const uint16_t* const rrow = Rt + at<LDK>(32 * rt + c, 8 * g);   // pass 0 (a row of Rt is a column of dS)

  for (int it = 0; it < nitems; ++it) {
    const int L = cur.L;
    const bool sfx = SFX && cur.sfx;
    const Item after = item_of(it + 2);
    if constexpr (MODE == FB_PLAIN) {   // the loads of it + 2 chunks are on their way or done
      if (p.pace && k.tid == 0) fprt::pace_store(p.pace + stream, p.pace_base + (uint32_t)(it + 2));
    }
    // ---- the previous item's outputs leave (nothing writes the staging tiles before the next barrier)
    if (it > 0) {
      drain_tile<DV>(k, OUTV, p.dv, p.dv_sfx, prev);
      drain_tile<DK>(k, OUTK, p.dk, p.dk_sfx, prev);
    }
    // ---- stretch 1: scores D[j][i] = W[j] . X[i] and read-out wread(i) sum_a R^T[n][a] X[i][a], the
    // operands of a k-step requested a few k-steps ahead
    f32x16 acc[2], sc = {0};
    acc[0] = f32x16{0};
    acc[1] = f32x16{0};
    {
      u32x4 wf[KS], x0[KS], x1[KS], ra[KS];
      auto request = [&](int t) {
        if (scores) wf[t] = frag_cols(s_wrow, t);
        x0[t] = frag_cols(xrow0, t);
        x1[t] = frag_cols(xrow1, t);
        // pass 0: R^T = dS^T[n][a] is a row of Rt; pass 1: R^T = dS[a][n] runs along the rows of Rt
        ra[t] = pass == 0 ? frag_cols(rrow, t) : frag_rows<LDK>(Rt, tr_seq, t, 32 * rt);
      };
      constexpr int AHEAD = 2;   // k-steps of operands in flight (a third one costs the 128-wide instantiations their last registers)
      if (sfx || !has_out) {   // no read-out: only the score tile
        if (scores) {
#pragma unroll
          for (int t = 0; t < KS; ++t) {
            wf[t] = frag_cols(s_wrow, t);
            x0[t] = frag_cols(s_ib ? xrow1 : xrow0, t);
          }
          fprt::sched_fence();
#pragma unroll
          for (int t = 0; t < KS; ++t) sc = fprt::mfma_32x32x16_bf16(wf[t], x0[t], sc);
          score_finish(sc, mw, s_jb == s_ib, true, c, g, xp_pass + rt * FB_XP, lane);
        }
      } else if (scores) {
#pragma unroll
        for (int t = 0; t < AHEAD; ++t) request(t);
        fprt::sched_fence();
#pragma unroll
        for (int t = 0; t < KS; ++t) {
          sc = fprt::mfma_32x32x16_bf16(wf[t], s_ib ? x1[t] : x0[t], sc);
          acc[0] = fprt::mfma_32x32x16_bf16(ra[t], x0[t], acc[0]);
          acc[1] = fprt::mfma_32x32x16_bf16(ra[t], x1[t], acc[1]);
          if (t + AHEAD < KS) request(t + AHEAD);
          fprt::sched_fence();
        }
        score_finish(sc, mw, s_jb == s_ib, true, c, g, xp_pass + rt * FB_XP, lane);
      } else {
#pragma unroll
        for (int t = 0; t < AHEAD; ++t) request(t);
        fprt::sched_fence();
#pragma unroll
        for (int t = 0; t < KS; ++t) {
          acc[0] = fprt::mfma_32x32x16_bf16(ra[t], x0[t], acc[0]);
          acc[1] = fprt::mfma_32x32x16_bf16(ra[t], x1[t], acc[1]);
          if (t + AHEAD < KS) request(t + AHEAD);
          fprt::sched_fence();
        }
      }
    }
    float wread0 = wread_full0, wread1 = wread_full1;
    if (L != CH) {   // the last chunk of the sequence, visited first
      const int e0 = L - 1 - c, e1 = L - 1 - 32 - c;
      wread0 = p.scale * fprt::exp2_approx((float)(e0 > 0 ? e0 : 0) * lg);
      wread1 = p.scale * fprt::exp2_approx((float)(e1 > 0 ? e1 : 0) * lg);
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      acc[0][r] *= wread0;
      acc[1][r] *= wread1;
    }
    fprt::block_sync();

    // FOLD: the next chunk's suffix rows travel during this stretch only (registers are scarce in the first one)
    if constexpr (FOLD) pf_s = load_suffix(it + 1);
    // BLOCKS: this chunk starts at a block boundary: the gradient of the state there travels during this stretch
    const uint16_t* const inject = BLOCKS && !cur.sfx && L > 0 ? block_grad((int)(cur.row - (uint32_t)k.b * k.T)) : nullptr;
    u32x4 pf_b[BP];
    // ---- stretch 2: Y^T[n][i] += sum_j Z^T[n][j] P^T[j][i]
    if (has_out) {
      u32x4 za[4], pq0[4], pq1[2];
#pragma unroll
      for (int tj = 0; tj < 4; ++tj) {
        za[tj] = frag_rows<LDZ>(Zs, tr_acc, tj, 32 * rt);
        pq0[tj] = ld128(xp_pass + (tj >> 1) * FB_XP + 512 * (tj & 1) + lane * 8);
        if (tj >= 2) pq1[tj - 2] = ld128(xp_pass + 2 * FB_XP + 512 * (tj & 1) + lane * 8);
      }
      fprt::sched_fence();
#pragma unroll
      for (int tj = 0; tj < 4; ++tj) {
        acc[0] = fprt::mfma_32x32x16_bf16(za[tj], pq0[tj], acc[0]);
        if (tj >= 2) acc[1] = fprt::mfma_32x32x16_bf16(za[tj], pq1[tj - 2], acc[1]);
      }
    }
    if constexpr (BLOCKS) {
      const fprt::BufView bv = fprt::make_buf(inject, inject ? (uint32_t)(DK * DV * 2) : 0u);
#pragma unroll
      for (int u = 0; u < BP; ++u) pf_b[u] = fprt::buf_load128(bv, (uint32_t)(k.tid + FB_THREADS * u) * 16);
    }
    // state update, dS[a][n] = gamma^L dS + sum_j gamma^(j+1) q[j][a] dO[j][n], operands two k-steps ahead
    {
      u32x4 ua[4], ub[4][TPW];
      auto request_u = [&](int t) {
        ua[t] = frag_rows<LDK>(Qs, tr_nat_k, t, 32 * at_);
#pragma unroll
        for (int u = 0; u < TPW; ++u) ub[t][u] = frag_rows<LDV>(Gs, tr_nat_v, t, 32 * (nt0 + u));
      };
      if (owns) {
        request_u(0);
        request_u(1);
      }
      fprt::sched_fence();
      if (has_out) {
        put_output<LDZ>(out, c, 32 * rt, g, acc[0]);
        put_output<LDZ>(out, 32 + c, 32 * rt, g, acc[1]);
      }
      const float gL = sfx ? 1.f : L == CH ? gL_full : fprt::exp2_approx((float)L * lg);
#pragma unroll
      for (int u = 0; u < TPW; ++u) {
#pragma unroll
        for (int r = 0; r < 16; ++r) racc[u][r] *= gL;
      }
      float wk[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) wk[e] = wk0[e];
      fprt::sched_fence();
      if (owns) {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const u32x4 wa = weigh(ua[t], wk);
#pragma unroll
          for (int u = 0; u < TPW; ++u) racc[u] = fprt::mfma_32x32x16_bf16(wa, ub[t][u], racc[u]);
          if (t + 2 < 4) request_u(t + 2);
          if (t < 3) {
#pragma unroll
            for (int e = 0; e < 8; ++e) wk[e] *= g16;
          }
          fprt::sched_fence();
        }
      }
    }
    if constexpr (FOLD) {
      // the suffix at this chunk's first token: what it adds to dS is not decayed (it reads the state as it is there)
      if (owns && suffix_of(it).L > 0) {
        const u32x4 ua = frag_rows<LDK>(QS, tr_nat_k, 0, 32 * at_);
        u32x4 ub[TPW];
#pragma unroll
        for (int u = 0; u < TPW; ++u) ub[u] = frag_rows<LDV>(GS, tr_nat_v, 0, 32 * (nt0 + u));
        fprt::sched_fence();
        const u32x4 wa = weigh(ua, wk0);
#pragma unroll
        for (int u = 0; u < TPW; ++u) racc[u] = fprt::mfma_32x32x16_bf16(wa, ub[u], racc[u]);
      }
    }
    // nobody reads this chunk's k and v tiles or the old copy of dS any more
    if (BLOCKS && inject) {
      // the block state's gradient takes the place of the k and v tiles, [dk][dv] as it is stored, and every wave
      // adds its tiles of it to dS; the next chunk's k and v tiles follow in the third stretch
      uint16_t* const Bt = Ks;
#pragma unroll
      for (int u = 0; u < BP; ++u) {
        const int pc = k.tid + FB_THREADS * u;
        st128(Bt + at<LDV>(pc / (DV / 8), 8 * (pc % (DV / 8))), pf_b[u]);
      }
      fprt::block_sync();
      if (owns) {
#pragma unroll
        for (int u = 0; u < TPW; ++u) {
#pragma unroll
          for (int r = 0; r < 16; ++r)
            racc[u][r] += bf16_bits_to_float(reinterpret_cast<const u16_m*>(Bt)[at<LDV>(32 * at_ + acc_row(r, g), 32 * (nt0 + u) + c)]);
        }
      }
    } else {
      stage_tile<DK>(k, Ks, pf_k);
      stage_tile<DV>(k, Vs, pf_v);
      load_tile<DK>(k, p.k, p.k_sfx, after, pf_k);
      load_tile<DV>(k, p.v, p.v_sfx, after, pf_v);
    }
    if (owns) {
#pragma unroll
      for (int u = 0; u < TPW; ++u) put_state<LDK>(Rt, 32 * (nt0 + u) + c, 32 * at_, g, racc[u]);
    }
    fprt::block_sync();

    // ---- stretch 3: every read of this chunk's q and dO tiles is done
    if (BLOCKS && inject) {
      stage_tile<DK>(k, Ks, pf_k);
      stage_tile<DV>(k, Vs, pf_v);
      load_tile<DK>(k, p.k, p.k_sfx, after, pf_k);
      load_tile<DV>(k, p.v, p.v_sfx, after, pf_v);
    }
    stage_tile<DK>(k, Qs, pf_q);
    stage_tile<DV>(k, Gs, pf_g);
    load_tile<DK, true>(k, p.q, p.q_sfx, after, pf_q);
    load_tile<DV>(k, p.dO, p.dO_sfx, after, pf_g);
    if constexpr (FOLD) stage_suffix(pf_s);
    fprt::block_sync();
    prev = cur;
    cur = nxt;
    nxt = after;
  }
  drain_tile<DV>(k, OUTV, p.dv, p.dv_sfx, prev);
  drain_tile<DK>(k, OUTK, p.dk, p.dk_sfx, prev);
  if (p.ds0) store_state<DK, DV, false>(k, Rt, p.ds0 + (size_t)stream * DK * DV);
}

// ---------------------------------------------------------------------------------------------
// forward workgroup: dq.  In pass notation X = dO, W = v, Z = k, R[a = dv][n = dk] = S^T.
// Waves 0..3 ("output") own rows 32 w .. of Y^T = dq^T for both 32-token halves (two of them when dk = 64);
// waves 4..7 ("state") make the score tiles and own the tiles of rows 32 (w - 4) .. of R (two of them
// when dv = 64).
// STATE: the copy that waves 4..7 run; the two copies meet at the same barriers.
// SFX: POP suffixes hang off the block boundaries (item_forward): a suffix reads R without
// advancing it (no checkpoints in this form).
template <int DK, int DV, bool STATE, int MODE>
FP_DEVICE void fused_bwd_forward(const FusedBwdArgs& p, char* lds, int stream) {
  using namespace fb;
  using GK = FbTile<DK>;
  using GV = FbTile<DV>;
  constexpr int LDK = GK::LD, LDV = GV::LD;
  constexpr bool SFX = MODE == FB_STOPS, FOLD = MODE == FB_FOLD;
  constexpr int KS = DV / 16;          // k-steps of the contraction of scores and read-out
  constexpr int NCT = DK / 32;         // output waves with rows of dq^T; column tiles of R per state wave
  constexpr int NRT = DV / 32;         // state waves with rows of R
  const Common k = make_common(p, stream);
  uint16_t* const Xs = reinterpret_cast<uint16_t*>(lds);   // X = dO [64][LDV]
  uint16_t* const Ws = Xs + GV::ELEMS;                     // W = v  [64][LDV]
  uint16_t* const Zs = Ws + GV::ELEMS;                     // Z = k  [64][LDK]
  uint16_t* const Rt = Zs + GK::ELEMS;                     // bf16(R) as Rt[n = dk][a = dv]
  uint16_t* const OUT = Rt + DK * LDV;                     // staging: dq [64][LDK]
  uint16_t* const XP = OUT + GK::ELEMS;                    // score tiles (0,0), (0,1), (1,1)
  uint16_t* const XS = XP + 3 * FB_XP;                     // FOLD: 32 rows for dO_s (the first Ls are not zero)
  uint16_t* const OUTS = XS + 2 * FB_SFX_ROWS * LDV;       // FOLD: two staging tiles of 32 rows of dq_s, used in turn
  constexpr int SFX_OUT = 2 * FB_SFX_ROWS * LDK;
  const int g = k.g, c = k.c, lane = k.lane;
  constexpr bool state_role = STATE;
  const int rt = k.wave & 3;
  const float lg = k.lg;
  const bool has_out = NCT >= 4 || rt < NCT, owns = NRT >= 4 || rt < NRT;

  // score tile of state wave rt < 3: (jb, ib) = (0,0), (0,1), (1,1); live entries have i >= j
  const int s_jb = rt == 2 ? 1 : 0, s_ib = rt == 0 ? 0 : 1;
  float mw[16];
  score_weights(p.scale, lg, s_jb == s_ib, false, c, g, mw);
  const uint16_t* const s_wrow = Ws + at<LDV>(32 * s_jb + score_row(c), 8 * g);
  const uint16_t* const s_xrow = Xs + at<LDV>(32 * s_ib + c, 8 * g);
  const TrLane tr_acc = tr_lane<LDK>(lane, TR_ACC), tr_nat_k = tr_lane<LDK>(lane, TR_NAT), tr_nat_v = tr_lane<LDV>(lane, TR_NAT);

  // The walk: without checkpoints the chunks in order; with them the segments from the last to the
  // first, the chunks of a segment in order.  seg_chunks = chunks per segment.
  const int seg_chunks = p.ckpt ? p.ckpt_every / CH : k.nch;
  const int nseg = (k.nch + seg_chunks - 1) / seg_chunks;
  auto chunk_of = [&](int it) {   // chunk visited in iteration `it`, -1 beyond the walk
    if (it < 0 || it >= k.nch) return -1;
    if (nseg == 1) return it;
    // the last segment may be shorter than the others
    const int tail = k.nch - (nseg - 1) * seg_chunks;
    if (it < tail) return (nseg - 1) * seg_chunks + it;
    const int j = it - tail;
    return (nseg - 2 - j / seg_chunks) * seg_chunks + j % seg_chunks;
  };
  // state matrix that a segment starts from: s0 for the first, else the checkpoint before it
  auto segment_state = [&](int seg) -> const uint16_t* {
    if (seg == 0) return p.s0 ? p.s0 + (size_t)stream * DK * DV : nullptr;
    const size_t nck = (size_t)(k.T / p.ckpt_every);
    return p.ckpt + (((size_t)k.b * nck + (seg - 1)) * p.H + k.h) * DK * DV;
  };
  // item visited in iteration `it`
  // FOLD: the chunks in order and one more, empty, at T for the suffix there
  auto item_of = [&](int it) { return SFX ? item_forward(k, it) : FOLD ? chunk_item(k, it) : chunk_item(k, chunk_of(it)); };
  const int nitems = SFX ? item_count(k) : FOLD ? k.nch + 1 : k.nch;
  // FOLD: the suffix that hangs off the first token of the chunk visited it-th (L = 0: none), this thread's 16 bytes
  // of its dO_s rows (32 rows, zero from row Ls on), and its rows of dq_s
  auto suffix_of = [&](int it) {
    return it >= 0 && it < nitems && (it * CH) % k.block == 0 ? suffix_item(k, it * CH / k.block) : Item{0u, 0, false};
  };
  const int sx_row = k.tid / GV::PPR, sx_piece = k.tid % GV::PPR;     // dO_s: 32 rows of DV / 8 pieces
  const int sq_row = k.tid / GK::PPR, sq_piece = k.tid % GK::PPR;     // dq_s: 32 rows of DK / 8 pieces
  auto load_suffix = [&](int it) {
    Item sx = suffix_of(it);
    if (sx_row >= 2 * FB_SFX_ROWS) sx.L = 0;
    sx.sfx = true;
    return fprt::buf_load128(item_view<DV>(k, nullptr, p.dO_sfx, sx), (uint32_t)sx_row * ((uint32_t)k.H * DV * 2) + sx_piece * 16);
  };
  auto stage_suffix = [&](u32x4 v) {
    if (sx_row < 2 * FB_SFX_ROWS) st128(XS + at<LDV>(sx_row, 8 * sx_piece), v);
  };
  auto drain_suffix = [&](int it) {
    const Item sx = suffix_of(it);
    if (sx.L == 0 || sq_row >= 2 * FB_SFX_ROWS) return;
    const uint16_t* const tile = OUTS + ((it * CH / k.block) & 1) * SFX_OUT;
    fprt::buf_store128_nt(item_view<DK>(k, nullptr, p.dq_sfx, sx), (uint32_t)sq_row * ((uint32_t)k.H * DK * 2) + sq_piece * 16,
                          ld128(tile + at<LDK>(sq_row, 8 * sq_piece)));
  };
  Item cur = item_of(0), nxt = item_of(1), prev = cur;
  u32x4 pf_x[GV::NU], pf_w[GV::NU], pf_z[GK::NU], pf_s = {0, 0, 0, 0};
  load_tile<DV>(k, p.dO, p.dO_sfx, cur, pf_x);
  load_tile<DV>(k, p.v, p.v_sfx, cur, pf_w);
  load_tile<DK>(k, p.k, p.k_sfx, cur, pf_z);
  if constexpr (FOLD) pf_s = load_suffix(0);
  // R[a][n] = S[n][a]: the copy is the state matrix as it is stored
  load_state<DK, DV, true>(k, Rt, segment_state(nseg - 1));
  stage_tile<DV>(k, Xs, pf_x);
  stage_tile<DV>(k, Ws, pf_w);
  stage_tile<DK>(k, Zs, pf_z);
  if constexpr (FOLD) stage_suffix(pf_s);
  load_tile<DV>(k, p.dO, p.dO_sfx, nxt, pf_x);
  load_tile<DV>(k, p.v, p.v_sfx, nxt, pf_w);
  load_tile<DK>(k, p.k, p.k_sfx, nxt, pf_z);
  fprt::block_sync();
  f32x16 racc[NCT];
  if constexpr (state_role) {
#pragma unroll
    for (int u = 0; u < NCT; ++u) racc[u] = owns ? get_state<LDV>(Rt, 32 * u + c, 32 * rt, g) : f32x16{0};
  }
  const uint16_t* const xrow0 = Xs + at<LDV>(c, 8 * g);
  const uint16_t* const xrow1 = Xs + at<LDV>(32 + c, 8 * g);
  const uint16_t* const rrow = Rt + at<LDV>(32 * rt + c, 8 * g);
  const float wread0 = fprt::exp2_approx((float)(c + 1) * lg), wread1 = fprt::exp2_approx((float)(32 + c + 1) * lg);
  const float g16 = fprt::exp2_approx(16.f * lg);
  const float gL_full = fprt::exp2_approx((float)CH * lg);
  float wk_full[8];   // wkey of the tokens of the last k-step of a full chunk
#pragma unroll
  for (int e = 0; e < 8; ++e) wk_full[e] = p.scale * fprt::exp2_approx((float)(CH - 1 - (48 + nat_token(g, e))) * lg);

  // Per chunk, three stretches separated by workgroup barriers, as in the reverse workgroup:
  //   1  what reads X (dO): the read-out of R (output waves), the score tiles (state waves)
  //   2  Y^T += Z^T P^T and the outputs (output waves); the state update and the new copy of R
  //      (state waves); the next chunk's X tile
  //   3  the next chunk's W and Z tiles
  int patience = 256;   // polls of the pacing word that this workgroup affords in all
  for (int it = 0; it < nitems; ++it) {
    const int next = SFX ? 0 : chunk_of(it + 1);
    const bool fresh = !SFX && next >= 0 && next != chunk_of(it) + 1;   // the next chunk starts another segment
    const bool sfx = SFX && cur.sfx;
    const int L = cur.L;
    const Item after = item_of(it + 2);
    if constexpr (MODE == FB_PLAIN) {
      // the loads that this iteration issues (behind its first barrier) open another segment: not before the reverse
      // workgroup has asked for that segment's last chunk
      const int c2 = chunk_of(it + 2);
      if (p.pace && nseg > 1 && c2 >= 0 && c2 % seg_chunks == 0 && k.tid == 0) {
        const int last = (c2 + seg_chunks < k.nch ? c2 + seg_chunks : k.nch) - 1;
        const uint32_t want = p.pace_base + (uint32_t)(k.nch - last);
        while (patience > 0 && (int32_t)(fprt::pace_load(p.pace + stream) - want) < 0) {
          fprt::nap();
          --patience;
        }
      }
    }
    if (it > 0) {   // nothing writes the staging tile before the next barrier
      drain_tile<DK>(k, OUT, p.dq, p.dq_sfx, prev);
      if constexpr (FOLD) drain_suffix(it - 1);
    }
    f32x16 acc[2];
    if constexpr (state_role) {
      if (rt < 3) {
        u32x4 wf[KS], xf[KS];
        f32x16 sc = {0};
        constexpr int AH = KS < 4 ? KS : 4;
#pragma unroll
        for (int t = 0; t < AH; ++t) {
          wf[t] = frag_cols(s_wrow, t);
          xf[t] = frag_cols(s_xrow, t);
        }
        fprt::sched_fence();
#pragma unroll
        for (int t = 0; t < KS; ++t) {
          sc = fprt::mfma_32x32x16_bf16(wf[t], xf[t], sc);
          if (t + AH < KS) {
            wf[t + AH] = frag_cols(s_wrow, t + AH);
            xf[t + AH] = frag_cols(s_xrow, t + AH);
          }
          fprt::sched_fence();
        }
        score_finish(sc, mw, s_jb == s_ib, false, c, g, XP + rt * FB_XP, lane);
      }
    } else if (has_out) {
      // Y^T[n][i] = gamma^(i+1) sum_a R^T[n][a] X[i][a]
      acc[0] = f32x16{0};
      acc[1] = f32x16{0};
      {
        u32x4 ra[KS], x0[KS], x1[KS];
        auto request = [&](int t) {
          ra[t] = frag_cols(rrow, t);
          x0[t] = frag_cols(xrow0, t);
          x1[t] = frag_cols(xrow1, t);
        };
        constexpr int AH = KS < 4 ? KS : 4;
#pragma unroll
        for (int t = 0; t < AH; ++t) request(t);
        fprt::sched_fence();
#pragma unroll
        for (int t = 0; t < KS; ++t) {
          acc[0] = fprt::mfma_32x32x16_bf16(ra[t], x0[t], acc[0]);
          acc[1] = fprt::mfma_32x32x16_bf16(ra[t], x1[t], acc[1]);
          if (t + AH < KS) request(t + AH);
          fprt::sched_fence();
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          acc[0][r] *= wread0;
          acc[1][r] *= wread1;
        }
      }
      if constexpr (FOLD) {
        // the suffix at this chunk's first token reads the same R: its rows of dq_s, as far as they come from the state
        const Item sx = suffix_of(it);
        if (sx.L > 0) {
          const uint16_t* const xsrow = XS + at<LDV>(c, 8 * g);
          f32x16 as = {0};
          u32x4 ra[KS], xs[KS];
#pragma unroll
          for (int t = 0; t < KS; ++t) {
            ra[t] = frag_cols(rrow, t);
            xs[t] = frag_cols(xsrow, t);
          }
          fprt::sched_fence();
#pragma unroll
          for (int t = 0; t < KS; ++t) as = fprt::mfma_32x32x16_bf16(ra[t], xs[t], as);
#pragma unroll
          for (int r = 0; r < 16; ++r) as[r] *= wread0;
          put_output<LDK>(OUTS + ((it * CH / k.block) & 1) * SFX_OUT, c, 32 * rt, g, as);
        }
      }
    }
    fprt::block_sync();

    // FOLD: the next chunk's suffix rows travel during the second stretch only (registers are scarce in the first)
    if constexpr (FOLD) pf_s = load_suffix(it + 1);
    if constexpr (!state_role) {
      // Y^T[n][i] += sum_j Z^T[n][j] P^T[j][i]; tokens j < 32 reach both halves (tiles (0,0), (0,1)),
      // the others only the second
      if (has_out) {
        u32x4 za[4], pq1[4], pq0[2];
#pragma unroll
        for (int tj = 0; tj < 4; ++tj) {
          za[tj] = frag_rows<LDK>(Zs, tr_acc, tj, 32 * rt);
          pq1[tj] = ld128(XP + (tj < 2 ? 1 : 2) * FB_XP + 512 * (tj & 1) + lane * 8);
          if (tj < 2) pq0[tj] = ld128(XP + 512 * (tj & 1) + lane * 8);
        }
        fprt::sched_fence();
#pragma unroll
        for (int tj = 0; tj < 4; ++tj) {
          acc[1] = fprt::mfma_32x32x16_bf16(za[tj], pq1[tj], acc[1]);
          if (tj < 2) acc[0] = fprt::mfma_32x32x16_bf16(za[tj], pq0[tj], acc[0]);
        }
        put_output<LDK>(OUT, c, 32 * rt, g, acc[0]);
        put_output<LDK>(OUT, 32 + c, 32 * rt, g, acc[1]);
      }
    } else if (!sfx && owns) {
      // R[a][n] = gamma^L R + sum_j s gamma^(L-1-j) W[j][a] Z[j][n]
      const float gL = L == CH ? gL_full : fprt::exp2_approx((float)L * lg);
#pragma unroll
      for (int u = 0; u < NCT; ++u) {
#pragma unroll
        for (int r = 0; r < 16; ++r) racc[u][r] *= gL;
      }
      // wkey(j) = s gamma^(L-1-j).  Full chunk: the last k-step's weights, times gamma^16 per
      // earlier k-step.  Short chunk (the last one of a sequence): exponents clamped at 0 one by
      // one (those rows are zero, the weight only has to stay finite).
      float w[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) w[e] = wk_full[e];
      u32x4 ua[4], ub[4][NCT];
      auto request_u = [&](int t) {
        ua[t] = frag_rows<LDV>(Ws, tr_nat_v, t, 32 * rt);
#pragma unroll
        for (int u = 0; u < NCT; ++u) ub[t][u] = frag_rows<LDK>(Zs, tr_nat_k, t, 32 * u);
      };
      request_u(3);
      request_u(2);
      fprt::sched_fence();
#pragma unroll
      for (int tt = 0; tt < 4; ++tt) {
        const int t = 3 - tt;
        if (L != CH) {
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const int x = L - 1 - (16 * t + nat_token(g, e));
            w[e] = p.scale * fprt::exp2_approx((float)(x > 0 ? x : 0) * lg);
          }
        }
        const u32x4 wa = weigh(ua[t], w);
#pragma unroll
        for (int u = 0; u < NCT; ++u) racc[u] = fprt::mfma_32x32x16_bf16(wa, ub[t][u], racc[u]);
        if (t >= 2) request_u(t - 2);
        if (tt < 3) {
#pragma unroll
          for (int e = 0; e < 8; ++e) w[e] *= g16;
        }
        fprt::sched_fence();
      }
      if (!fresh) {
#pragma unroll
        for (int u = 0; u < NCT; ++u) put_state<LDV>(Rt, 32 * u + c, 32 * rt, g, racc[u]);
      }
    }
    // nobody reads this chunk's X tile or the old copy of R any more
    stage_tile<DV>(k, Xs, pf_x);
    load_tile<DV>(k, p.dO, p.dO_sfx, after, pf_x);
    if (fresh) load_state<DK, DV, true>(k, Rt, segment_state(next / seg_chunks));   // the next segment's starting state
    fprt::block_sync();

    stage_tile<DV>(k, Ws, pf_w);
    stage_tile<DK>(k, Zs, pf_z);
    load_tile<DV>(k, p.v, p.v_sfx, after, pf_w);
    load_tile<DK>(k, p.k, p.k_sfx, after, pf_z);
    if constexpr (FOLD) stage_suffix(pf_s);   // read in the first stretch only
    if constexpr (state_role) {
      if (fresh && owns) {
#pragma unroll
        for (int u = 0; u < NCT; ++u) racc[u] = get_state<LDV>(Rt, 32 * u + c, 32 * rt, g);
      }
    }
    fprt::block_sync();
    prev = cur;
    cur = nxt;
    nxt = after;
  }
  drain_tile<DK>(k, OUT, p.dq, p.dq_sfx, prev);
  if constexpr (FOLD) drain_suffix(nitems - 1);
}

// launch index -> kind and stream: the reverse workgroups (the longer ones) come first
// MODE: how POP suffixes take part (FbMode; p.block > 0 unless FB_PLAIN)
template <int DK, int DV, int MODE>
FP_DEVICE void fused_bwd(const FusedBwdArgs& p, char* lds, int block) {
  const int streams = p.B * p.H;
  if (block < streams) {
    if (fprt::thread_index() < 256) fused_bwd_reverse<DK, DV, 0, MODE>(p, lds, block);
    else fused_bwd_reverse<DK, DV, 1, MODE>(p, lds, block);
  }
  else if (fprt::thread_index() < 256) fused_bwd_forward<DK, DV, false, MODE == FB_BLOCKS ? FB_PLAIN : MODE>(p, lds, block - streams);
  else fused_bwd_forward<DK, DV, true, MODE == FB_BLOCKS ? FB_PLAIN : MODE>(p, lds, block - streams);
}

// ---------------------------------------------------------------------------------------------
// FB_FOLD, second launch: what stays inside a POP suffix of at most 16 tokens.  With
// D[i][j] = scale gamma^(i - j) for j <= i, A = D . (q_s k_s^T) and dA = D . (dO_s v_s^T), both rounded to bf16:
//   dv_s = A^T dO_s,   dk_s = dA^T q_s,   dq_s += dA k_s   (dq_s holds the part that came from the carried state).
// One workgroup of 4 waves takes the (suffix, head) pairs m = block, block + grid, ...: three score tiles by one wave
// each, then every wave a 32-column slice of each of the three outputs (the dq_s slice starts from what the first launch
// wrote, so that the sum is rounded once); the next pair's rows are on their way in registers meanwhile.  The three
// products are the dv pass, the dk pass and the dq pass of the chunk kernels above on one 16-token tile, and are written
// with their pieces.
constexpr int SI_THREADS = 256;
// q, k, dk, dq (dk wide) and v, dO, dv (dv wide), 32 rows each; score tiles
constexpr int si_lds_bytes(int dk, int dv) { return 2 * (2 * FB_SFX_ROWS * (4 * (dk + 8) + 3 * (dv + 8)) + 3 * FB_XP); }

template <int DK, int DV>
FP_DEVICE void suffix_intra_bwd(const FusedBwdArgs& p, char* lds) {
  using namespace fb;
  constexpr int LDK = DK + 8, LDV = DV + 8;
  constexpr int TK = 2 * FB_SFX_ROWS * LDK, TV = 2 * FB_SFX_ROWS * LDV;   // tiles of 32 rows (a score tile wants 32)
  const int tid = fprt::thread_index(), wave = tid >> 6, lane = tid & 63, g = lane >> 5, c = lane & 31;
  uint16_t* const Qs = reinterpret_cast<uint16_t*>(lds);   // inputs: rows >= Ls are zero
  uint16_t* const Ks = Qs + TK;
  uint16_t* const Vs = Ks + TK;
  uint16_t* const Gs = Vs + TV;
  uint16_t* const ODV = Gs + TV;                           // outputs
  uint16_t* const ODK = ODV + TV;
  uint16_t* const ODQ = ODK + TK;
  uint16_t* const XP = ODQ + TK;
  const uint32_t rowk = (uint32_t)p.H * DK * 2, rowv = (uint32_t)p.H * DV * 2;
  const int pairs = p.B * (p.T / p.block + 1) * p.H;
  // this thread's 16-byte piece of the 16 rows of a tensor (a 64-wide tensor has pieces for half of the threads)
  const int rk = tid / (DK / 8), ck = tid % (DK / 8), rv = tid / (DV / 8), cv = tid % (DV / 8);
  const bool live_k = rk < FB_SFX_ROWS, live_v = rv < FB_SFX_ROWS;
  const TrLane tr_acc_k = tr_lane<LDK>(lane, TR_ACC), tr_acc_v = tr_lane<LDV>(lane, TR_ACC);
  // pass of the score tile this wave makes (waves 0..2): X, W and whether it is the backward-walking kind
  //   0 dv: X = k, W = q, reverse     1 dk: X = v, W = dO, reverse     2 dq: X = dO, W = v, forward
  const uint16_t* const s_xrow = wave == 0 ? Ks + at<LDK>(c, 8 * g) : wave == 1 ? Vs + at<LDV>(c, 8 * g) : Gs + at<LDV>(c, 8 * g);
  const uint16_t* const s_wrow = wave == 0   ? Qs + at<LDK>(score_row(c), 8 * g)
                                 : wave == 1 ? Gs + at<LDV>(score_row(c), 8 * g)
                                             : Vs + at<LDV>(score_row(c), 8 * g);

  auto view = [&](const void* base, int m, int rows, int D) {
    const char* ptr = static_cast<const char*>(base) + ((size_t)(m / p.H) * p.Ls * p.H + (size_t)(m % p.H)) * D * 2;
    return fprt::make_buf(ptr, rows > 0 ? (uint32_t)(rows - 1) * ((uint32_t)p.H * D * 2) + D * 2 : 0u);
  };
  // registers <- the rows of pair m: q, k, v, dO and the dq_s written so far
  struct Rows {
    u32x4 q, k, v, d, dq;
  };
  auto load = [&](int m, Rows& r) {
    const int rows = m < pairs ? p.Ls : 0, mm = m < pairs ? m : 0;
    const int nk = live_k ? rows : 0, nv = live_v ? rows : 0;
    const uint32_t offk = (uint32_t)rk * rowk + ck * 16, offv = (uint32_t)rv * rowv + cv * 16;
    r.q = fprt::buf_load128(view(p.q_sfx, mm, nk, DK), offk);
    r.k = fprt::buf_load128(view(p.k_sfx, mm, nk, DK), offk);
    r.dq = fprt::buf_load128(view(p.dq_sfx, mm, nk, DK), offk);
    r.v = fprt::buf_load128(view(p.v_sfx, mm, nv, DV), offv);
    r.d = fprt::buf_load128(view(p.dO_sfx, mm, nv, DV), offv);
  };

  // rows 16 .. 31 of every tile are never written below: they start, and stay, zero
  for (int i = tid * 8; i < 4 * TK + 3 * TV; i += SI_THREADS * 8) st128(Qs + i, u32x4{0, 0, 0, 0});
  Rows cur;
  load(fprt::block_index(), cur);
  fprt::block_sync();
  for (int m = fprt::block_index(); m < pairs; m += fprt::grid_size()) {
    const float lg = p.log2g[m % p.H];
    if (live_k) {
      st128(Qs + at<LDK>(rk, 8 * ck), cur.q);
      st128(Ks + at<LDK>(rk, 8 * ck), cur.k);
      // what the carried state gave to dq_s waits in the dq staging tile: the product below is added to it in fp32
      st128(ODQ + at<LDK>(rk, 8 * ck), cur.dq);
    }
    if (live_v) {
      st128(Vs + at<LDV>(rv, 8 * cv), cur.v);
      st128(Gs + at<LDV>(rv, 8 * cv), cur.d);
    }
    load(m + fprt::grid_size(), cur);
    fprt::block_sync();
    if (wave < 3) {
      float mw[16];
      score_weights(p.scale, lg, true, wave < 2, c, g, mw);
      f32x16 sc = {0};
      if (wave == 0) {
        u32x4 wf[DK / 16], xf[DK / 16];
#pragma unroll
        for (int t = 0; t < DK / 16; ++t) {
          wf[t] = frag_cols(s_wrow, t);
          xf[t] = frag_cols(s_xrow, t);
        }
        fprt::sched_fence();
#pragma unroll
        for (int t = 0; t < DK / 16; ++t) sc = fprt::mfma_32x32x16_bf16(wf[t], xf[t], sc);
      } else {
        u32x4 wf[DV / 16], xf[DV / 16];
#pragma unroll
        for (int t = 0; t < DV / 16; ++t) {
          wf[t] = frag_cols(s_wrow, t);
          xf[t] = frag_cols(s_xrow, t);
        }
        fprt::sched_fence();
#pragma unroll
        for (int t = 0; t < DV / 16; ++t) sc = fprt::mfma_32x32x16_bf16(wf[t], xf[t], sc);
      }
      score_finish(sc, mw, true, wave < 2, c, g, XP + wave * FB_XP, lane);
    }
    fprt::block_sync();
    // Y^T[n][i] = sum_j Z^T[n][j] P^T[j][i] for this wave's 32 columns n of each output: Z = dO (dv_s), q (dk_s), k (dq_s)
    if (32 * wave < DV) {
      const u32x4 za = frag_rows<LDV>(Gs, tr_acc_v, 0, 32 * wave), pq = ld128(XP + lane * 8);
      f32x16 acc = {0};
      acc = fprt::mfma_32x32x16_bf16(za, pq, acc);
      put_output<LDV>(ODV, c, 32 * wave, g, acc);
    }
    if (32 * wave < DK) {
      const u32x4 zq = frag_rows<LDK>(Qs, tr_acc_k, 0, 32 * wave), pk = ld128(XP + FB_XP + lane * 8);
      f32x16 acc = {0};
      acc = fprt::mfma_32x32x16_bf16(zq, pk, acc);
      put_output<LDK>(ODK, c, 32 * wave, g, acc);
      const u32x4 zk = frag_rows<LDK>(Ks, tr_acc_k, 0, 32 * wave), pd = ld128(XP + 2 * FB_XP + lane * 8);
      acc = get_state<LDK>(ODQ, c, 32 * wave, g);   // the layout put_output writes: [token][feature]
      acc = fprt::mfma_32x32x16_bf16(zk, pd, acc);
      put_output<LDK>(ODQ, c, 32 * wave, g, acc);
    }
    fprt::block_sync();
    // rows < Ls leave
    if (live_v) fprt::buf_store128_nt(view(p.dv_sfx, m, p.Ls, DV), (uint32_t)rv * rowv + cv * 16, ld128(ODV + at<LDV>(rv, 8 * cv)));
    if (live_k) {
      const uint32_t off = (uint32_t)rk * rowk + ck * 16;
      fprt::buf_store128_nt(view(p.dk_sfx, m, p.Ls, DK), off, ld128(ODK + at<LDK>(rk, 8 * ck)));
      fprt::buf_store128_nt(view(p.dq_sfx, m, p.Ls, DK), off, ld128(ODQ + at<LDK>(rk, 8 * ck)));
    }
    // (the next pair's rows are staged by the thread that has just read this pair's results from the same places,
    // and every read of the input tiles is behind the barrier above)
  }
}

// The shapes the kernels above are instantiated for.
inline bool fused_bwd_dims(int dk, int dv) { return (dk == 64 || dk == 128) && (dv == 64 || dv == 128); }
// Pacing can only work when both workgroups of every stream are on the device at once (one workgroup per compute
// unit), sit behind the same L2 (launch indices s and streams + s on the same XCD: streams a multiple of 8) and
// there are checkpoints to cut the dq walk into segments.  `force`: whatever the device (the CPU harness).
inline bool fused_bwd_paces(const FusedBwdArgs& a, int compute_units, bool force = false) {
  if (!a.want_pace || !a.ckpt || a.ckpt_every <= 0 || a.block > 0 || a.d_blocks) return false;
  const long long streams = (long long)a.B * a.H;
  if (streams > PACE_SLOTS || (a.T + CH - 1) / CH >= 0xffff) return false;
  return force || (2 * streams <= compute_units && streams % 8 == 0);
}


// What the kernel assumes about its arguments; nullptr or a message for the caller.
inline const char* check_fused_bwd(const FusedBwdArgs& a) {
  if (a.B < 1 || a.T < 1 || a.H < 1 || a.H > MAX_HEADS || (long long)a.B * a.H * 2 > 0x7fffffffLL || !a.q || !a.k || !a.v ||
      !a.dO || !a.dq || !a.dk || !a.dv)
    return "fused backward: bad arguments";
  if (!fused_bwd_dims(a.dk_dim, a.dv_dim)) return "fused backward: dk and dv of 64 or 128";
  if (a.ckpt && (a.ckpt_every <= 0 || a.ckpt_every % CH != 0 || a.block > 0 || a.d_blocks))
    return "fused backward: checkpoints every positive multiple of 64 tokens, and not together with suffixes or block states";
  if (a.d_blocks && (a.blocks_every <= 0 || a.blocks_every % CH != 0 || a.block > 0 || a.ds_out))
    return "fused backward with block-state gradients: blocks of a positive multiple of 64 tokens, no suffixes, no final-state gradient";
  if (a.block > 0) {
    if (a.block % CH != 0 || a.T % a.block != 0 || a.Ls < 1 || a.Ls > CH)
      return "fused backward with suffixes: block a multiple of 64 that divides T, 1 <= Ls <= 64";
    if (a.fold && a.Ls > FB_SFX_ROWS) return "fused backward with folded suffixes: Ls <= 16";
    if (!a.q_sfx || !a.k_sfx || !a.v_sfx || !a.dO_sfx || !a.dq_sfx || !a.dk_sfx || !a.dv_sfx)
      return "fused backward with suffixes: all seven suffix tensors are needed";
    if ((long long)a.B * (a.T / a.block + 1) * a.Ls >= (1LL << 32)) return "fused backward with suffixes: too many suffix rows";
  }
  return nullptr;
}

}  // namespace fpk
