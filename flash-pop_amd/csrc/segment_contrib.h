// State-only pass for states of 128 rows: what a sequence of whole chunks adds to the carried
// state when nothing else is wanted of the pass (the first step of the split-sequence path),
//   U[a][n] = sum over the tokens j of  weight(j) W[j][a] Z[j][n],
// chunk by chunk as R <- gamma^64 R + (wkey W)^T Z from R = 0, with wkey(j) = s_update gamma^(63 - j)
// walking forward and s_update gamma^(j + 1) walking backward, the weighted W rounded to bf16 as the
// pass kernel rounds it.
//
// One workgroup per (sequence, head, 128 columns of Z) holds its whole 128 x 128 tile of R in the
// accumulators of its 8 waves (two 32 x 32 tiles each), so W is read once per 128 columns, Z once,
// and nothing else moves.  The W and Z tiles of a chunk sit row-major in LDS (two stages) and both
// MFMA operands come from them through the transposing LDS read (the tile layout and the operand
// helpers are those of retention_bwd_fused.h); two more chunks are on their way in registers.  One
// workgroup barrier per chunk.
#pragma once
#include "pass_args.h"
#include "lds_access.h"
#include "retention_bwd_fused.h"

namespace fpk {

// two stages of a W and a Z tile; the bf16 copy of R that the final store reads takes their place
constexpr int sc_lds_bytes() { return 2 * (4 * FB_TILE); }
static_assert(4 * FB_TILE >= FB_D * FB_LD, "the state copy fits where the tiles were");

template <bool REV>
FP_DEVICE void segment_contrib(const ContribArgs& p, char* lds) {
  using namespace fb;
  const int tid = fprt::thread_index(), wave = tid >> 6, lane = tid & 63, g = lane >> 5, c = lane & 31;
  // the workgroups of one (sequence, head) differ by a multiple of the stream count: with a multiple
  // of 8 streams they sit on the same XCD and share the W rows in its L2
  const int streams = p.B * p.H;
  const int ct = fprt::block_index() / streams, stream = fprt::block_index() % streams;
  const int h = stream % p.H, b = stream / p.H;
  const int nch = p.T / CH;
  const float lg = p.log2g[h];
  const uint32_t roww = (uint32_t)p.H * FB_D * 2, rowz = (uint32_t)p.H * p.dB * 2;   // bytes between tokens
  const char* const wbase = reinterpret_cast<const char*>(p.W) + ((size_t)b * p.T * p.H + h) * FB_D * 2;
  const char* const zbase = reinterpret_cast<const char*>(p.Z) + ((size_t)b * p.T * p.H + h) * p.dB * 2 + (size_t)ct * FB_D * 2;
  const fprt::BufView wv = fprt::make_buf(wbase, (uint32_t)(p.T - 1) * roww + FB_D * 2);
  const fprt::BufView zv = fprt::make_buf(zbase, (uint32_t)(p.T - 1) * rowz + FB_D * 2);
  const fprt::BufView none = fprt::make_buf(wbase, 0u);   // visits beyond the walk read zeros and move nothing

  uint16_t* const TL = reinterpret_cast<uint16_t*>(lds);   // stage s: W tile at 2 s, Z tile at 2 s + 1
  const int ld_row = tid >> 4, ld_piece = tid & 15;        // this thread's 16-byte pieces: rows ld_row, ld_row + 32

  // registers <- the chunk visited it-th
  auto load = [&](int it, u32x4 (&pf)[4]) {
    const bool live = it < nch;
    const uint32_t t0 = (uint32_t)(REV ? nch - 1 - it : it) * CH;
    const fprt::BufView w = live ? wv : none, z = live ? zv : none;
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const uint32_t row = live ? t0 + ld_row + 32 * u : 0u;
      pf[u] = fprt::buf_load128(w, row * roww + ld_piece * 16);
      pf[2 + u] = fprt::buf_load128(z, row * rowz + ld_piece * 16);
    }
  };
  auto stage = [&](int s, const u32x4 (&pf)[4]) {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      st128(TL + (2 * s) * FB_TILE + at(ld_row + 32 * u, 8 * ld_piece), pf[u]);
      st128(TL + (2 * s + 1) * FB_TILE + at(ld_row + 32 * u, 8 * ld_piece), pf[2 + u]);
    }
  };

  // this wave's tiles of R: rows a = 32 at_ .., columns n = 32 (nt0 + {0, 1}) ..
  const int at_ = wave & 3, nt0 = 2 * (wave >> 2);
  const TrLane tr_nat = tr_lane(lane, TR_NAT);
  // weights of the k-step taken first (the last 16 tokens walking forward, the first 16 walking
  // backward); each further k-step is 16 tokens further from where the state is read
  float wk_first[8];
#pragma unroll
  for (int e = 0; e < 8; ++e)
    wk_first[e] = p.s_update * fprt::exp2_approx((float)(REV ? nat_token(g, e) + 1 : 15 - nat_token(g, e)) * lg);
  const float g16 = fprt::exp2_approx(16.f * lg), gL = fprt::exp2_approx((float)CH * lg);

  f32x16 racc[2];
  racc[0] = f32x16{0};
  racc[1] = f32x16{0};

  auto update = [&](int s) {
    const uint16_t* const Ws = TL + (2 * s) * FB_TILE;
    const uint16_t* const Zs = Ws + FB_TILE;
    u32x4 ua[4], ub0[4], ub1[4];
    auto request = [&](int tt) {
      const int t = REV ? tt : 3 - tt;
      ua[tt] = frag_rows(Ws, tr_nat, t, 32 * at_);
      ub0[tt] = frag_rows(Zs, tr_nat, t, 32 * nt0);
      ub1[tt] = frag_rows(Zs, tr_nat, t, 32 * (nt0 + 1));
    };
    request(0);
    request(1);
    fprt::sched_fence();
#pragma unroll
    for (int u = 0; u < 2; ++u) {
#pragma unroll
      for (int r = 0; r < 16; ++r) racc[u][r] *= gL;
    }
    float wk[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) wk[e] = wk_first[e];
    fprt::sched_fence();
#pragma unroll
    for (int tt = 0; tt < 4; ++tt) {
      const u32x4 wa = weigh(ua[tt], wk);
      racc[0] = fprt::mfma_32x32x16_bf16(wa, ub0[tt], racc[0]);
      racc[1] = fprt::mfma_32x32x16_bf16(wa, ub1[tt], racc[1]);
      if (tt + 2 < 4) request(tt + 2);
      if (tt < 3) {
#pragma unroll
        for (int e = 0; e < 8; ++e) wk[e] *= g16;
      }
      fprt::sched_fence();
    }
  };

  // Chunk it is multiplied from stage it & 1 while chunk it + 1 moves from registers into the
  // other stage and the loads of chunk it + 3 take its place; chunk it + 2 is on its way in the
  // second set of registers.
  u32x4 pa[4], pb[4];
  load(0, pa);
  load(1, pb);
  stage(0, pa);
  load(2, pa);
  fprt::block_sync();
  for (int it = 0; it < nch; it += 2) {
    stage(1, pb);
    load(it + 3, pb);
    update(0);
    fprt::block_sync();
    if (it + 1 >= nch) break;
    stage(0, pa);
    load(it + 4, pa);
    update(1);
    fprt::block_sync();
  }

  // R -> bf16 -> its 128 columns of the rows of U[b][h] (element (a, n) at a * dB + n)
  uint16_t* const Rt = TL;   // every read of the tiles is behind the last barrier
#pragma unroll
  for (int u = 0; u < 2; ++u) put_state(Rt, 32 * (nt0 + u) + c, 32 * at_, g, racc[u]);
  fprt::block_sync();
  char* const ubase = reinterpret_cast<char*>(p.U) + ((size_t)stream * FB_D * p.dB + (size_t)ct * FB_D) * 2;
  const fprt::BufView uv = fprt::make_buf(ubase, (uint32_t)(FB_D - 1) * p.dB * 2 + FB_D * 2);
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int pc = tid + FB_THREADS * u, a = pc >> 4, n8 = (pc & 15) * 8;
    u32x4 d;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const uint32_t lo = reinterpret_cast<const u16_m*>(Rt)[at(n8 + 2 * w, a)];
      const uint32_t hi = reinterpret_cast<const u16_m*>(Rt)[at(n8 + 2 * w + 1, a)];
      d[w] = lo | (hi << 16);
    }
    fprt::buf_store128(uv, (uint32_t)a * p.dB * 2 + n8 * 2, d);
  }
}

// Host side: argument check, shared by the GPU launcher and the CPU test harness.
inline const char* check_contrib(const ContribArgs& a) {
  if (a.B < 1 || a.T < CH || a.T % CH != 0 || a.H < 1 || a.H > MAX_HEADS) return "state-only pass: whole chunks, B, H >= 1 expected";
  if (a.dB < FB_D || a.dB % FB_D != 0) return "state-only pass: Z must have a multiple of 128 columns";
  if (!a.W || !a.Z || !a.U) return "state-only pass: null pointer";
  if ((long long)a.B * a.H * (a.dB / FB_D) > 0x7fffffffLL) return "state-only pass: too many sequences";
  return nullptr;
}

}  // namespace fpk
