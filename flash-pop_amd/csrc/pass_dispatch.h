// Validation of one pass launch and the choice of kernel instantiation, shared by the device
// launcher and the CPU thread harness so that both take the same decisions.
#pragma once
#include <cstring>

#include "pass_args.h"
#include "retention_pass_ws.h"

namespace fpk {

// Number of kernel instantiations `dispatch_pass` can pick from (its `slot` argument is below this).
constexpr int PASS_KERNELS = 22;

// Checks what the walks assume about `a` and chooses a.slots (workgroups per (head, column tile))
// for a device with `compute_units` units.  Returns nullptr, or a message for the caller.
inline const char* plan_pass(PassArgs& a, int compute_units) {
  const bool blocks = a.block > 0 && (a.Bout || a.Bin);
  const bool narrow = a.dA == 64 || a.dA == 128;   // one visit per chunk
  const bool suffix = a.Ls > 0;
  if (a.dA != 64 && a.dA != 128 && a.dA != 192 && a.dA != 256) return "unsupported contraction width (dA must be 64, 128, 192 or 256)";
  if (a.dB < BV || a.dB % BV != 0) return "dB must be a multiple of 64";
  if (suffix) {
    // the C-ABI layer reports these to the caller in its own words
    if (blocks || a.block <= 0 || a.nblk != a.T / a.block || !a.Xs || !a.Ws || !a.Zs || !a.Ys)
      return "suffix walk: needs nblk == T / block and all four suffix tensors";
    if (a.Ls > CH && !narrow) return "suffixes longer than 64 tokens need dk and dv of 64 or 128";
    a.slots = a.B;
  }
  // One workgroup per (batch entry, head, column tile) while that fits the chip once; beyond that
  // the plain walk lets each workgroup take several batch entries one after another, which keeps
  // its load pipeline full across short sequences.
  if (a.slots <= 0) {
    a.slots = a.B;
    if (narrow && !blocks && !suffix) {
      int fit = compute_units / (a.H * (a.dB / BV));
      if (fit < 1) fit = 1;
      if (fit < a.B) a.slots = fit;
    }
  }
  if (a.slots > a.B) a.slots = a.B;
  if (a.state_only && (blocks || suffix || !a.Rout))
    return "state-only walk: needs a final-state buffer, no block states and no suffixes";
  // (with two visits per chunk only the first half of the state is handed over between sequences)
  if (a.slots < a.B && (!narrow || blocks || suffix))
    return "several batch entries per workgroup: only for the plain and state-only walks with dA of 64 or 128";
  return nullptr;
}

// Consecutive workgroup numbers go to the 8 XCDs in turn, and each XCD has an L2 of its own.  The
// workgroups that read the same rows should meet in one L2: the column tiles of a stream and, in a
// launch that holds several passes over the same tensors, the passes of a stream.  Launch index
// `block` of `passes * nwg` -> which pass (0 .. passes - 1) and which of its nwg workgroups.
struct WorkgroupId {
  int pass, wg;
};
FP_DEVICE WorkgroupId place_workgroup(int block, int nwg, int passes) {
  // XCD x runs the launch indices x, x + 8, ...; give it a contiguous range of the passes * nwg
  // logical numbers (one more for the first `rem` XCDs when 8 does not divide the total), in
  // which the passes of a workgroup and then the column tiles of a stream are neighbours.
  const int total = nwg * passes, per = total >> 3, rem = total & 7;
  const int xcd = block & 7, j = block >> 3;
  const int logical = xcd * per + (xcd < rem ? xcd : rem) + j;
  return WorkgroupId{logical % passes, logical / passes};
}

// Passes can share a launch if they walk the same shape in the same way (then they are the same
// kernel instantiation with the same grid); their tensors, direction and scales may differ.
inline bool same_walk(const PassArgs& a, const PassArgs& b) {
  return a.B == b.B && a.T == b.T && a.H == b.H && a.dA == b.dA && a.dB == b.dB && a.nblk == b.nblk &&
         a.block == b.block && a.Ls == b.Ls && a.state_only == b.state_only && a.slots == b.slots &&
         (a.Bout != nullptr || a.Bin != nullptr) == (b.Bout != nullptr || b.Bin != nullptr) &&
         std::memcmp(a.log2g, b.log2g, sizeof a.log2g) == 0;
}

// Plans every pass of a launch and checks that they fit together.  Returns nullptr or a message.
inline const char* plan_passes(PassArgs* planned, const PassArgs* const* passes, int n, int compute_units) {
  if (n < 1 || n > MAX_PASSES_PER_LAUNCH) return "a launch holds one to three passes";
  for (int i = 0; i < n; ++i) {
    planned[i] = *passes[i];
    if (const char* why = plan_pass(planned[i], compute_units)) return why;
    if (i > 0 && !same_walk(planned[0], planned[i])) return "passes that share a launch must walk the same shape the same way";
  }
  return nullptr;
}

// Calls run.template go<DA, MODE, NH>(slot) for the instantiation a planned `a` needs; `slot`
// numbers the instantiations 0 .. PASS_KERNELS - 1.
template <typename Run>
int dispatch_pass(const PassArgs& a, Run&& run) {
  const bool blocks = a.block > 0 && (a.Bout || a.Bin);
  const bool suffix = a.Ls > 0, multi = a.slots < a.B;
  // trailing tokens after the last block boundary, or suffixes in several parts: the general suffix walk
  const bool suffix_any = suffix && (a.T != a.nblk * a.block || a.Ls > CH);
  if (a.dA == 64) {
    if (suffix_any) return run.template go<64, WALK_SUFFIX_ANY, 1>(14);
    if (suffix) return run.template go<64, WALK_SUFFIX, 1>(0);
    if (blocks) return run.template go<64, WALK_BLOCKS, 1>(1);
    if (a.state_only) return run.template go<64, WALK_STATE, 1>(2);
    if (multi) return run.template go<64, WALK_MULTI, 1>(3);
    return run.template go<64, WALK_PLAIN, 1>(4);
  }
  if (a.dA == 128) {
    if (suffix_any) return run.template go<128, WALK_SUFFIX_ANY, 1>(15);
    if (suffix) return run.template go<128, WALK_SUFFIX, 1>(5);
    if (blocks) return run.template go<128, WALK_BLOCKS, 1>(6);
    if (a.state_only) return run.template go<128, WALK_STATE, 1>(7);
    if (multi) return run.template go<128, WALK_MULTI, 1>(8);
    return run.template go<128, WALK_PLAIN, 1>(9);
  }
  if (a.dA == 192) {   // three visits per chunk, 64 of the 192 contraction columns each
    if (suffix_any) return run.template go<64, WALK_SUFFIX_ANY, 3>(17);
    if (suffix) return run.template go<64, WALK_SUFFIX, 3>(18);
    if (a.state_only) return run.template go<64, WALK_STATE, 3>(19);
    if (blocks) return run.template go<64, WALK_BLOCKS, 3>(20);
    return run.template go<64, WALK_PLAIN, 3>(21);
  }
  // dA = 256: two visits per chunk, 128 of the 256 contraction columns each
  if (suffix_any) return run.template go<128, WALK_SUFFIX_ANY, 2>(16);
  if (suffix) return run.template go<128, WALK_SUFFIX, 2>(12);
  if (a.state_only) return run.template go<128, WALK_STATE, 2>(13);
  if (blocks) return run.template go<128, WALK_BLOCKS, 2>(10);
  return run.template go<128, WALK_PLAIN, 2>(11);
}

}  // namespace fpk
