// The fused backward, the kernel for the suffixes folded into it and the two kernels for many short
// sequences on the CPU thread harness, for ONE pair of head dimensions: compiled once per pair with
// -DEMU_DK=64|128 -DEMU_DV=64|128, so that the harness builds in parallel.  Test infrastructure only.
#include "device_rt.h"
#include "retention_bwd_fused.h"
#include "short_seq.h"
#include "run_grid.h"

#if !defined(EMU_DK) || !defined(EMU_DV)
#error "compile with -DEMU_DK=<key width> -DEMU_DV=<value width>"
#endif

#define EMU_CAT4(a, b, c, d) a##b##c##d
#define EMU_NAME(stem, dk, dv) EMU_CAT4(stem, dk, _, dv)

namespace {
constexpr int DK = EMU_DK, DV = EMU_DV;

template <int MODE>
int walk(const fpk::FusedBwdArgs& a) {
  return run_grid(fpk::FB_THREADS, 2 * a.B * a.H, fpk::fb_lds_bytes(DK, DV, MODE),
                  [&](char* l) { fpk::fused_bwd<DK, DV, MODE>(a, l, fprt::block_index()); });
}
}  // namespace

// `a` has passed check_fused_bwd and carries the launcher's choice of folding the suffixes
int EMU_NAME(emu_bwd_fused_, EMU_DK, EMU_DV)(const fpk::FusedBwdArgs& a) {
  if (a.d_blocks) return walk<fpk::FB_BLOCKS>(a);
  if (a.fold) {
    if (int rc = walk<fpk::FB_FOLD>(a)) return rc;
    const int pairs = a.B * (a.T / a.block + 1) * a.H;
    return run_grid(fpk::SI_THREADS, pairs < 3 ? pairs : 3, fpk::si_lds_bytes(DK, DV),
                    [&](char* l) { fpk::suffix_intra_bwd<DK, DV>(a, l); });
  }
  if (a.block > 0) return walk<fpk::FB_STOPS>(a);
  return walk<fpk::FB_PLAIN>(a);
}

// `a` has passed check_short_seq_bwd
int EMU_NAME(emu_short_bwd_, EMU_DK, EMU_DV)(const fpk::FusedBwdArgs& a) {
  const int pairs = a.B * a.H, nwg = pairs < 3 ? pairs : 3;   // several pairs per workgroup
  return run_grid(fpk::FB_THREADS, nwg, fpk::ss_lds_bytes(DK, DV), [&](char* l) { fpk::short_seq_bwd<DK, DV>(a, l); });
}

// `a` has passed check_short_seq_fwd
int EMU_NAME(emu_short_fwd_, EMU_DK, EMU_DV)(const fpk::ShortFwdArgs& a) {
  const int pairs = a.B * a.H, nwg = pairs < 3 ? pairs : 3;
  return run_grid(fpk::FB_THREADS, nwg, fpk::ss_fwd_lds_bytes(DK, DV), [&](char* l) { fpk::short_seq_fwd<DK, DV>(a, l); });
}
