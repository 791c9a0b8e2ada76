// The pass kernel on the CPU thread harness for ONE contraction width: compiled once per width
// with -DEMU_FAMILY=64 / 128 / 192 / 256 (dA = DA x visits per chunk), so that the harness builds
// in parallel.  Test infrastructure only.
#include "device_rt.h"
#include "pass_dispatch.h"
#include "run_grid.h"

#ifndef EMU_FAMILY
#error "compile with -DEMU_FAMILY=<contraction width>"
#endif

namespace {

// one launch of n passes (n = 1: a plain launch) over the planned arguments
struct FamilyRun {
  const fpk::PassArgs* planned;
  int n;
  template <int DA, int MODE, int NH>
  int go(int /*slot*/) const {
    if constexpr (DA * NH == EMU_FAMILY) {
      const fpk::PassArgs& a = planned[0];
      const int nwg = a.slots * a.H * (a.dB / fpk::BV);
      const fpk::PassArgs* const p = planned;
      const int passes = n;
      return run_grid(fpk::NTHREADS_WS, passes * nwg, fpk::lds_bytes_ws(DA), [&](char* l) {
        const fpk::WorkgroupId id = fpk::place_workgroup(fprt::block_index(), nwg, passes);
        fpk::retention_pass_ws<DA, MODE, NH>(a, fpk::tensors_of(p[id.pass]), l, id.wg, nwg);
      });
    } else {
      return 1;   // another width's translation unit
    }
  }
};

}  // namespace

#define EMU_CAT2(a, b) a##b
#define EMU_CAT(a, b) EMU_CAT2(a, b)
int EMU_CAT(emu_pass_, EMU_FAMILY)(const fpk::PassArgs* planned, int n) {
  return fpk::dispatch_pass(planned[0], FamilyRun{planned, n});
}
