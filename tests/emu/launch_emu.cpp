// CPU implementation of fpk_launch_pass: runs the kernel bodies with one OS thread per GPU
// lane, workgroups one after another.  Test infrastructure only.
#include "device_rt.h"
#include "pass_dispatch.h"
#include "segment_scan.h"
#include "segment_contrib.h"
#include "retention_bwd_fused.h"
#include "short_seq.h"
#include "decode_step.h"
#include "layer_ops.h"

#include <vector>

namespace fprt {
thread_local LaneCtx g_lane;
}

#include "run_grid.h"

// The pass kernel's instantiations are compiled one contraction width per translation unit
// (pass_family.cpp, built once per width) so that the harness builds in parallel.
int emu_pass_64(const fpk::PassArgs* planned, int n);
int emu_pass_128(const fpk::PassArgs* planned, int n);
int emu_pass_192(const fpk::PassArgs* planned, int n);
int emu_pass_256(const fpk::PassArgs* planned, int n);

namespace {

int run_family(const fpk::PassArgs* planned, int n) {
  switch (planned[0].dA) {
    case 64: return emu_pass_64(planned, n);
    case 128: return emu_pass_128(planned, n);
    case 192: return emu_pass_192(planned, n);
    default: return emu_pass_256(planned, n);
  }
}

}  // namespace

int fpk_launch_pass(const fpk::PassArgs& args, void* /*stream*/, const char** err) {
  fpk::PassArgs a = args;
  if (const char* why = fpk::plan_pass(a, fpk_compute_units())) {
    *err = why;
    return 1;
  }
  return run_family(&a, 1);
}

int fpk_launch_passes(const fpk::PassArgs* const* passes, int n, void* stream, const char** err) {
  if (n == 1) return fpk_launch_pass(*passes[0], stream, err);
  fpk::PassArgs planned[fpk::MAX_PASSES_PER_LAUNCH];
  if (const char* why = fpk::plan_passes(planned, passes, n, fpk_compute_units())) {
    *err = why;
    return 1;
  }
  return run_family(planned, n);
}

// the harness's stand-in for the library's own scratch array (host memory here)
int fpk_static_scratch(void** ptr, const char** /*err*/) {
  static std::vector<unsigned char> scratch(fpk::STATIC_SCRATCH_BYTES);
  *ptr = scratch.data();
  return 0;
}

// A test can pretend that streams are capturing (the C entry points of the pass kernels must refuse then).
static int g_emu_capturing = 0;
extern "C" void emu_set_capturing(int on) { g_emu_capturing = on; }
int fpk_stream_is_capturing(void* /*stream*/) { return g_emu_capturing; }

// Pretends the chip has 8 compute units, so that small test shapes take the paths that large
// ones take on a real device (several sequences per workgroup, split sequences).
int fpk_compute_units() { return 8; }

// one translation unit per pair of head dimensions (fused_family.cpp)
#define EMU_FUSED_FAMILY(DK, DV)                                  \
  int emu_bwd_fused_##DK##_##DV(const fpk::FusedBwdArgs& a);      \
  int emu_short_bwd_##DK##_##DV(const fpk::FusedBwdArgs& a);      \
  int emu_short_fwd_##DK##_##DV(const fpk::ShortFwdArgs& a);
EMU_FUSED_FAMILY(128, 128)
EMU_FUSED_FAMILY(64, 128)
EMU_FUSED_FAMILY(128, 64)
EMU_FUSED_FAMILY(64, 64)
#undef EMU_FUSED_FAMILY

int fpk_launch_bwd_fused(const fpk::FusedBwdArgs& args, void* /*stream*/, const char** err) {
  fpk::FusedBwdArgs a = args;
  a.fold = a.block > 0 && a.Ls <= fpk::FB_SFX_ROWS;
  if (const char* why = fpk::check_fused_bwd(a)) {
    *err = why;
    return 1;
  }
  // the two workgroups of a stream run one after the other here, so the pacing words are written and read but never waited for
  static uint32_t pace_words[fpk::PACE_SLOTS];
  static uint32_t launches = 1;
  a.pace = nullptr;
  if (fpk::fused_bwd_paces(a, fpk_compute_units(), true)) {   // whatever the pretended device
    a.pace = pace_words;
    a.pace_base = launches++ << 16;
  }
  if (a.dk_dim == 128 && a.dv_dim == 128) return emu_bwd_fused_128_128(a);
  if (a.dk_dim == 64 && a.dv_dim == 128) return emu_bwd_fused_64_128(a);
  if (a.dk_dim == 128 && a.dv_dim == 64) return emu_bwd_fused_128_64(a);
  return emu_bwd_fused_64_64(a);
}

int fpk_launch_short_bwd(const fpk::FusedBwdArgs& a, void* /*stream*/, const char** err) {
  if (const char* why = fpk::check_short_seq_bwd(a)) {
    *err = why;
    return 1;
  }
  if (a.dk_dim == 128 && a.dv_dim == 128) return emu_short_bwd_128_128(a);
  if (a.dk_dim == 64 && a.dv_dim == 128) return emu_short_bwd_64_128(a);
  if (a.dk_dim == 128 && a.dv_dim == 64) return emu_short_bwd_128_64(a);
  return emu_short_bwd_64_64(a);
}

int fpk_launch_short_fwd(const fpk::ShortFwdArgs& a, void* /*stream*/, const char** err) {
  if (const char* why = fpk::check_short_seq_fwd(a)) {
    *err = why;
    return 1;
  }
  if (a.dk_dim == 128 && a.dv_dim == 128) return emu_short_fwd_128_128(a);
  if (a.dk_dim == 64 && a.dv_dim == 128) return emu_short_fwd_64_128(a);
  if (a.dk_dim == 128 && a.dv_dim == 64) return emu_short_fwd_128_64(a);
  return emu_short_fwd_64_64(a);
}

int fpk_launch_contrib(const fpk::ContribArgs& a, void* /*stream*/, const char** err) {
  if (const char* why = fpk::check_contrib(a)) {
    *err = why;
    return 1;
  }
  return run_grid(fpk::FB_THREADS, a.B * a.H * (a.dB / fpk::FB_D), fpk::sc_lds_bytes(), [&](char* l) {
    if (a.reverse) fpk::segment_contrib<true>(a, l);
    else fpk::segment_contrib<false>(a, l);
  });
}

int fpk_launch_scan(const fpk::ScanArgs& a, void* /*stream*/, const char** err) {
  if (a.M % fpk::SCAN_VEC != 0 || a.B < 1 || a.S < 1 || a.H < 1 || !a.U || !a.init) {
    *err = "segment scan: bad arguments";
    return 1;
  }
  const long long items = (long long)a.B * a.H * (a.M / fpk::SCAN_VEC);
  const int blocks = (int)((items + fpk::SCAN_THREADS - 1) / fpk::SCAN_THREADS);
  // no barriers inside: the lanes can run one after another on this thread
  for (int blk = 0; blk < blocks; ++blk) {
    for (int t = 0; t < fpk::SCAN_THREADS; ++t) {
      fprt::g_lane.tid = t;
      fprt::g_lane.block = blk;
      fprt::g_lane.grid = blocks;
      fpk::segment_scan(a);
    }
  }
  return 0;
}

int fpk_launch_decode(const fpk::DecodeArgs& a, void* /*stream*/, const char** err) {
  if (a.B < 1 || a.H < 1 || a.H > fpk::MAX_HEADS || a.dk < 1 || a.dv < 8 || a.dv % 8 != 0 ||
      a.dv > fpk::DECODE_THREADS || !a.q || !a.k || !a.v || !a.s_out || !a.o) {
    *err = "decode step: bad arguments";
    return 1;
  }
  return run_grid(fpk::DECODE_THREADS, a.B * a.H, fpk::decode_lds_bytes(a.dv), [&](char* l) { fpk::decode_step(a, l); });
}

int fpk_launch_rotary(const fpk::RotaryArgs& args, void* /*stream*/, const char** err) {
  fpk::RotaryArgs a = args;
  long long blocks = 0;
  if (const char* why = fpk::plan_rotary(a, blocks)) {
    *err = why;
    return 1;
  }
  // no barriers and no lane exchanges inside: the lanes can run one after another on this thread
  for (long long blk = 0; blk < blocks; ++blk) {
    for (int t = 0; t < fpk::LAYER_THREADS; ++t) {
      fprt::g_lane.tid = t;
      fprt::g_lane.block = (int)blk;
      fprt::g_lane.grid = (int)blocks;
      fpk::rotary_qk(a);
    }
  }
  return 0;
}

int fpk_launch_gated_norm(const fpk::GatedNormArgs& a, void* /*stream*/, const char** err) {
  long long blocks = 0;
  if (const char* why = fpk::plan_gated_norm(a, blocks)) {
    *err = why;
    return 1;
  }
  return run_grid(fpk::LAYER_THREADS, (int)blocks, 0, [&](char*) {
    if (a.out) fpk::gated_norm_fwd(a);
    else fpk::gated_norm_bwd(a);
  });
}
