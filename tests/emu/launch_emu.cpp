// CPU implementation of fpk_launch_pass: runs the kernel bodies with one OS thread per GPU
// lane, workgroups one after another.  Test infrastructure only.
#include "device_rt.h"
#include "retention_pass_ws.h"
#include "segment_scan.h"
#include "decode_step.h"

#include <thread>
#include <vector>

namespace fprt {
thread_local LaneCtx g_lane;
}

namespace {

template <typename Body>
int run_grid(int nthreads, int nwg, int lds_bytes, Body body) {
  // exactly the bytes the GPU launch reserves, on the heap so that ASan sees overruns
  std::vector<char>* lds = new std::vector<char>(lds_bytes);
  pthread_barrier_t wg_bar;
  pthread_barrier_init(&wg_bar, nullptr, nthreads);
  std::vector<fprt::WaveShared> waves(nthreads / 64);
  for (auto& w : waves) pthread_barrier_init(&w.bar, nullptr, 64);
  std::vector<std::thread> lanes;
  for (int t = 0; t < nthreads; ++t) {
    lanes.emplace_back([&, t] {
      fprt::g_lane.tid = t;
      fprt::g_lane.grid = nwg;
      fprt::g_lane.wave = &waves[t >> 6];
      fprt::g_lane.wg_bar = &wg_bar;
      for (int wg = 0; wg < nwg; ++wg) {
        fprt::g_lane.block = wg;
        body(lds->data());
        pthread_barrier_wait(&wg_bar);
      }
    });
  }
  for (auto& th : lanes) th.join();
  for (auto& w : waves) pthread_barrier_destroy(&w.bar);
  pthread_barrier_destroy(&wg_bar);
  delete lds;
  return 0;
}

}  // namespace

int fpk_launch_pass(const fpk::PassArgs& args, void* /*stream*/, const char** err) {
  fpk::PassArgs a = args;
  const bool blocks = a.block > 0 && (a.Bout || a.Bin);
  const bool ws = a.dA == 64 || a.dA == 128;
  const bool suffix = a.Ls > 0;
  if (suffix) {
    if (!ws || blocks || a.block <= 0 || a.T != a.nblk * a.block || a.Ls > fpk::CH || !a.Xs || !a.Ws || !a.Zs || !a.Ys) {
      *err = "suffix walk: needs dA of 64 or 128, T == nblk * block, 1 <= Ls <= 64 and all four suffix tensors";
      return 1;
    }
    a.slots = a.B;
  }
  // Pretend the chip is tiny, so that the several-entries-per-workgroup path is exercised:
  // at most two workgroups per (head, column tile).
  if (a.slots <= 0) a.slots = (ws && !blocks && !suffix && a.B > 2) ? 2 : a.B;
  if (a.slots > a.B) a.slots = a.B;
  const bool multi = a.slots < a.B;
  if (a.state_only && (!ws || blocks || suffix || !a.Rout)) {
    *err = "state-only walk: needs dA of 64 or 128, a final-state buffer, no block states and no suffixes";
    return 1;
  }
  if (multi && (!ws || blocks || suffix)) {
    *err = "several batch entries per workgroup: only for the plain walk with dA of 64 or 128";
    return 1;
  }
  const int nwg = a.slots * a.H * (a.dB / fpk::BV);
  switch (a.dA) {
    case 64:
      if (suffix) return run_grid(fpk::NTHREADS_WS, nwg, fpk::lds_bytes_ws(64), [&](char* l) { fpk::retention_pass_ws<64, fpk::WALK_SUFFIX>(a, l); });
      if (blocks) return run_grid(fpk::NTHREADS_WS, nwg, fpk::lds_bytes_ws(64), [&](char* l) { fpk::retention_pass_ws<64, fpk::WALK_BLOCKS>(a, l); });
      if (a.state_only) return run_grid(fpk::NTHREADS_WS, nwg, fpk::lds_bytes_ws(64), [&](char* l) { fpk::retention_pass_ws<64, fpk::WALK_STATE>(a, l); });
      if (multi) return run_grid(fpk::NTHREADS_WS, nwg, fpk::lds_bytes_ws(64), [&](char* l) { fpk::retention_pass_ws<64, fpk::WALK_MULTI>(a, l); });
      return run_grid(fpk::NTHREADS_WS, nwg, fpk::lds_bytes_ws(64), [&](char* l) { fpk::retention_pass_ws<64, fpk::WALK_PLAIN>(a, l); });
    case 128:
      if (suffix) return run_grid(fpk::NTHREADS_WS, nwg, fpk::lds_bytes_ws(128), [&](char* l) { fpk::retention_pass_ws<128, fpk::WALK_SUFFIX>(a, l); });
      if (blocks) return run_grid(fpk::NTHREADS_WS, nwg, fpk::lds_bytes_ws(128), [&](char* l) { fpk::retention_pass_ws<128, fpk::WALK_BLOCKS>(a, l); });
      if (a.state_only) return run_grid(fpk::NTHREADS_WS, nwg, fpk::lds_bytes_ws(128), [&](char* l) { fpk::retention_pass_ws<128, fpk::WALK_STATE>(a, l); });
      if (multi) return run_grid(fpk::NTHREADS_WS, nwg, fpk::lds_bytes_ws(128), [&](char* l) { fpk::retention_pass_ws<128, fpk::WALK_MULTI>(a, l); });
      return run_grid(fpk::NTHREADS_WS, nwg, fpk::lds_bytes_ws(128), [&](char* l) { fpk::retention_pass_ws<128, fpk::WALK_PLAIN>(a, l); });
    case 256:
      if (blocks) return run_grid(fpk::NTHREADS_WS, nwg, fpk::lds_bytes_ws(128), [&](char* l) { fpk::retention_pass_ws<128, fpk::WALK_BLOCKS, 2>(a, l); });
      return run_grid(fpk::NTHREADS_WS, nwg, fpk::lds_bytes_ws(128), [&](char* l) { fpk::retention_pass_ws<128, fpk::WALK_PLAIN, 2>(a, l); });
    default: *err = "unsupported contraction width (dA must be 64, 128 or 256)"; return 1;
  }
}

// Pretends the chip has 8 compute units, so that small test shapes take the paths that large
// ones take on a real device (several sequences per workgroup, split sequences).
int fpk_compute_units() { return 8; }

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
      fpk::DECODE_THREADS % (a.dv / 8) != 0 || a.dv > fpk::DECODE_THREADS || !a.q || !a.k || !a.v || !a.s_out || !a.o) {
    *err = "decode step: bad arguments";
    return 1;
  }
  return run_grid(fpk::DECODE_THREADS, a.B * a.H, fpk::decode_lds_bytes(a.dv), [&](char* l) { fpk::decode_step(a, l); });
}
