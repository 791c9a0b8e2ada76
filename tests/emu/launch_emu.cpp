// CPU implementation of fpk_launch_pass: runs the kernel body with 256 OS threads per
// workgroup, workgroups one after another.  Test infrastructure only.
#include "device_rt.h"
#include "retention_pass.h"

#include <thread>
#include <vector>

namespace fprt {
thread_local LaneCtx g_lane;
}

namespace {

template <int DA>
int launch(const fpk::PassArgs& a) {
  const int nwg = a.B * a.H * (a.dB / fpk::BV);
  // exactly the bytes the GPU launch reserves, on the heap so that ASan sees overruns
  std::vector<char>* lds = new std::vector<char>(fpk::lds_bytes(DA));
  pthread_barrier_t wg_bar;
  pthread_barrier_init(&wg_bar, nullptr, fpk::NTHREADS);
  std::vector<fprt::WaveShared> waves(fpk::NTHREADS / 64);
  for (auto& w : waves) pthread_barrier_init(&w.bar, nullptr, 64);
  std::vector<std::thread> lanes;
  for (int t = 0; t < fpk::NTHREADS; ++t) {
    lanes.emplace_back([&, t] {
      fprt::g_lane.tid = t;
      fprt::g_lane.grid = nwg;
      fprt::g_lane.wave = &waves[t >> 6];
      fprt::g_lane.wg_bar = &wg_bar;
      for (int wg = 0; wg < nwg; ++wg) {
        fprt::g_lane.block = wg;
        fpk::retention_pass<DA>(a, lds->data());
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

int fpk_launch_pass(const fpk::PassArgs& a, void* /*stream*/, const char** err) {
  switch (a.dA) {
    case 64: return launch<64>(a);
    case 128: return launch<128>(a);
    case 256: return launch<256>(a);
    default: *err = "unsupported contraction width (dA must be 64, 128 or 256)"; return 1;
  }
}
