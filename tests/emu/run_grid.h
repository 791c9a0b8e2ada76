// One OS thread per GPU lane, the workgroups of a launch one after another (shared by the harness's
// translation units).  Test infrastructure only.
#pragma once
#include "device_rt.h"

#include <thread>
#include <vector>

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
