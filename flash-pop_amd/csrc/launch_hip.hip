// gfx950 entry points of the pass kernels and the launcher the C-ABI layer calls.
#include <atomic>

#include "device_rt.h"
#include "retention_pass_ws.h"
#include "segment_scan.h"
#include "decode_step.h"

namespace {

// 8 waves, double-buffered LDS; NH = 2 covers dA = 256 in two visits per chunk.
template <int DA, int MODE, int NH = 1>
__global__ __launch_bounds__(fpk::NTHREADS_WS) void retention_pass_ws_kernel(const fpk::PassArgs args) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  fpk::retention_pass_ws<DA, MODE, NH>(args, lds);
}

__global__ __launch_bounds__(fpk::SCAN_THREADS) void segment_scan_kernel(const fpk::ScanArgs args) {
  fpk::segment_scan(args);
}

__global__ __launch_bounds__(fpk::DECODE_THREADS) void decode_step_kernel(const fpk::DecodeArgs args) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  fpk::decode_step(args, lds);
}

// LDS above 64 KB has to be opted into once per device and kernel.  One bit per kernel (`slot`)
// and device, shared by all threads of the process: once any thread has run a kernel on a device,
// no thread calls hipFuncSetAttribute for it again (which matters to callers that capture
// launches into a graph after a warm-up run).  Setting the attribute twice in a race is harmless.
constexpr int kMaxDevices = 64;
std::atomic<uint32_t> g_armed[kMaxDevices];

template <typename Kernel>
int launch(Kernel kernel, int threads, int lds, int slot, const fpk::PassArgs& a, hipStream_t stream,
           const char** err) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) {
    *err = "hipGetDevice failed";
    return 1;
  }
  const bool tracked = dev >= 0 && dev < kMaxDevices;
  if (!tracked || !(g_armed[dev].load(std::memory_order_acquire) & (1u << slot))) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, lds) !=
        hipSuccess) {
      (void)hipGetLastError();
      *err = "hipFuncSetAttribute(MaxDynamicSharedMemorySize) failed";
      return 1;
    }
    if (tracked) g_armed[dev].fetch_or(1u << slot, std::memory_order_release);
  }
  const int nwg = a.slots * a.H * (a.dB / fpk::BV);
  hipLaunchKernelGGL(kernel, dim3(nwg), dim3(threads), lds, stream, a);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    *err = hipGetErrorString(e);
    return 1;
  }
  return 0;
}

}  // namespace

#ifdef FPK_PROFILE
extern "C" int fpk_prof_set(void* buf) {
  return (int)hipMemcpyToSymbol(HIP_SYMBOL(fprt::g_prof_buf), &buf, sizeof buf);
}
#endif
#ifdef FPK_DBGFLAGS
extern "C" int fpk_dbg_set(int flags) {
  return (int)hipMemcpyToSymbol(HIP_SYMBOL(fprt::g_dbg_flags), &flags, sizeof flags);
}
#endif

// Compute units of the current device (cached per thread and device).
int fpk_compute_units() {
  static thread_local int dev_cached = -1, cus = 0;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 256;
  if (dev != dev_cached) {
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
    dev_cached = dev;
  }
  return cus;
}

int fpk_launch_pass(const fpk::PassArgs& args, void* stream, const char** err) {
  hipStream_t s = static_cast<hipStream_t>(stream);
  fpk::PassArgs a = args;
  const bool blocks = a.block > 0 && (a.Bout || a.Bin);
  const bool ws = a.dA == 64 || a.dA == 128;
  const bool suffix = a.Ls > 0;
  if (suffix) {
    // what the suffix walk assumes; the C-ABI layer reports these to the caller in its own words
    if (!ws || blocks || a.block <= 0 || a.T != a.nblk * a.block || a.Ls > fpk::CH || !a.Xs || !a.Ws || !a.Zs || !a.Ys) {
      *err = "suffix walk: needs dA of 64 or 128, T == nblk * block, 1 <= Ls <= 64 and all four suffix tensors";
      return 1;
    }
    a.slots = a.B;
  }
  // One workgroup per (batch entry, head, column tile) while that fits the chip once; beyond that
  // the plain wave-specialised kernel lets each workgroup walk several batch entries, which keeps
  // its load pipeline full across short sequences.
  if (a.slots <= 0) {
    a.slots = a.B;
    if (ws && !blocks && !suffix) {
      const int per_slot = a.H * (a.dB / fpk::BV);
      int fit = fpk_compute_units() / per_slot;
      if (fit < 1) fit = 1;
      if (fit < a.B) a.slots = fit;
    }
  }
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
  switch (a.dA) {
    case 64:
      if (suffix) return launch(retention_pass_ws_kernel<64, fpk::WALK_SUFFIX>, fpk::NTHREADS_WS, fpk::lds_bytes_ws(64), 7, a, s, err);
      if (blocks) return launch(retention_pass_ws_kernel<64, fpk::WALK_BLOCKS>, fpk::NTHREADS_WS, fpk::lds_bytes_ws(64), 0, a, s, err);
      if (a.state_only) return launch(retention_pass_ws_kernel<64, fpk::WALK_STATE>, fpk::NTHREADS_WS, fpk::lds_bytes_ws(64), 9, a, s, err);
      if (multi) return launch(retention_pass_ws_kernel<64, fpk::WALK_MULTI>, fpk::NTHREADS_WS, fpk::lds_bytes_ws(64), 1, a, s, err);
      return launch(retention_pass_ws_kernel<64, fpk::WALK_PLAIN>, fpk::NTHREADS_WS, fpk::lds_bytes_ws(64), 2, a, s, err);
    case 128:
      if (suffix) return launch(retention_pass_ws_kernel<128, fpk::WALK_SUFFIX>, fpk::NTHREADS_WS, fpk::lds_bytes_ws(128), 8, a, s, err);
      if (blocks) return launch(retention_pass_ws_kernel<128, fpk::WALK_BLOCKS>, fpk::NTHREADS_WS, fpk::lds_bytes_ws(128), 3, a, s, err);
      if (a.state_only) return launch(retention_pass_ws_kernel<128, fpk::WALK_STATE>, fpk::NTHREADS_WS, fpk::lds_bytes_ws(128), 10, a, s, err);
      if (multi) return launch(retention_pass_ws_kernel<128, fpk::WALK_MULTI>, fpk::NTHREADS_WS, fpk::lds_bytes_ws(128), 4, a, s, err);
      return launch(retention_pass_ws_kernel<128, fpk::WALK_PLAIN>, fpk::NTHREADS_WS, fpk::lds_bytes_ws(128), 5, a, s, err);
    case 256:   // two visits per chunk, 128 of the 256 contraction columns each
      if (blocks) return launch(retention_pass_ws_kernel<128, fpk::WALK_BLOCKS, 2>, fpk::NTHREADS_WS, fpk::lds_bytes_ws(128), 6, a, s, err);
      return launch(retention_pass_ws_kernel<128, fpk::WALK_PLAIN, 2>, fpk::NTHREADS_WS, fpk::lds_bytes_ws(128), 11, a, s, err);
    default: *err = "unsupported contraction width (dA must be 64, 128 or 256)"; return 1;
  }
}

int fpk_launch_scan(const fpk::ScanArgs& a, void* stream, const char** err) {
  if (a.M % fpk::SCAN_VEC != 0 || a.B < 1 || a.S < 1 || a.H < 1 || !a.U || !a.init) {
    *err = "segment scan: bad arguments";
    return 1;
  }
  const long long items = (long long)a.B * a.H * (a.M / fpk::SCAN_VEC);
  const long long blocks = (items + fpk::SCAN_THREADS - 1) / fpk::SCAN_THREADS;
  if (blocks > 0x7fffffffLL) {
    *err = "segment scan: too many state matrices";
    return 1;
  }
  hipLaunchKernelGGL(segment_scan_kernel, dim3((unsigned)blocks), dim3(fpk::SCAN_THREADS), 0,
                     static_cast<hipStream_t>(stream), a);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    *err = hipGetErrorString(e);
    return 1;
  }
  return 0;
}

int fpk_launch_decode(const fpk::DecodeArgs& a, void* stream, const char** err) {
  if (a.B < 1 || a.H < 1 || a.H > fpk::MAX_HEADS || a.dk < 1 || a.dv < 8 || a.dv % 8 != 0 ||
      fpk::DECODE_THREADS % (a.dv / 8) != 0 || a.dv > fpk::DECODE_THREADS || !a.q || !a.k || !a.v || !a.s_out || !a.o) {
    *err = "decode step: bad arguments";
    return 1;
  }
  hipLaunchKernelGGL(decode_step_kernel, dim3((unsigned)(a.B * a.H)), dim3(fpk::DECODE_THREADS),
                     fpk::decode_lds_bytes(a.dv), static_cast<hipStream_t>(stream), a);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    *err = hipGetErrorString(e);
    return 1;
  }
  return 0;
}
