// gfx950 entry points of the pass kernels and the launcher the C-ABI layer calls.
#include <atomic>

#include "device_rt.h"
#include "pass_dispatch.h"
#include "segment_scan.h"
#include "segment_contrib.h"
#include "retention_bwd_fused.h"
#include "short_seq.h"
#include "decode_step.h"
#include "layer_ops.h"

namespace {

// 8 waves, double-buffered LDS; NH = 2 covers dA = 256 in two visits per chunk.
template <int DA, int MODE, int NH = 1>
__global__ __launch_bounds__(fpk::NTHREADS_WS) void retention_pass_ws_kernel(const fpk::PassArgs args) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  const int nwg = fprt::grid_size();
  fpk::retention_pass_ws<DA, MODE, NH>(args, fpk::tensors_of(args), lds, fpk::place_workgroup(fprt::block_index(), nwg, 1).wg, nwg);
}

// Up to three independent passes over the same shape in one grid (see fpk_launch_passes).
template <int DA, int MODE, int NH = 1>
__global__ __launch_bounds__(fpk::NTHREADS_WS) void retention_pass_multi_kernel(const fpk::PassArgs first,
                                                                                const fpk::PassTensors second,
                                                                                const fpk::PassTensors third,
                                                                                const int passes) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  const int nwg = fprt::grid_size() / passes;
  const fpk::WorkgroupId id = fpk::place_workgroup(fprt::block_index(), nwg, passes);
  const fpk::PassTensors io = id.pass == 0 ? fpk::tensors_of(first) : id.pass == 1 ? second : third;
  fpk::retention_pass_ws<DA, MODE, NH>(first, io, lds, id.wg, nwg);
}

// MODE: how POP suffixes take part (fpk::FbMode): none, as extra stops of the walks, or (at most 16 tokens) folded into
// the chunks at their boundaries, with suffix_intra_bwd_kernel for what stays inside such a suffix
template <int DK, int DV, int MODE>
__global__ __launch_bounds__(fpk::FB_THREADS) void retention_bwd_fused_kernel(const fpk::FusedBwdArgs args) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  fpk::fused_bwd<DK, DV, MODE>(args, lds, fprt::block_index());
}
template <int DK, int DV>
__global__ __launch_bounds__(fpk::SI_THREADS) void suffix_intra_bwd_kernel(const fpk::FusedBwdArgs args) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  fpk::suffix_intra_bwd<DK, DV>(args, lds);
}

template <int DK, int DV>
__global__ __launch_bounds__(fpk::FB_THREADS) void short_seq_bwd_kernel(const fpk::FusedBwdArgs args) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  fpk::short_seq_bwd<DK, DV>(args, lds);
}

template <int DK, int DV>
__global__ __launch_bounds__(fpk::FB_THREADS) void short_seq_fwd_kernel(const fpk::ShortFwdArgs args) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  fpk::short_seq_fwd<DK, DV>(args, lds);
}

__global__ __launch_bounds__(fpk::SCAN_THREADS) void segment_scan_kernel(const fpk::ScanArgs args) {
  fpk::segment_scan(args);
}

template <bool REV>
__global__ __launch_bounds__(fpk::FB_THREADS) void segment_contrib_kernel(const fpk::ContribArgs args) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  fpk::segment_contrib<REV>(args, lds);
}

__global__ __launch_bounds__(fpk::DECODE_THREADS) void decode_step_kernel(const fpk::DecodeArgs args) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  fpk::decode_step(args, lds);
}

__global__ __launch_bounds__(fpk::LAYER_THREADS) void rotary_qk_kernel(const fpk::RotaryArgs args) {
  fpk::rotary_qk(args);
}

__global__ __launch_bounds__(fpk::LAYER_THREADS) void gated_norm_fwd_kernel(const fpk::GatedNormArgs args) {
  fpk::gated_norm_fwd(args);
}

__global__ __launch_bounds__(fpk::LAYER_THREADS) void gated_norm_bwd_kernel(const fpk::GatedNormArgs args) {
  fpk::gated_norm_bwd(args);
}

// LDS above 64 KB has to be opted into once per device and kernel.  One bit per kernel (`slot`)
// and device, shared by all threads of the process: once any thread has run a kernel on a device,
// no thread calls hipFuncSetAttribute for it again (which matters to callers that capture
// launches into a graph after a warm-up run).  Setting the attribute twice in a race is harmless.
constexpr int kMaxDevices = 64;
static_assert(2 * fpk::PASS_KERNELS <= 57, "one bit per kernel instantiation, single and paired; the top six for the others");
std::atomic<uint64_t> g_armed[kMaxDevices][2];   // slots 0..63: pass kernels and the small ones; 64..127: the fused backward family

template <typename Kernel, typename... More>
int launch(Kernel kernel, int threads, int lds, int slot, int passes, hipStream_t stream, const char** err,
           const fpk::PassArgs& a, const More&... more) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) {
    *err = "hipGetDevice failed";
    return 1;
  }
  const bool tracked = dev >= 0 && dev < kMaxDevices;
  if (!tracked || !(g_armed[dev][0].load(std::memory_order_acquire) & (1ull << slot))) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, lds) !=
        hipSuccess) {
      (void)hipGetLastError();
      *err = "hipFuncSetAttribute(MaxDynamicSharedMemorySize) failed";
      return 1;
    }
    if (tracked) g_armed[dev][0].fetch_or(1ull << slot, std::memory_order_release);
  }
  const int nwg = a.slots * a.H * (a.dB / fpk::BV) * passes;
  hipLaunchKernelGGL(kernel, dim3(nwg), dim3(threads), lds, stream, a, more...);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    *err = hipGetErrorString(e);
    return 1;
  }
  return 0;
}

}  // namespace


// ---- scratch memory that no call allocates ------------------------------------------------------
// fp_retention_fwd_split_static runs the split-sequence forward without a workspace from the
// caller: the segment states live in this array, of which every device holds its own copy at
// its own address from the moment the code object is loaded until the process ends.  The name of
// the array means nothing to host code; its address on the current device comes from
// hipGetSymbolAddress, once per device, and is what kernels and host calls are given afterwards.
static __device__ __align__(256) unsigned char scratch[fpk::STATIC_SCRATCH_BYTES];

namespace {
std::atomic<void*> g_scratch_ptr[kMaxDevices];
}

int fpk_static_scratch(void** ptr, const char** err) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) {
    *err = "hipGetDevice failed";
    return 1;
  }
  if (dev < 0 || dev >= kMaxDevices) {
    *err = "device index beyond the table of per-device scratch addresses";
    return 1;
  }
  void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!p) {
    // first call on this device (it is the current one): look the array's address up and keep it
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) {
      (void)hipGetLastError();
      *err = "hipGetSymbolAddress(scratch) failed";
      return 1;
    }
    g_scratch_ptr[dev].store(p, std::memory_order_release);
  }
  *ptr = p;
  return 0;
}

// ---- pacing words of the fused backward -----------------------------------------------------------
// One word per (batch, head) stream, through which the reverse workgroup of a stream tells the dq workgroup how
// far it is (FusedBwdArgs::pace).  Every launch tags its values with a number of its own, so nothing is ever
// cleared; launches that overlap on one device share the words and at worst pace each other badly.
static __device__ __align__(256) uint32_t pace_words[fpk::PACE_SLOTS];

namespace {
std::atomic<void*> g_pace_ptr[kMaxDevices];
std::atomic<uint32_t> g_pace_launch{1};

// the words' address on the current device (nullptr: pacing stays off for this launch)
uint32_t* pace_words_here() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
  void* p = g_pace_ptr[dev].load(std::memory_order_acquire);
  if (!p) {
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(pace_words)) != hipSuccess || !p) {
      (void)hipGetLastError();
      return nullptr;
    }
    g_pace_ptr[dev].store(p, std::memory_order_release);
  }
  return static_cast<uint32_t*>(p);
}
}  // namespace

int fpk_stream_is_capturing(void* stream) {
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(static_cast<hipStream_t>(stream), &status) != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  return status != hipStreamCaptureStatusNone;
}

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

namespace {

struct DeviceRun {
  const fpk::PassArgs& a;
  hipStream_t stream;
  const char** err;
  template <int DA, int MODE, int NH>
  int go(int slot) const {
    return launch(retention_pass_ws_kernel<DA, MODE, NH>, fpk::NTHREADS_WS, fpk::lds_bytes_ws(DA), slot, 1, stream, err, a);
  }
};

struct DeviceMultiRun {
  const fpk::PassArgs* planned;
  int n;
  hipStream_t stream;
  const char** err;
  template <int DA, int MODE, int NH>
  int go(int slot) const {
    return launch(retention_pass_multi_kernel<DA, MODE, NH>, fpk::NTHREADS_WS, fpk::lds_bytes_ws(DA),
                  fpk::PASS_KERNELS + slot, n, stream, err, planned[0], fpk::tensors_of(planned[1]),
                  fpk::tensors_of(planned[n - 1]), n);
  }
};

}  // namespace

int fpk_launch_pass(const fpk::PassArgs& args, void* stream, const char** err) {
  fpk::PassArgs a = args;
  if (const char* why = fpk::plan_pass(a, fpk_compute_units())) {
    *err = why;
    return 1;
  }
  return fpk::dispatch_pass(a, DeviceRun{a, static_cast<hipStream_t>(stream), err});
}

int fpk_launch_passes(const fpk::PassArgs* const* passes, int n, void* stream, const char** err) {
  if (n == 1) return fpk_launch_pass(*passes[0], stream, err);
  fpk::PassArgs planned[fpk::MAX_PASSES_PER_LAUNCH];
  if (const char* why = fpk::plan_passes(planned, passes, n, fpk_compute_units())) {
    *err = why;
    return 1;
  }
  return fpk::dispatch_pass(planned[0], DeviceMultiRun{planned, n, static_cast<hipStream_t>(stream), err});
}

namespace {

// opts a kernel into `lds` bytes of dynamic LDS once per device (bit `bit` of the 128 per device)
int arm(const void* kernel, int lds, int bit, const char** err) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) {
    *err = "hipGetDevice failed";
    return 1;
  }
  const uint64_t mask = 1ull << (bit & 63);
  const int word = bit >> 6;
  const bool tracked = dev >= 0 && dev < kMaxDevices;
  if (!tracked || !(g_armed[dev][word].load(std::memory_order_acquire) & mask)) {
    if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess) {
      (void)hipGetLastError();
      *err = "hipFuncSetAttribute(MaxDynamicSharedMemorySize) failed";
      return 1;
    }
    if (tracked) g_armed[dev][word].fetch_or(mask, std::memory_order_release);
  }
  return 0;
}

int launched(const char** err) {
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    *err = hipGetErrorString(e);
    return 1;
  }
  return 0;
}

}  // namespace

namespace {

// one (dk, dv) instantiation of the fused backward family; `slot` numbers its five kernels 64 + 5 slot ..
template <int DK, int DV>
int launch_bwd_fused(const fpk::FusedBwdArgs& a, int slot, hipStream_t st, const char** err) {
  const dim3 grid((unsigned)(2 * a.B * a.H)), threads(fpk::FB_THREADS);
  const int bit = 64 + 5 * slot;
  if (a.d_blocks) {
    constexpr int lds = fpk::fb_lds_bytes(DK, DV, fpk::FB_BLOCKS);
    if (arm(reinterpret_cast<const void*>(retention_bwd_fused_kernel<DK, DV, fpk::FB_BLOCKS>), lds, bit + 4, err)) return 1;
    hipLaunchKernelGGL((retention_bwd_fused_kernel<DK, DV, fpk::FB_BLOCKS>), grid, threads, lds, st, a);
    return launched(err);
  }
  if (a.fold) {
    constexpr int lds = fpk::fb_lds_bytes(DK, DV, fpk::FB_FOLD), lds_si = fpk::si_lds_bytes(DK, DV);
    if (arm(reinterpret_cast<const void*>(retention_bwd_fused_kernel<DK, DV, fpk::FB_FOLD>), lds, bit + 2, err)) return 1;
    if (arm(reinterpret_cast<const void*>(suffix_intra_bwd_kernel<DK, DV>), lds_si, bit + 3, err)) return 1;
    hipLaunchKernelGGL((retention_bwd_fused_kernel<DK, DV, fpk::FB_FOLD>), grid, threads, lds, st, a);
    if (launched(err)) return 1;
    // what stays inside the suffixes, after the part of dq_s that comes from the carried state is written
    const long long pairs = (long long)a.B * (a.T / a.block + 1) * a.H;
    const long long wgs = 8LL * fpk_compute_units();
    hipLaunchKernelGGL((suffix_intra_bwd_kernel<DK, DV>), dim3((unsigned)(pairs < wgs ? pairs : wgs)), dim3(fpk::SI_THREADS),
                       lds_si, st, a);
    return launched(err);
  }
  if (a.block > 0) {
    constexpr int lds = fpk::fb_lds_bytes(DK, DV, fpk::FB_STOPS);
    if (arm(reinterpret_cast<const void*>(retention_bwd_fused_kernel<DK, DV, fpk::FB_STOPS>), lds, bit + 1, err)) return 1;
    hipLaunchKernelGGL((retention_bwd_fused_kernel<DK, DV, fpk::FB_STOPS>), grid, threads, lds, st, a);
  } else {
    constexpr int lds = fpk::fb_lds_bytes(DK, DV, fpk::FB_PLAIN);
    if (arm(reinterpret_cast<const void*>(retention_bwd_fused_kernel<DK, DV, fpk::FB_PLAIN>), lds, bit, err)) return 1;
    hipLaunchKernelGGL((retention_bwd_fused_kernel<DK, DV, fpk::FB_PLAIN>), grid, threads, lds, st, a);
  }
  return launched(err);
}

}  // namespace

int fpk_launch_bwd_fused(const fpk::FusedBwdArgs& args, void* stream, const char** err) {
  fpk::FusedBwdArgs a = args;
  a.fold = a.block > 0 && a.Ls <= fpk::FB_SFX_ROWS;
  if (const char* why = fpk::check_fused_bwd(a)) {
    *err = why;
    return 1;
  }
  a.pace = nullptr;
  if (fpk::fused_bwd_paces(a, fpk_compute_units())) {
    a.pace = pace_words_here();
    a.pace_base = g_pace_launch.fetch_add(1, std::memory_order_relaxed) << 16;
  }
  const hipStream_t st = static_cast<hipStream_t>(stream);
  if (a.dk_dim == 128 && a.dv_dim == 128) return launch_bwd_fused<128, 128>(a, 0, st, err);
  if (a.dk_dim == 64 && a.dv_dim == 128) return launch_bwd_fused<64, 128>(a, 1, st, err);
  if (a.dk_dim == 128 && a.dv_dim == 64) return launch_bwd_fused<128, 64>(a, 2, st, err);
  return launch_bwd_fused<64, 64>(a, 3, st, err);
}

namespace {

template <int DK, int DV>
int launch_short_bwd(const fpk::FusedBwdArgs& a, int slot, hipStream_t st, const char** err) {
  constexpr int lds = fpk::ss_lds_bytes(DK, DV);
  if (arm(reinterpret_cast<const void*>(short_seq_bwd_kernel<DK, DV>), lds, 64 + 20 + slot, err)) return 1;
  const long long pairs = (long long)a.B * a.H, wgs = fpk_compute_units();   // one workgroup per unit: its LDS fills it
  hipLaunchKernelGGL((short_seq_bwd_kernel<DK, DV>), dim3((unsigned)(pairs < wgs ? pairs : wgs)), dim3(fpk::FB_THREADS), lds, st, a);
  return launched(err);
}

template <int DK, int DV>
int launch_short_fwd(const fpk::ShortFwdArgs& a, int slot, hipStream_t st, const char** err) {
  constexpr int lds = fpk::ss_fwd_lds_bytes(DK, DV);
  if (arm(reinterpret_cast<const void*>(short_seq_fwd_kernel<DK, DV>), lds, 64 + 24 + slot, err)) return 1;
  const long long pairs = (long long)a.B * a.H, wgs = fpk_compute_units();   // one workgroup per unit, as in the backward
  hipLaunchKernelGGL((short_seq_fwd_kernel<DK, DV>), dim3((unsigned)(pairs < wgs ? pairs : wgs)), dim3(fpk::FB_THREADS), lds, st, a);
  return launched(err);
}

}  // namespace

int fpk_launch_short_fwd(const fpk::ShortFwdArgs& a, void* stream, const char** err) {
  if (const char* why = fpk::check_short_seq_fwd(a)) {
    *err = why;
    return 1;
  }
  const hipStream_t st = static_cast<hipStream_t>(stream);
  if (a.dk_dim == 128 && a.dv_dim == 128) return launch_short_fwd<128, 128>(a, 0, st, err);
  if (a.dk_dim == 64 && a.dv_dim == 128) return launch_short_fwd<64, 128>(a, 1, st, err);
  if (a.dk_dim == 128 && a.dv_dim == 64) return launch_short_fwd<128, 64>(a, 2, st, err);
  return launch_short_fwd<64, 64>(a, 3, st, err);
}

int fpk_launch_short_bwd(const fpk::FusedBwdArgs& a, void* stream, const char** err) {
  if (const char* why = fpk::check_short_seq_bwd(a)) {
    *err = why;
    return 1;
  }
  const hipStream_t st = static_cast<hipStream_t>(stream);
  if (a.dk_dim == 128 && a.dv_dim == 128) return launch_short_bwd<128, 128>(a, 0, st, err);
  if (a.dk_dim == 64 && a.dv_dim == 128) return launch_short_bwd<64, 128>(a, 1, st, err);
  if (a.dk_dim == 128 && a.dv_dim == 64) return launch_short_bwd<128, 64>(a, 2, st, err);
  return launch_short_bwd<64, 64>(a, 3, st, err);
}

int fpk_launch_contrib(const fpk::ContribArgs& a, void* stream, const char** err) {
  if (const char* why = fpk::check_contrib(a)) {
    *err = why;
    return 1;
  }
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) {
    *err = "hipGetDevice failed";
    return 1;
  }
  const void* const kernel = a.reverse ? reinterpret_cast<const void*>(segment_contrib_kernel<true>)
                                       : reinterpret_cast<const void*>(segment_contrib_kernel<false>);
  const uint64_t bit = 1ull << (a.reverse ? 60 : 61);
  const bool tracked = dev >= 0 && dev < kMaxDevices;
  if (!tracked || !(g_armed[dev][0].load(std::memory_order_acquire) & bit)) {
    if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, fpk::sc_lds_bytes()) != hipSuccess) {
      (void)hipGetLastError();
      *err = "hipFuncSetAttribute(MaxDynamicSharedMemorySize) failed";
      return 1;
    }
    if (tracked) g_armed[dev][0].fetch_or(bit, std::memory_order_release);
  }
  const dim3 grid((unsigned)(a.B * a.H * (a.dB / fpk::FB_D))), threads(fpk::FB_THREADS);
  if (a.reverse)
    hipLaunchKernelGGL(segment_contrib_kernel<true>, grid, threads, fpk::sc_lds_bytes(), static_cast<hipStream_t>(stream), a);
  else
    hipLaunchKernelGGL(segment_contrib_kernel<false>, grid, threads, fpk::sc_lds_bytes(), static_cast<hipStream_t>(stream), a);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    *err = hipGetErrorString(e);
    return 1;
  }
  return 0;
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
      a.dv > fpk::DECODE_THREADS || !a.q || !a.k || !a.v || !a.s_out || !a.o) {
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

int fpk_launch_rotary(const fpk::RotaryArgs& args, void* stream, const char** err) {
  fpk::RotaryArgs a = args;
  long long blocks = 0;
  if (const char* why = fpk::plan_rotary(a, blocks)) {
    *err = why;
    return 1;
  }
  hipLaunchKernelGGL(rotary_qk_kernel, dim3((unsigned)blocks), dim3(fpk::LAYER_THREADS), 0,
                     static_cast<hipStream_t>(stream), a);
  return launched(err);
}

int fpk_launch_gated_norm(const fpk::GatedNormArgs& a, void* stream, const char** err) {
  long long blocks = 0;
  if (const char* why = fpk::plan_gated_norm(a, blocks)) {
    *err = why;
    return 1;
  }
  if (a.out)
    hipLaunchKernelGGL(gated_norm_fwd_kernel, dim3((unsigned)blocks), dim3(fpk::LAYER_THREADS), 0,
                       static_cast<hipStream_t>(stream), a);
  else
    hipLaunchKernelGGL(gated_norm_bwd_kernel, dim3((unsigned)blocks), dim3(fpk::LAYER_THREADS), 0,
                       static_cast<hipStream_t>(stream), a);
  return launched(err);
}
