// gfx950 entry points of the pass kernel and the launcher the C-ABI layer calls.
#include "device_rt.h"
#include "retention_pass.h"

namespace {

template <int DA>
__global__ __launch_bounds__(fpk::NTHREADS) void retention_pass_kernel(const fpk::PassArgs args) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  fpk::retention_pass<DA>(args, lds);
}

template <int DA>
int launch(const fpk::PassArgs& a, hipStream_t stream, const char** err) {
  // LDS above 64 KB has to be opted into, once per device and kernel.
  static thread_local int armed_device = -1;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) {
    *err = "hipGetDevice failed";
    return 1;
  }
  constexpr int lds = fpk::lds_bytes(DA);
  if (armed_device != dev) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&retention_pass_kernel<DA>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess) {
      (void)hipGetLastError();
      *err = "hipFuncSetAttribute(MaxDynamicSharedMemorySize) failed";
      return 1;
    }
    armed_device = dev;
  }
  const int nwg = a.B * a.H * (a.dB / fpk::BV);
  hipLaunchKernelGGL(retention_pass_kernel<DA>, dim3(nwg), dim3(fpk::NTHREADS), lds, stream, a);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    *err = hipGetErrorString(e);
    return 1;
  }
  return 0;
}

}  // namespace

int fpk_launch_pass(const fpk::PassArgs& a, void* stream, const char** err) {
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (a.dA) {
    case 64: return launch<64>(a, s, err);
    case 128: return launch<128>(a, s, err);
    case 256: return launch<256>(a, s, err);
    default: *err = "unsupported contraction width (dA must be 64, 128 or 256)"; return 1;
  }
}
