// CPU stand-in for the device primitives: one OS thread per GPU lane, pthread barriers for
// workgroup and wave synchronisation, MFMA evaluated from the documented lane layout.
// Test infrastructure only: lets the kernel body run under ASan / gdb and be compared with
// the oracle without a GPU.  Never part of the shipped library.
#pragma once
#include <pthread.h>
#include <stdint.h>

#include <cmath>
#include <cstring>

#define FP_DEVICE inline __attribute__((always_inline))

namespace fprt {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

struct WaveShared {
  uint16_t A[64][8];
  uint16_t Bm[64][8];
  float xchg[64];
  uint16_t tr[64][4];
  pthread_barrier_t bar;
};

struct LaneCtx {
  int tid, block, grid;
  WaveShared* wave;
  pthread_barrier_t* wg_bar;
};

extern thread_local LaneCtx g_lane;

FP_DEVICE int thread_index() { return g_lane.tid; }
FP_DEVICE int block_index() { return g_lane.block; }
FP_DEVICE int grid_size() { return g_lane.grid; }
FP_DEVICE void block_sync() { pthread_barrier_wait(g_lane.wg_bar); }

FP_DEVICE float bf16_to_f32(uint16_t b) {
  uint32_t u = (uint32_t)b << 16;
  float f;
  std::memcpy(&f, &u, 4);
  return f;
}

FP_DEVICE uint16_t f32_to_bf16_rne(float f) {
  uint32_t u;
  std::memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);   // NaN stays NaN
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

FP_DEVICE f32x16 mfma_32x32x16_bf16(u32x4 a, u32x4 b, f32x16 c) {
  WaveShared* w = g_lane.wave;
  const int lane = g_lane.tid & 63;
  std::memcpy(w->A[lane], &a, 16);
  std::memcpy(w->Bm[lane], &b, 16);
  pthread_barrier_wait(&w->bar);
  const int g = lane >> 5, n = lane & 31;
  for (int r = 0; r < 16; ++r) {
    const int m = 8 * (r >> 2) + 4 * g + (r & 3);
    float acc = c[r];
    for (int k = 0; k < 16; ++k) {
      acc += bf16_to_f32(w->A[m + 32 * (k >> 3)][k & 7]) * bf16_to_f32(w->Bm[n + 32 * (k >> 3)][k & 7]);
    }
    c[r] = acc;
  }
  pthread_barrier_wait(&w->bar);
  return c;
}

FP_DEVICE uint32_t pack_bf16x2(float lo, float hi) {
  return (uint32_t)f32_to_bf16_rne(lo) | ((uint32_t)f32_to_bf16_rne(hi) << 16);
}

FP_DEVICE float exp2_approx(float x) { return std::exp2(x); }
FP_DEVICE void sincos_f32(float x, float& s, float& c) { s = std::sin(x); c = std::cos(x); }
FP_DEVICE float sigmoid_f32(float x) { return 1.0f / (1.0f + std::exp(-x)); }
FP_DEVICE float rsqrt_f32(float x) { return 1.0f / std::sqrt(x); }

FP_DEVICE void sched_fence() {}
FP_DEVICE void pace_store(uint32_t* p, uint32_t v) { __atomic_store_n(p, v, __ATOMIC_RELAXED); }
FP_DEVICE uint32_t pace_load(const uint32_t* p) { return __atomic_load_n(p, __ATOMIC_RELAXED); }
FP_DEVICE void nap() {}
// lanes are independent OS threads here, so lane-to-lane exchange through LDS needs a real barrier
FP_DEVICE void wave_sync() { pthread_barrier_wait(&g_lane.wave->bar); }
FP_DEVICE float lane_xor(float v, int mask) {
  const int lane = g_lane.tid & 63;
  g_lane.wave->xchg[lane] = v;
  wave_sync();
  const float r = g_lane.wave->xchg[lane ^ mask];
  wave_sync();
  return r;
}

// ds_read_b64_tr_b16: within each group of 16 lanes, lane i receives element i % 4 of the four
// values read by lanes 4 e + i / 4, e = 0..3
FP_DEVICE u32x2 lds_read_tr16_b64(const uint16_t* p) {
  WaveShared* w = g_lane.wave;
  const int lane = g_lane.tid & 63;
  std::memcpy(w->tr[lane], p, 8);
  wave_sync();
  const int grp = lane & ~15, i = lane & 15;
  uint16_t out[4];
  for (int e = 0; e < 4; ++e) out[e] = w->tr[grp + 4 * e + i / 4][i % 4];
  wave_sync();
  u32x2 v;
  std::memcpy(&v, out, 8);
  return v;
}


struct BufView {
  const char* base;
  uint32_t nbytes;
};
FP_DEVICE BufView make_buf(const void* base, uint32_t nbytes) { return BufView{static_cast<const char*>(base), nbytes}; }
FP_DEVICE u32x4 buf_load128(BufView b, uint32_t off) {
  u32x4 v = {0u, 0u, 0u, 0u};
  if ((uint64_t)off + 16 <= b.nbytes) std::memcpy(&v, b.base + off, 16);
  return v;
}
FP_DEVICE u32x2 buf_load64(BufView b, uint32_t off) {
  u32x2 v = {0u, 0u};
  if ((uint64_t)off + 8 <= b.nbytes) std::memcpy(&v, b.base + off, 8);
  return v;
}
FP_DEVICE void buf_store128(BufView b, uint32_t off, u32x4 v) {
  if ((uint64_t)off + 16 <= b.nbytes) std::memcpy(const_cast<char*>(b.base) + off, &v, 16);
}
FP_DEVICE void buf_store64(BufView b, uint32_t off, u32x2 v) {
  if ((uint64_t)off + 8 <= b.nbytes) std::memcpy(const_cast<char*>(b.base) + off, &v, 8);
}
// the non-temporal forms differ only in how the device's caches treat the data
FP_DEVICE u32x4 buf_load128_nt(BufView b, uint32_t off) { return buf_load128(b, off); }
FP_DEVICE void buf_store128_nt(BufView b, uint32_t off, u32x4 v) { buf_store128(b, off, v); }

}  // namespace fprt
