// Device primitives the pass kernel is written against (gfx950 / CDNA4).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define FP_DEVICE __device__ __forceinline__

namespace fprt {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));

FP_DEVICE int thread_index() { return threadIdx.x; }
FP_DEVICE int block_index() { return blockIdx.x; }
FP_DEVICE int grid_size() { return gridDim.x; }
FP_DEVICE void block_sync() { __syncthreads(); }

// D = A(32x16) * B(16x32) + C, bf16 inputs, fp32 accumulate (v_mfma_f32_32x32x16_bf16).
// Lane l supplies A[l%32][8*(l/32) + e] and B[8*(l/32) + e][l%32], e = 0..7, and holds
// D[8*(r/4) + 4*(l/32) + r%4][l%32] in element r.
FP_DEVICE f32x16 mfma_32x32x16_bf16(u32x4 a, u32x4 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0,
                                                 0, 0);
}

// Two floats -> two bf16 (round to nearest even), `lo` in bits 0..15 (v_cvt_pk_bf16_f32).
FP_DEVICE uint32_t pack_bf16x2(float lo, float hi) {
  f32x2_t f = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2_t));
}

// 2^x for x <= 0 (v_exp_f32, ~1 ulp; results below the normal range flush to zero).
FP_DEVICE float exp2_approx(float x) { return __builtin_amdgcn_exp2f(x); }
// full-precision elementary functions for the elementwise kernels
FP_DEVICE void sincos_f32(float x, float& s, float& c) { sincosf(x, &s, &c); }
// 1 / (1 + e^-x) from the hardware's 2^x and reciprocal (v_exp_f32, v_rcp_f32: ~1 ulp each; 0 and 1
// at the far ends, where e^-x overflows or vanishes)
FP_DEVICE float sigmoid_f32(float x) { return __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(-1.44269504f * x)); }
FP_DEVICE float rsqrt_f32(float x) { return 1.0f / sqrtf(x); }
// value held by lane (this lane ^ mask) of the wave; every lane of the wave has to call it
FP_DEVICE float lane_xor(float v, int mask) { return __shfl_xor(v, mask, 64); }

// Transposing LDS read (ds_read_b64_tr_b16).  Every lane passes the address of four consecutive
// 16-bit values; within each group of 16 lanes, lane i receives element i % 4 of the values read
// by lanes 4 e + i / 4, e = 0..3.  With lane 4 r + q of a group pointing at columns 4 q .. 4 q + 3 of
// row r of a row-major block of 4 rows x 16 columns, lane i gets column i of the four rows: an
// MFMA operand that runs along the rows of a row-major tile.
typedef short s16x4_t __attribute__((ext_vector_type(4)));
FP_DEVICE u32x2 lds_read_tr16_b64(const uint16_t* p) {
  return __builtin_bit_cast(
      u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)(p)));
}

// Orders LDS traffic between the lanes of one wave.  The hardware executes a wave's LDS
// instructions in order, so this only has to stop the compiler from reordering them.
FP_DEVICE void wave_sync() { __builtin_amdgcn_wave_barrier(); }

// Nothing may be moved across this point by the instruction scheduler.
FP_DEVICE void sched_fence() { __builtin_amdgcn_sched_barrier(0); }

// Bounds-checked view of global memory (raw buffer resource): loads beyond `nbytes` return
// zero and stores beyond it are dropped by the hardware, which is how ragged chunk tails
// are handled without branches.  Offsets are bytes from `base`, below 4 GiB.
struct BufView {
  __amdgpu_buffer_rsrc_t rsrc;
};
FP_DEVICE BufView make_buf(const void* base, uint32_t nbytes) {
  return BufView{__builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)nbytes, 0x00020000)};
}
FP_DEVICE u32x4 buf_load128(BufView b, uint32_t off) { return __builtin_amdgcn_raw_buffer_load_b128(b.rsrc, off, 0, 0); }
FP_DEVICE u32x2 buf_load64(BufView b, uint32_t off) { return __builtin_amdgcn_raw_buffer_load_b64(b.rsrc, off, 0, 0); }
FP_DEVICE void buf_store128(BufView b, uint32_t off, u32x4 v) { __builtin_amdgcn_raw_buffer_store_b128(v, b.rsrc, off, 0, 0); }
// the same with the non-temporal hint: data that nobody reads again soon need not stay in the caches
FP_DEVICE u32x4 buf_load128_nt(BufView b, uint32_t off) { return __builtin_amdgcn_raw_buffer_load_b128(b.rsrc, off, 0, 2); }
FP_DEVICE void buf_store128_nt(BufView b, uint32_t off, u32x4 v) { __builtin_amdgcn_raw_buffer_store_b128(v, b.rsrc, off, 0, 2); }
FP_DEVICE void buf_store64(BufView b, uint32_t off, u32x2 v) { __builtin_amdgcn_raw_buffer_store_b64(v, b.rsrc, off, 0, 0); }

// A word that another workgroup of the same launch polls (relaxed, device scope), and a short sleep between polls.
FP_DEVICE void pace_store(uint32_t* p, uint32_t v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
FP_DEVICE uint32_t pace_load(const uint32_t* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
FP_DEVICE void nap() { __builtin_amdgcn_s_sleep(8); }

}  // namespace fprt
