// Small helpers shared by the kernel bodies: aliasing-safe 8- and 16-byte accesses, bf16 <-> fp32,
// and the row of a 32x32 MFMA accumulator that an element belongs to.  Written against the fprt
// primitives only, so the same code also runs under the CPU thread harness used by the tests.
#pragma once
#include "pass_args.h"

namespace fpk {

using fprt::f32x16;
using fprt::u32x2;
using fprt::u32x4;

typedef u32x4 __attribute__((may_alias, aligned(16))) u32x4_m;
typedef u32x2 __attribute__((may_alias, aligned(8))) u32x2_m;
typedef uint16_t __attribute__((may_alias)) u16_m;

FP_DEVICE u32x4 ld128(const uint16_t* p) { return *reinterpret_cast<const u32x4_m*>(p); }
FP_DEVICE u32x2 ld64(const uint16_t* p) { return *reinterpret_cast<const u32x2_m*>(p); }
FP_DEVICE void st128(uint16_t* p, u32x4 v) { *reinterpret_cast<u32x4_m*>(p) = v; }
FP_DEVICE void st64(uint16_t* p, u32x2 v) { *reinterpret_cast<u32x2_m*>(p) = v; }

FP_DEVICE float bf16_bits_to_float(uint32_t bits16) { return __builtin_bit_cast(float, bits16 << 16); }
// element e (0..7) of eight packed bf16
FP_DEVICE float bf16_elem(u32x4 v, int e) {
  uint32_t d = v[e >> 1];
  return __builtin_bit_cast(float, (e & 1) ? (d & 0xffff0000u) : (d << 16));
}
FP_DEVICE uint16_t float_to_bf16_bits(float x) { return (uint16_t)(fprt::pack_bf16x2(x, 0.f) & 0xffffu); }

// row of the 32x32 MFMA accumulator held in element r by a lane of half-wave g
FP_DEVICE int acc_row(int r, int g) { return 8 * (r >> 2) + 4 * g + (r & 3); }

}  // namespace fpk
