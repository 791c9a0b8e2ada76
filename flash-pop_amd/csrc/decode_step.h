// Recurrent decode step (see DecodeArgs in pass_args.h): one workgroup per (batch, head).
// A thread owns 8 adjacent columns of S (16 bytes) in every (256 / (dv / 8))-th row: it updates
// them, stores them and accumulates its part of o = q S'; the row groups' partial sums meet in LDS.
// The whole state is read once and written once, which is all the HBM traffic the step has.
#pragma once
#include "pass_args.h"
#include "lds_access.h"

namespace fpk {

FP_DEVICE void decode_step(const DecodeArgs& p, char* lds) {
  float* part = reinterpret_cast<float*>(lds);            // [row groups][dv]
  const int tid = fprt::thread_index();
  const int bh = fprt::block_index();
  const int h = bh % p.H;
  const int tpr = p.dv / 8;                                 // threads per row
  const int ngroups = DECODE_THREADS / tpr;                 // rows in flight
  const int cg = tid % tpr, rg = tid / tpr;
  const float g = p.gamma[h];
  const uint16_t* q = p.q + (size_t)bh * p.dk;
  const uint16_t* k = p.k + (size_t)bh * p.dk;
  const size_t mat = (size_t)bh * p.dk * p.dv;

  const u32x4 vv = ld128(p.v + (size_t)bh * p.dv + 8 * cg);
  float v[8], acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    v[e] = bf16_elem(vv, e);
    acc[e] = 0.f;
  }
  // (dv = 192: 24 threads per row, 10 rows in flight, the last 16 threads idle)
  for (int row = rg < ngroups ? rg : p.dk; row < p.dk; row += ngroups) {
    const float kr = p.scale * bf16_bits_to_float(reinterpret_cast<const u16_m*>(k)[row]);
    const float qr = bf16_bits_to_float(reinterpret_cast<const u16_m*>(q)[row]);
    const size_t at = mat + (size_t)row * p.dv + 8 * cg;
    float s[8];
    if (p.s_in) {
      const u32x4 sv = ld128(p.s_in + at);
#pragma unroll
      for (int e = 0; e < 8; ++e) s[e] = g * bf16_elem(sv, e) + kr * v[e];
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) s[e] = kr * v[e];
    }
    u32x4 out;
#pragma unroll
    for (int e = 0; e < 4; ++e) out[e] = fprt::pack_bf16x2(s[2 * e], s[2 * e + 1]);
    st128(p.s_out + at, out);
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] += qr * s[e];
  }
  if (rg < ngroups) {
#pragma unroll
    for (int e = 0; e < 8; ++e) part[rg * p.dv + 8 * cg + e] = acc[e];
  }
  fprt::block_sync();
  if (tid < p.dv) {
    float sum = 0.f;
    for (int r = 0; r < ngroups; ++r) sum += part[r * p.dv + tid];
    reinterpret_cast<u16_m*>(p.o)[(size_t)bh * p.dv + tid] = float_to_bf16_bits(sum);
  }
}

}  // namespace fpk
