// Segment scan (see ScanArgs in pass_args.h): one thread carries SCAN_VEC elements of one
// (batch, head) state matrix through the S segments in fp32.
#pragma once
#include "pass_args.h"
#include "lds_access.h"

namespace fpk {

FP_DEVICE void segment_scan(const ScanArgs& p) {
  const int per_mat = p.M / SCAN_VEC;
  const long long item = (long long)fprt::block_index() * SCAN_THREADS + fprt::thread_index();
  if (item >= (long long)p.B * p.H * per_mat) return;
  const int piece = (int)(item % per_mat);
  const int h = (int)((item / per_mat) % p.H);
  const int b = (int)(item / ((long long)per_mat * p.H));
  const float gseg = fprt::exp2_approx((float)p.Tseg * p.log2g[h]);
  const size_t in_mat = (size_t)piece * SCAN_VEC;
  float r[SCAN_VEC];
  if (p.R0) {
    const u32x4 v = ld128(p.R0 + ((size_t)b * p.H + h) * p.M + in_mat);
#pragma unroll
    for (int e = 0; e < SCAN_VEC; ++e) r[e] = bf16_elem(v, e);
  } else {
#pragma unroll
    for (int e = 0; e < SCAN_VEC; ++e) r[e] = 0.f;
  }
  for (int i = 0; i < p.S; ++i) {
    const int s = p.reverse ? p.S - 1 - i : i;
    const size_t at = (((size_t)b * p.S + s) * p.H + h) * p.M + in_mat;
    u32x4 o;
#pragma unroll
    for (int e = 0; e < SCAN_VEC / 2; ++e) o[e] = fprt::pack_bf16x2(r[2 * e], r[2 * e + 1]);
    st128(p.init + at, o);
    const u32x4 u = ld128(p.U + at);
#pragma unroll
    for (int e = 0; e < SCAN_VEC; ++e) r[e] = gseg * r[e] + bf16_elem(u, e);
  }
  if (p.fin) {
    u32x4 o;
#pragma unroll
    for (int e = 0; e < SCAN_VEC / 2; ++e) o[e] = fprt::pack_bf16x2(r[2 * e], r[2 * e + 1]);
    st128(p.fin + ((size_t)b * p.H + h) * p.M + in_mat, o);
  }
}

}  // namespace fpk
