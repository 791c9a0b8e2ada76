// Measurement aid: the global-memory access pattern of one retention pass with nothing else.
// Same grid and workgroup placement as the pass kernel at dA = 128 (one workgroup per (batch,
// head, 64-column tile), 512 threads); per 64-token item waves 0-3 read the X rows of their head
// (256 bytes per row) and the Z tile (128 bytes per row) and write the Y tile, waves 4-7 read the
// W rows; the loads of the next item are in flight while the current one is consumed.  No LDS, no
// barriers, no arithmetic: how long this takes is how fast the device streams these tensors in
// this layout, which is the floor for a pass that has to touch the same bytes.
// Functionally it copies Z to Y (X and W only feed a checksum that is never stored).
#pragma once
#include "pass_args.h"
#include "lds_access.h"

namespace fpk {

FP_DEVICE void stream_probe(const StreamProbeArgs& p, int wg) {
  const int ntile = p.dB / BV;
  const int tile = wg % ntile, h = (wg / ntile) % p.H, b = (wg / ntile) / p.H;
  const int tid = fprt::thread_index();
  const size_t rowA = (size_t)p.H * p.dA, rowB = (size_t)p.H * p.dB;      // elements
  const uint16_t* X = p.X + (size_t)b * p.T * rowA + (size_t)h * p.dA;
  const uint16_t* W = p.W + (size_t)b * p.T * rowA + (size_t)h * p.dA;
  const uint16_t* Z = p.Z + (size_t)b * p.T * rowB + (size_t)h * p.dB + tile * BV;
  uint16_t* Y = p.Y + (size_t)b * p.T * rowB + (size_t)h * p.dB + tile * BV;
  const int items = p.T / CH;
  u32x4 sum = {0, 0, 0, 0};
  if (tid < 256) {
    // X: 4 pieces of 16 bytes per thread and item; Z / Y: one 32-byte piece of a row per thread
    const int zrow = tid >> 2, zcol = (tid & 3) * 16;
    u32x4 x[4], z0, z1;
    auto issue = [&](int it) {
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int q = tid + 256 * u;
        x[u] = ld128(X + (size_t)(it * CH + q / 16) * rowA + (q % 16) * 8);
      }
      z0 = ld128(Z + (size_t)(it * CH + zrow) * rowB + zcol);
      z1 = ld128(Z + (size_t)(it * CH + zrow) * rowB + zcol + 8);
    };
    issue(0);
    for (int it = 0; it < items; ++it) {
      const u32x4 y0 = z0, y1 = z1;
#pragma unroll
      for (int u = 0; u < 4; ++u) sum ^= x[u];
      if (it + 1 < items) issue(it + 1);
      st128(Y + (size_t)(it * CH + zrow) * rowB + zcol, y0);
      st128(Y + (size_t)(it * CH + zrow) * rowB + zcol + 8, y1);
    }
  } else {
    const int lt = tid - 256;
    u32x4 w[4];
    auto issue = [&](int it) {
#pragma unroll
      for (int r = 0; r < 4; ++r)
        w[r] = ld128(W + (size_t)(it * CH + 4 * ((lt & 63) >> 2) + r) * rowA + 32 * (lt >> 6) + 8 * (lt & 3));
    };
    issue(0);
    for (int it = 0; it < items; ++it) {
#pragma unroll
      for (int r = 0; r < 4; ++r) sum ^= w[r];
      if (it + 1 < items) issue(it + 1);
    }
  }
  // keeps the X and W loads alive without ever storing: no bf16 pattern repeats this word four times
  if (sum[0] == 0x7fc17fc1u && sum[1] == 0x7fc27fc2u && sum[2] == 0x7fc37fc3u && sum[3] == 0x7fc47fc4u) Y[0] = 0;
}

inline const char* plan_stream_probe(const StreamProbeArgs& a, long long& blocks) {
  if (!a.X || !a.W || !a.Z || !a.Y) return "stream probe: null pointer";
  if (a.B < 1 || a.H < 1 || a.T < CH || a.T % CH != 0 || a.dA != 128 || a.dB < BV || a.dB % BV != 0)
    return "stream probe: T a multiple of 64, dA = 128 and dB a multiple of 64 expected";
  blocks = (long long)a.B * a.H * (a.dB / BV);
  return blocks > 0x7fffffffLL ? "stream probe: too many workgroups" : nullptr;
}

}  // namespace fpk
