// Measurement hooks, not part of the C ABI (not declared in mdattn.h; bench.py binds them by name).
//
// mdattn_probe_dq_atomics: the f32 atomic-add traffic a single-pass backward would generate for dq.  Such a pass makes
// key rows the resident rows of a workgroup (8 waves x 32 keys) and streams the query tiles past them; every (query
// tile, key block) pair then yields a 32 x head_dim partial of dq that has to be added into global memory.  The probe
// issues exactly those atomics and nothing else: with `per_wave` every wave adds its own partial (no exchange inside
// the workgroup), without it the workgroup adds one partial per query tile, as if its eight waves had reduced theirs
// first (each wave adds an eighth).  The time of the launch is a lower bound of what the atomics would add to a
// backward pass that saved its two duplicate matrix products.
#include "mdattn_common.h"

namespace mdattn {
__global__ __launch_bounds__(512) void probe_dq_atomics_kernel(float* dq, int Sq, int D, int nkt, int per_wave) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int h = blockIdx.x / nkt;
  float* base = dq + (int64_t)h * Sq * D;
  const int tile_floats = 32 * D;
  const int nqt = Sq / 32;
  const int per_lane = per_wave ? tile_floats / 64 : tile_floats / 512;
  const int first = per_wave ? 0 : wave * per_lane;
  // the workgroups of one head start at different query tiles, as drifting workgroups of a real pass would
  int t = (int)(((int64_t)(blockIdx.x % nkt) * nqt) / nkt);
  for (int i = 0; i < nqt; ++i) {
    float* tile = base + (int64_t)t * tile_floats;
    for (int j = 0; j < per_lane; ++j) unsafeAtomicAdd(tile + (first + j) * 64 + lane, 1.0f);
    t = t + 1 == nqt ? 0 : t + 1;
  }
}
}  // namespace mdattn

extern "C" int mdattn_probe_dq_atomics(void* stream, float* dq, int H, int Sq, int Skv, int D, int per_wave) {
  if (!dq || H <= 0 || Sq < 32 || Skv < 256 || D <= 0 || D % 16) return MDATTN_E_BADARG;
  const int nkt = Skv / 256;
  MDATTN_LAUNCH(mdattn::probe_dq_atomics_kernel, dim3(H * nkt), dim3(512), 0, (hipStream_t)stream, dq, Sq / 32 * 32, D, nkt, per_wave);
  return mdattn::launch_status();
}
