// Streaming calibration kernels: a plain read (sum) and a plain copy of a known number of bytes.
// They give the achievable HBM rate for a launch of a given size on this device and the scale of
// the profiler's FETCH_SIZE / WRITE_SIZE counters (known bytes moved per dispatch).
#include "common.h"
#include "../../include/adamah_hip.h"
#include <algorithm>

namespace adamah {

__global__ void __launch_bounds__(256)
k_probe_read(const uint4* __restrict__ src, uint64_t n_vec, uint32_t* __restrict__ sink) {
  uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x;
  const uint64_t stride = (uint64_t)gridDim.x * 256u;
  uint32_t acc = 0;
  for (; i + 3 * stride < n_vec; i += 4 * stride) {
    const uint4 a = src[i], b = src[i + stride], c = src[i + 2 * stride], d = src[i + 3 * stride];
    acc += (a.x ^ a.y ^ a.z ^ a.w) + (b.x ^ b.y ^ b.z ^ b.w) + (c.x ^ c.y ^ c.z ^ c.w) + (d.x ^ d.y ^ d.z ^ d.w);
  }
  for (; i < n_vec; i += stride) { const uint4 a = src[i]; acc += a.x ^ a.y ^ a.z ^ a.w; }
  if (acc == 0x9E3779B9u) sink[0] = acc;   // practically never true: keeps the loads alive
}

__global__ void __launch_bounds__(256)
k_probe_copy(const uint4* __restrict__ src, uint4* __restrict__ dst, uint64_t n_vec) {
  uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x;
  const uint64_t stride = (uint64_t)gridDim.x * 256u;
  for (; i < n_vec; i += stride) dst[i] = src[i];
}

}  // namespace adamah

using namespace adamah;

extern "C" {

// mode 0: read `bytes_per_launch` bytes per launch; mode 1: copy them (read + write).  Launches walk
// through a `pool_bytes` buffer so consecutive launches touch different memory.  Returns the
// average microseconds per launch over `launches` launches (HIP events on the library stream),
// or a negative error code.
float adamah_hip_stream_probe(uint64_t bytes_per_launch, uint64_t pool_bytes, uint32_t mode, uint32_t wg_per_cu,
                              uint32_t launches) { ADAMAH_API();
  if (!g.initialized || bytes_per_launch < 4096 || pool_bytes < bytes_per_launch || launches == 0 || wg_per_cu == 0)
    return (float)ADAMAH_ERR_INVALID;
  uint8_t *src = nullptr, *dst = nullptr;
  uint32_t* sink = nullptr;
  if (hipMalloc((void**)&src, pool_bytes) != hipSuccess) return (float)ADAMAH_ERR_MEMORY;
  if (hipMalloc((void**)&sink, 256) != hipSuccess) { hipFree(src); return (float)ADAMAH_ERR_MEMORY; }
  if (mode == 1 && hipMalloc((void**)&dst, pool_bytes) != hipSuccess) { hipFree(src); hipFree(sink); return (float)ADAMAH_ERR_MEMORY; }
  hipMemsetAsync(src, 0x5A, pool_bytes, g.stream);
  const uint64_t n_vec = bytes_per_launch / 16, slots = pool_bytes / bytes_per_launch;
  const uint32_t grid = (uint32_t)std::min<uint64_t>((uint64_t)g.n_cu * wg_per_cu, (n_vec + 255) / 256);
  float ms = -1.0f;
  for (int pass = 0; pass < 2; pass++) {           // pass 0 warms up, pass 1 is timed
    if (pass == 1) hipEventRecord(g.timer_ev[0], g.stream);
    for (uint32_t l = 0; l < launches; l++) {
      const uint64_t off = (l % slots) * bytes_per_launch;
      if (mode == 0) k_probe_read<<<grid, 256, 0, g.stream>>>((const uint4*)(src + off), n_vec, sink);
      else k_probe_copy<<<grid, 256, 0, g.stream>>>((const uint4*)(src + off), (uint4*)(dst + off), n_vec);
    }
    if (pass == 1) {
      hipEventRecord(g.timer_ev[1], g.stream);
      hipEventSynchronize(g.timer_ev[1]);
      hipEventElapsedTime(&ms, g.timer_ev[0], g.timer_ev[1]);
    }
  }
  hipStreamSynchronize(g.stream);
  hipFree(src); hipFree(sink);
  if (dst) hipFree(dst);
  if (check_launch() != ADAMAH_OK || ms < 0) return (float)ADAMAH_ERR_BACKEND;
  return ms * 1000.0f / (float)launches;
}

}  // extern "C"
