// Diagnostic kernels, linked into the diagnostic library only (libxla_amd_qmm_timeline.so, see
// xla_amd/build.py); the operators never call them.
//
// xla_amd_qmm_diag_stream: a kernel that only reads `bytes` bytes, shaped like the weight-streaming
// kernel's memory side (workgroups of `waves` waves, every wave keeping `depth` 1 KB loads in flight over
// its own contiguous region, nontemporal), for measuring what the memory system gives a launch of that
// shape and size: the floor under the decode GEMV's time.
#include "qmm_common.h"

namespace {

template <int D>
__global__ void __launch_bounds__(1024) diag_stream_kernel(const char* __restrict__ p, int n, int* sink) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const size_t wave_id = (size_t)blockIdx.x * (blockDim.x >> 6) + wave;
  const char* base = p + wave_id * (size_t)n * 1024 + lane * 16;
  i32x4 r[D];
  i32x4 acc = {0, 0, 0, 0};
  qmm_static_for<D>([&](auto dc) {
    constexpr int d = dc;
    r[d] = __builtin_nontemporal_load((const i32x4*)(base + (size_t)min(d, n - 1) * 1024));
  });
  for (int i = 0; i < n; i += D) {
    qmm_static_for<D>([&](auto dc) {
      constexpr int d = dc;
      acc ^= r[d];
      r[d] = __builtin_nontemporal_load((const i32x4*)(base + (size_t)min(i + d + D, n - 1) * 1024));
    });
  }
  if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x12345678) sink[0] = 1;  // (keeps the loads alive)
}

}  // namespace

// Reads the first grid * waves * kb_per_wave KB of `buf` (the caller sizes it); depth in {4, 8, 16}.
extern "C" int xla_amd_qmm_diag_stream(const void* buf, int* sink, int grid, int waves, int depth, int kb_per_wave,
                                       void* stream) {
  if (!buf || !sink || grid <= 0 || waves <= 0 || waves > 16 || kb_per_wave <= 0)
    return qmm_fail(XLA_AMD_QMM_EINVAL, "diag_stream: bad arguments");
  hipStream_t s = (hipStream_t)stream;
  if (depth == 4) hipLaunchKernelGGL(diag_stream_kernel<4>, dim3(grid), dim3(waves * 64), 0, s, (const char*)buf, kb_per_wave, sink);
  else if (depth == 8) hipLaunchKernelGGL(diag_stream_kernel<8>, dim3(grid), dim3(waves * 64), 0, s, (const char*)buf, kb_per_wave, sink);
  else if (depth == 16) hipLaunchKernelGGL(diag_stream_kernel<16>, dim3(grid), dim3(waves * 64), 0, s, (const char*)buf, kb_per_wave, sink);
  else return qmm_fail(XLA_AMD_QMM_EINVAL, "diag_stream: depth must be 4, 8 or 16");
  return QMM_CHECK_LAUNCH("diag_stream launch");
}
