// Error reporting, version and the shape-based dispatcher of libxla_amd_qmm.so.
#include <stdarg.h>
#include <stdio.h>

#include "qmm_common.h"
#include "qmm_skinny.h"

static thread_local char g_err[512] = "";

int qmm_fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int qmm_check_hip(hipError_t e, const char* what) {
  if (e == hipSuccess) return XLA_AMD_QMM_OK;
  return qmm_fail(XLA_AMD_QMM_EHIP, "%s: %s", what, hipGetErrorString(e));
}

int qmm_set_max_lds(const void* kernel, int bytes, std::atomic<uint64_t>& done, const char* what) {
  int dev = 0;
  int rc = qmm_check_hip(hipGetDevice(&dev), what);
  if (rc != XLA_AMD_QMM_OK) return rc;
  const uint64_t bit = dev >= 0 && dev < 64 ? (1ull << dev) : 0;
  if (bit && (done.load(std::memory_order_acquire) & bit)) return XLA_AMD_QMM_OK;
  rc = qmm_check_hip(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes), what);
  if (rc == XLA_AMD_QMM_OK && bit) done.fetch_or(bit, std::memory_order_release);
  return rc;
}

extern "C" int xla_amd_qmm_abi_version(void) { return XLA_AMD_QMM_ABI_VERSION; }

extern "C" const char* xla_amd_qmm_last_error(void) { return g_err; }

extern "C" size_t xla_amd_qmm_packed_bytes(int64_t N, int64_t K, int bits) {
  if (N <= 0 || K <= 0) return 0;
  if (bits == 8) return (size_t)N * (size_t)K;
  if (bits == 4 && K % 8 == 0) return (size_t)N * (size_t)K / 2;
  return 0;
}

// Channels per group of the tiled copy.  A wave of the streaming kernel owns one group over all of K
// (or, with KW waves splitting K, a KW-th of it), and a launch should fill the chip's 256 compute units
// x 4 waves in whole rounds: 14336 channels in groups of 16 are 896 waves = 224 workgroups, 32 compute
// units idle for the whole launch; in groups of 14 they are 1024 waves on all 256.  So per-channel int8
// weights are tiled in groups of 16, 14, 12 or 10 channels, whichever fills the last round best (the
// wider group unless a narrower one gains 4 % or more); blockwise and int4 weights keep 16.
extern "C" int xla_amd_qmm_tile_group(int64_t N, int64_t K, int64_t C, int bits) {
  if (N <= 0 || K <= 0) return 0;
  if (C <= 0) C = K;
  if (bits != 8 || C != K || N < 4096) return 16;
  auto fill = [&](int64_t g) -> double {
    const int64_t groups = (N + g - 1) / g;
    const double used = (double)N / (double)(groups * g);  // channels past N in the last group
    int64_t kw = 1;
    if (groups * 2 <= 1024) kw = 2;
    if (groups * 4 <= 1024) kw = 4;
    const int64_t waves = groups * kw;
    if (waves <= 1024) return used * (double)waves / 1024.0;
    // more than one round of four-wave workgroups: eight computing waves per workgroup, 2048 per round
    const int64_t rounds = (groups + 2047) / 2048;
    return used * (double)groups / (double)(rounds * 2048);
  };
  int best = 16;
  double best_fill = fill(16);
  for (int g : {14, 12, 10}) {
    const double f = fill(g);
    if (f >= best_fill + 0.04) { best = g; best_fill = f; }
  }
  return best;
}

extern "C" size_t xla_amd_qmm_tiled_bytes(int64_t N, int64_t K, int64_t C, int bits) {
  if (N <= 0 || K <= 0 || K % 128 != 0 || (bits != 4 && bits != 8)) return 0;
  const int64_t g = xla_amd_qmm_tile_group(N, K, C, bits);
  const size_t rows = (size_t)((N + g - 1) / g) * (size_t)g;
  return bits == 8 ? rows * (size_t)K : rows * (size_t)K / 2;
}

// K slices over workgroups for the weight-streaming kernel.  A workgroup of that kernel owns 64
// (or 32, 16) output channels over all of K and copies every column of x it multiplies; with few
// channels and a long K the workgroups together copy several times the weight's bytes of x (out
// of L2), and there are too few of them for the memory system.  Slicing K gives each workgroup
// 64 channels of one slice: as many workgroups, a fraction of the x traffic.  The slices' sums are
// added by a second kernel, so this needs a workspace and is reached through
// xla_amd_qmm_weight_only_gemm.
int qmm_skinny_k_slices(int64_t M, int64_t N, int64_t K, int64_t C, int bits, int* k_per_slice) {
  *k_per_slice = (int)K;
  int64_t ks = bits == 4 ? 1024 : 512;  // columns per step of the streaming kernel
  if (C > 0 && C < K) {
    // blockwise weights: a slice is whole steps and whole quantization blocks
    if (C % 128 != 0 || K % C != 0 || N % 4 != 0) return 1;
    if (C > ks) { if (C % ks != 0) return 1; ks = C; }
    else if (ks % C != 0) return 1;
  }
  if (M > 32 || K % ks != 0) return 1;
  // (measured with cold weights at M = 32: 4096 x 14336 25.5 -> 17.8 us; with fewer than 8 rows the second kernel
  // costs more than the copies saved, and so it does with K = 4096 unless the output is narrow and x two tiles
  // high: 1024 x 4096 at M = 32 8.6 -> 7.5 us, 2048 x 4096 8.8 -> 8.4, but 4096 x 4096 9.4 -> 9.9)
  const int64_t g_ch = xla_amd_qmm_tile_group(N, K, C, bits);
  const int64_t cols = ((N + g_ch - 1) / g_ch + 3) / 4;  // workgroups of four channel groups
  if (M < 8 || K < 4096) return 1;
  if (K < 8192 && !(M > 16 && cols <= 16)) return 1;
  if (cols >= 128) return 1;  // enough workgroups of four channel groups already
  const int64_t steps = K / ks;
  int64_t slices = 256 / cols;
  if (slices > steps / 2) slices = steps / 2;  // at least two steps per slice
  if (slices < 2) return 1;
  const int64_t per = (steps + slices - 1) / slices;
  slices = (steps + per - 1) / per;
  if (slices < 2) return 1;
  *k_per_slice = (int)(per * ks);
  return (int)slices;
}

// The two regimes of a quantized linear layer on MI355X:
//  * few rows of x (decode): every weight byte is used M times, far below the
//    ~630 int8 ops/byte (or ~310 bf16 flops/byte) the chip can do per HBM
//    byte, so the weight is streamed exactly once by the skinny kernel;
//  * many rows with int8 activations (prefill): LDS-tiled int8 MFMA GEMM.
// Shapes neither fast kernel accepts run the one-thread-per-output kernels.
extern "C" int xla_amd_qmm_dispatch(int64_t M, int64_t N, int64_t K, int64_t C, int bits,
                                    int x_dt, int quantize_activation) {
  if (quantize_activation) {
    if (K % 64 == 0 && M * N >= 64 * 64) return XLA_AMD_KERNEL_W8A8_MFMA;
    return XLA_AMD_KERNEL_W8A8_GENERIC;
  }
  if (C <= 0) C = K;
  // many rows of 2-byte x against per-channel int8 weights: the tiled GEMM reads the weight once
  // per 128 rows, the streaming kernel once per 32
  if (C == K && bits == 8 && K % 128 == 0 && x_dt != XLA_AMD_DT_F32 && M > 32) return XLA_AMD_KERNEL_WEIGHT_ONLY_GEMM;
  // many rows of f32 x: the same GEMM over x split into three bf16 parts (xla_amd_qmm_weight_only_gemm_f32), three
  // times the arithmetic, where the streaming kernel makes a pass over the weight for every 16 rows (from 128 rows
  // on: 4096 x 4096 takes 103 us either way there, 14336 x 4096 118 against 250 us)
  if (C == K && bits == 8 && K % 128 == 0 && 3 * K <= (1 << 23) && x_dt == XLA_AMD_DT_F32 && M >= 128) return XLA_AMD_KERNEL_WEIGHT_ONLY_GEMM;
  // few rows against few channels and a long K: the streaming kernel over K slices, behind the GEMM's entry point
  if ((bits == 8 || bits == 4) && x_dt != XLA_AMD_DT_F32 && K % C == 0) {
    int per;
    if (qmm_skinny_k_slices(M, N, K, C, bits, &per) > 1) return XLA_AMD_KERNEL_WEIGHT_ONLY_GEMM;
  }
  // many rows against blockwise or int4 weights: the tiled GEMM with per-block rounding points (the caller
  // must also have scale / zero point / result of x's dtype; else it takes the streaming kernel, pass by pass).
  // Up to 64 rows two passes of the streaming kernel are as fast or faster (a 64 x 128 tile per workgroup and
  // no K split: 4096 channels are 32 workgroups).
  if ((C != K || bits == 4) && (bits == 8 || bits == 4) && K % 128 == 0 && C % 128 == 0 && N % 4 == 0 &&
      x_dt != XLA_AMD_DT_F32 && M > 64)
    return XLA_AMD_KERNEL_WEIGHT_ONLY_GEMM;
  if (K % 128 == 0 && C % 128 == 0 && (bits == 8 || bits == 4) && M >= 1 &&
      (C == K || (N % 4 == 0 && (K / C) * N >= 8)))  // blockwise: vector loads of 4 channels' scales
    return XLA_AMD_KERNEL_SKINNY_MFMA;
  return XLA_AMD_KERNEL_GENERIC;
}
