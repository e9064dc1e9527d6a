// Arguments and launchers of the weight-only tiled GEMM for blockwise and int4 weights
// (qmm_wo_gemm_bw.hip), called from the workspace entry point in qmm_wo_gemm.hip.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdint>

struct WoBwArgs {
  const void* x;      // [M, K], bf16 or f16
  const uint8_t* w;   // tiled weight, 8 or 4 bits
  const void* scale;  // [K/C, N] of x's dtype
  const void* zp;     // [K/C, N] of x's dtype, or null
  void* out;          // [M, N] of x's dtype
  int M, N, K, C;     // C: columns per quantization block (K for per-channel weights)
};

// bits = 4 or 8; x's dtype by launcher
int qmm_wo_bw_launch_bf16(const WoBwArgs& a, int bits, hipStream_t stream);
int qmm_wo_bw_launch_f16(const WoBwArgs& a, int bits, hipStream_t stream);
