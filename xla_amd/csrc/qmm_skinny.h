// Arguments and launchers of the weight-streaming kernel (qmm_skinny.hip), shared with the entry
// point that runs it over K slices (qmm_wo_gemm.hip).
#pragma once
#include <hip/hip_runtime.h>
#include <cstdint>

struct SkinnyArgs {
  const void* x;
  const uint8_t* w;  // K-major packed weight
  const void* scale;
  const void* zp;
  void* out;
  int M, N, K, C;  // M = rows of this pass (<= 16*MT)
  int G;           // channels per group of the tiled weight (xla_amd_qmm_tile_group)
  int scale_dt, zp_dt, out_dt;
  int dot_dt;    // dtype the dot product is rounded to before it is scaled (per-channel only)
  int store_dt;  // dtype of the stored tensor (out_dt, or a final cast of it)
  // K slices over workgroups: blockIdx.y = slice of k_per_slice columns (a
  // multiple of the kernel's step, 512 columns for int8 and 1024 for int4; K when there is one slice).  With slices the kernel stores its raw sums instead
  // of results: part [slices][M][N] dot products, part_xs [slices][M] row sums of x (zero point only).
  int k_per_slice;
  int slices;
  float* part;
  float* part_xs;
  // Blockwise weights (slices of whole quantization blocks): part holds the slices' sums of scale * round(block dot),
  // part_z [slices][M][N] their sums of round(block sum of x) * zero point; both only need adding and the final roundings.
  float* part_z;
  // Diagnostic build of the kernel only (its time notes): offset of their LDS area, -1 = none.
  int tl_off = -1;
};

int qmm_skinny_launch_f32(const SkinnyArgs& a, int bits, bool haszp, hipStream_t stream);
int qmm_skinny_launch_bf16(const SkinnyArgs& a, int bits, bool haszp, hipStream_t stream);
int qmm_skinny_launch_f16(const SkinnyArgs& a, int bits, bool haszp, hipStream_t stream);

// K slices the streaming kernel should run a per-channel launch of M <= 32 rows in (1 = none):
// few output channels against a long K, where every workgroup would otherwise copy all of x.
int qmm_skinny_k_slices(int64_t M, int64_t N, int64_t K, int64_t C, int bits, int* k_per_slice);

// The persistent form of the streaming kernel with all of x resident in LDS (qmm_skinny_resident.hip): how many
// workgroups a launch would run with (0: not a launch for it), and its launchers.
int qmm_skinny_resident_workgroups(const SkinnyArgs& a, int x_dt, int bits);
int qmm_skinny_resident_launch_bf16(const SkinnyArgs& a, bool haszp, int workgroups, hipStream_t stream);
int qmm_skinny_resident_launch_f16(const SkinnyArgs& a, bool haszp, int workgroups, hipStream_t stream);
