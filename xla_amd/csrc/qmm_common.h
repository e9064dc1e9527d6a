// Shared host/device helpers of libxla_amd_qmm.so (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "xla_amd_qmm.h"

// ---- host side -------------------------------------------------------------
// printf-style setter of the calling thread's error text; returns `code`.
int qmm_fail(int code, const char* fmt, ...);
// Maps a HIP status to XLA_AMD_QMM_OK / XLA_AMD_QMM_EHIP (recording the text).
int qmm_check_hip(hipError_t e, const char* what);
// Error of the launch that was just issued on the calling thread.
#define QMM_CHECK_LAUNCH(what) qmm_check_hip(hipGetLastError(), what)

// Raises a kernel's dynamic-LDS limit (hipFuncAttributeMaxDynamicSharedMemorySize) once per
// device: the attribute belongs to the function as loaded on the current device, so `done`
// (one mask per kernel instantiation, shared by all host threads) holds one bit per device
// ordinal; ordinals from 64 on set the attribute on every launch.
int qmm_set_max_lds(const void* kernel, int bytes, std::atomic<uint64_t>& done, const char* what);

static inline bool qmm_valid_dt(int dt) { return dt >= XLA_AMD_DT_F32 && dt <= XLA_AMD_DT_F16; }
static inline int qmm_dt_size(int dt) { return dt == XLA_AMD_DT_F32 ? 4 : 2; }
// torch's type promotion between two floating dtypes: equal -> itself,
// anything else involving f32, or bf16 with f16 -> f32.
__host__ __device__ static inline int qmm_promote(int a, int b) { return a == b ? a : XLA_AMD_DT_F32; }

// ---- device side -----------------------------------------------------------
// Compile-time loop: f(integral_constant<int, 0>) ... f(integral_constant<int, N-1>).
// Keeps register arrays indexed by constants where `#pragma unroll` gives up.
template <int V> struct qmm_const { static constexpr int value = V; constexpr operator int() const { return V; } };
template <int N, int I = 0, typename F>
__device__ __forceinline__ void qmm_static_for(F&& f) {
  if constexpr (I < N) {
    f(qmm_const<I>{});
    qmm_static_for<N, I + 1>(f);
  }
}

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x2 __attribute__((ext_vector_type(2)));
typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also makes
// every wave wait for its outstanding *global* loads (its fence covers all
// address spaces), which would drain the prefetch pipeline at every step.
__device__ __forceinline__ void qmm_lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// Workgroup barrier with no fence at all: waits for this wave's own LDS operations, then
// s_barrier.  For code that keeps global -> LDS copies in flight across the barrier and does
// its own vmcnt waits (a workgroup-scope fence makes the compiler wait for every such copy,
// since they are LDS writes); the memory clobber keeps LDS accesses on their side of it.
// Waits until at most N of this wave's vector memory operations are outstanding (they complete in order);
// the other counters are left alone.
template <int N> __device__ __forceinline__ void qmm_wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt has six bits");
  __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
}

__device__ __forceinline__ void qmm_bare_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

__device__ __forceinline__ float qmm_bf16_to_f32(uint16_t b) {
  return __uint_as_float(((uint32_t)b) << 16);
}

// Round-to-nearest-even f32 -> bf16 bit pattern (NaN stays NaN): the hardware conversion
// (v_cvt_pk_bf16_f32).
__device__ __forceinline__ uint16_t qmm_f32_to_bf16(float f) {
  return __builtin_bit_cast(uint16_t, (__bf16)f);
}
// Two values at once, lo in the low half.
__device__ __forceinline__ uint32_t qmm_f32x2_to_bf16x2(float lo, float hi) {
  typedef float qmm_f32x2_t __attribute__((ext_vector_type(2)));
  typedef __bf16 qmm_bf16x2_t __attribute__((ext_vector_type(2)));
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(qmm_f32x2_t{lo, hi}, qmm_bf16x2_t));
}
__device__ __forceinline__ uint32_t qmm_f32x2_to_f16x2(float lo, float hi) {
  typedef float qmm_f32x2_t __attribute__((ext_vector_type(2)));
  typedef _Float16 qmm_f16x2_t __attribute__((ext_vector_type(2)));
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(qmm_f32x2_t{lo, hi}, qmm_f16x2_t));
}

__device__ __forceinline__ float qmm_f16_to_f32(uint16_t h) {
  _Float16 v;
  __builtin_memcpy(&v, &h, 2);
  return (float)v;
}

__device__ __forceinline__ uint16_t qmm_f32_to_f16(float f) {
  _Float16 v = (_Float16)f;  // v_cvt_f16_f32: round-to-nearest-even
  uint16_t h;
  __builtin_memcpy(&h, &v, 2);
  return h;
}

// Value of f after a round trip through dtype dt (what storing a torch tensor
// of that dtype and reading it back does).
__device__ __forceinline__ float qmm_round_dt(float f, int dt) {
  if (dt == XLA_AMD_DT_BF16) return qmm_bf16_to_f32(qmm_f32_to_bf16(f));
  if (dt == XLA_AMD_DT_F16) return qmm_f16_to_f32(qmm_f32_to_f16(f));
  return f;
}

// Element i as raw bits, without a branch on the dtype and without touching the
// value: a prefetch written with qmm_load would wait for each element in turn
// (the conversion sits inside the dtype branch).  qmm_from_raw converts later.
__device__ __forceinline__ uint32_t qmm_load_raw(const void* p, int64_t i, int dt) {
  const int esz = dt == XLA_AMD_DT_F32 ? 4 : 2;
  const char* q = (const char*)p + i * esz;
  const uint32_t lo = *(const uint16_t*)q;
  const uint32_t hi = *(const uint16_t*)(q + (esz - 2));  // the same halfword again for 2-byte types
  return lo | (hi << 16);
}
__device__ __forceinline__ float qmm_from_raw(uint32_t raw, int dt) {
  if (dt == XLA_AMD_DT_BF16) return __uint_as_float(raw << 16);
  if (dt == XLA_AMD_DT_F16) return qmm_f16_to_f32((uint16_t)(raw & 0xffffu));
  return __uint_as_float(raw);
}

__device__ __forceinline__ float qmm_load(const void* p, int64_t i, int dt) {
  if (dt == XLA_AMD_DT_BF16) return qmm_bf16_to_f32(((const uint16_t*)p)[i]);
  if (dt == XLA_AMD_DT_F16) return qmm_f16_to_f32(((const uint16_t*)p)[i]);
  return ((const float*)p)[i];
}

// Stores a value that is already on dt's grid (or rounds it there).
__device__ __forceinline__ void qmm_store(void* p, int64_t i, float v, int dt) {
  if (dt == XLA_AMD_DT_BF16)
    ((uint16_t*)p)[i] = qmm_f32_to_bf16(v);
  else if (dt == XLA_AMD_DT_F16)
    ((uint16_t*)p)[i] = qmm_f32_to_f16(v);
  else
    ((float*)p)[i] = v;
}
