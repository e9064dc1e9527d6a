// Per-token dynamic int8 quantization of activations (HBM-bound elementwise +
// row reduction).  One workgroup per row.  Rows of up to 16384 elements stay in
// registers between the abs-max pass and the quantize pass (x is read exactly
// once); longer rows are read a second time, which hits L2.
//
// A row that holds a NaN: scale = NaN (torch.amax propagates it), every x_q of the row 0
// (the reference's cast of NaN to int8 is undefined).  An all-zero row: scale = 0, x_q = 0.
//
// The arithmetic is the reference's, op by op, in x's dtype:
//   max = amax(|x|); scale = RN_x(max / 127); r = RN_x(x / scale); q = int8(rint(r))
// RN_x(a / b) is obtained as RN_x(RN_f32(a / b)): a and b carry at most 11
// significant bits, so the f32 quotient never straddles a rounding boundary of
// the narrower type unless it is exact.
#include "qmm_common.h"

namespace {

constexpr int kThreads = 256;

// max that keeps a NaN (fmaxf would drop it): a row that holds a NaN gets a NaN scale, as torch.amax gives
__device__ __forceinline__ float nan_max(float a, float b) { return (a > b || a != a) ? a : b; }
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = nan_max(v, __shfl_xor(v, o, 64));
  return v;
}
__device__ __forceinline__ int wave_sum(int v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// RN_f32(xv / scale) for a row's scale.  2-byte x with a scale well inside the f32 range: one
// multiplication by the row's reciprocal (refined to within half an ulp once per row) and one
// correction step on the exact remainder.  The result is then rounded to x's 8- or 11-bit
// significand, which only asks for the f32 quotient to be exact where the true quotient is
// representable (a tie of the narrower type is) and on the right side of every tie elsewhere:
// the corrected quotient is within a fraction of an f32 ulp, x / scale of two such numbers
// is never that close to a tie without being one.  (Checked against the division for every
// pair of bf16 and of f16 values by the GPU tests.)  Otherwise: the IEEE division.
struct RowDivisor {
  float scale, rc;
  bool fast;
};
template <int XT>
__device__ __forceinline__ RowDivisor row_divisor(float scale) {
  RowDivisor d;
  d.scale = scale;
  d.fast = XT != XLA_AMD_DT_F32 && scale > 1e-30f && scale < 1e30f;  // (false for NaN too)
  float rc = __builtin_amdgcn_rcpf(scale);
  rc = fmaf(fmaf(-scale, rc, 1.0f), rc, rc);
  d.rc = rc;
  return d;
}
__device__ __forceinline__ int quantize_one(float xv, const RowDivisor& d, int x_dt, int policy) {
  if (d.fast) {
    // Every x of the row is finite and at most 127.25 scales in magnitude (190.5 when an f16 scale was
    // rounded in the subnormal range): no NaN, no infinity, nothing near the int32 range.
    const float q0 = xv * d.rc;
    const float q = fmaf(fmaf(-q0, d.scale, xv), d.rc, q0);
    const float r = rintf(qmm_round_dt(q, x_dt));  // rintf: round half to even
    if (policy == XLA_AMD_OVERFLOW_SATURATE) return (int)fminf(fmaxf(r, -128.f), 127.f);
    return (int)(int8_t)(int)r;
  }
  float r = rintf(qmm_round_dt(xv / d.scale, x_dt));
  if (!(fabsf(r) <= 3.0e38f)) r = 0.f;              // NaN/inf (zero scale) -> 0
  if (policy == XLA_AMD_OVERFLOW_SATURATE) return (int)fminf(fmaxf(r, -128.f), 127.f);
  r = fminf(fmaxf(r, -2147483648.f), 2147483520.f);
  return (int)(int8_t)(int)r;
}

// VEC = elements per thread per step: 8 (16-byte loads of 2-byte types, two
// for f32) when K % 8 == 0 and the row starts are 16-byte aligned, else 1.
// KEEP: vector steps of the row a thread keeps in registers (0 = read twice).
template <int XT, int VEC, int KEEP>
__global__ void __launch_bounds__(kThreads)
qmm_quantize_kernel(const void* __restrict__ x, int8_t* __restrict__ xq, void* __restrict__ x_scale,
                    int32_t* __restrict__ x_sum, int64_t K, int scale_out_dt, int policy) {
  __shared__ float smax[kThreads / 64];
  __shared__ int ssum[kThreads / 64];
  const int64_t m = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  constexpr int esz = XT == XLA_AMD_DT_F32 ? 4 : 2;
  const char* xrow = (const char*)x + (size_t)m * K * esz;

  auto load_vec = [&](int64_t k, float* f) __attribute__((always_inline)) {
    if constexpr (VEC == 1) {
      f[0] = qmm_load(xrow, k, XT);
    } else if constexpr (XT == XLA_AMD_DT_F32) {
      const f32x4* p = (const f32x4*)(xrow + k * 4);
      f32x4 a = p[0], b = p[1];
#pragma unroll
      for (int i = 0; i < 4; ++i) { f[i] = a[i]; f[4 + i] = b[i]; }
    } else {
      i32x4 a = *(const i32x4*)(xrow + k * 2);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        uint32_t d = (uint32_t)a[i];
        if constexpr (XT == XLA_AMD_DT_BF16) {
          f[2 * i] = __uint_as_float(d << 16);
          f[2 * i + 1] = __uint_as_float(d & 0xffff0000u);
        } else {
          f[2 * i] = qmm_f16_to_f32((uint16_t)(d & 0xffffu));
          f[2 * i + 1] = qmm_f16_to_f32((uint16_t)(d >> 16));
        }
      }
    }
  };

  // pass 1: row abs-max
  float mx = 0.f;
  float held[KEEP > 0 ? KEEP : 1][VEC];
  if constexpr (KEEP > 0) {
#pragma unroll
    for (int s = 0; s < KEEP; ++s) {
      const int64_t k = ((int64_t)s * kThreads + tid) * VEC;
      if (k < K) {
        load_vec(k, held[s]);
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
          mx = nan_max(fabsf(held[s][i]), mx);
        }
      }
    }
  } else {
    for (int64_t k = (int64_t)tid * VEC; k < K; k += (int64_t)kThreads * VEC) {
      float f[VEC];
      load_vec(k, f);
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        mx = nan_max(fabsf(f[i]), mx);
      }
    }
  }
  mx = wave_max(mx);
  if (lane == 0) smax[wv] = mx;
  __syncthreads();
  mx = smax[0];
#pragma unroll
  for (int i = 1; i < kThreads / 64; ++i) mx = nan_max(mx, smax[i]);
  const float scale = qmm_round_dt(mx / 127.0f, XT);
  const RowDivisor divisor = row_divisor<XT>(scale);

  // pass 2: quantize
  int lsum = 0;
  auto emit = [&](int64_t k, const float* f) __attribute__((always_inline)) {
    int q[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      q[i] = quantize_one(f[i], divisor, XT, policy);
      lsum += q[i];
    }
    if constexpr (VEC == 1) {
      xq[(size_t)m * K + k] = (int8_t)q[0];
    } else {
      uint32_t lo = 0, hi = 0;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        lo |= ((uint32_t)(uint8_t)q[i]) << (8 * i);
        hi |= ((uint32_t)(uint8_t)q[4 + i]) << (8 * i);
      }
      i32x2 v = {(int)lo, (int)hi};
      *(i32x2*)(xq + (size_t)m * K + k) = v;
    }
  };
  if constexpr (KEEP > 0) {
#pragma unroll
    for (int s = 0; s < KEEP; ++s) {
      const int64_t k = ((int64_t)s * kThreads + tid) * VEC;
      if (k < K) emit(k, held[s]);
    }
  } else {
    for (int64_t k = (int64_t)tid * VEC; k < K; k += (int64_t)kThreads * VEC) {
      float f[VEC];
      load_vec(k, f);
      emit(k, f);
    }
  }
  if (tid == 0) qmm_store(x_scale, m, scale, scale_out_dt);
  if (x_sum) {
    lsum = wave_sum(lsum);
    if (lane == 0) ssum[wv] = lsum;
    __syncthreads();
    if (tid == 0) {
      int t = 0;
#pragma unroll
      for (int i = 0; i < kThreads / 64; ++i) t += ssum[i];
      x_sum[m] = t;
    }
  }
}

template <int XT>
int launch(const void* x, int8_t* xq, void* x_scale, int32_t* x_sum, int64_t M, int64_t K,
           int scale_out_dt, int policy, bool vec, hipStream_t stream) {
  const dim3 grid((unsigned)M), block(kThreads);
  if (!vec)
    hipLaunchKernelGGL((qmm_quantize_kernel<XT, 1, 0>), grid, block, 0, stream, x, xq, x_scale, x_sum, K, scale_out_dt, policy);
  else if (K <= 2 * kThreads * 8)
    hipLaunchKernelGGL((qmm_quantize_kernel<XT, 8, 2>), grid, block, 0, stream, x, xq, x_scale, x_sum, K, scale_out_dt, policy);
  else if (K <= 4 * kThreads * 8)
    hipLaunchKernelGGL((qmm_quantize_kernel<XT, 8, 4>), grid, block, 0, stream, x, xq, x_scale, x_sum, K, scale_out_dt, policy);
  else if (K <= 8 * kThreads * 8)
    hipLaunchKernelGGL((qmm_quantize_kernel<XT, 8, 8>), grid, block, 0, stream, x, xq, x_scale, x_sum, K, scale_out_dt, policy);
  else
    hipLaunchKernelGGL((qmm_quantize_kernel<XT, 8, 0>), grid, block, 0, stream, x, xq, x_scale, x_sum, K, scale_out_dt, policy);
  return QMM_CHECK_LAUNCH("quantize_per_token launch");
}

}  // namespace

extern "C" int xla_amd_qmm_quantize_per_token(const void* x, int8_t* x_q, void* x_scale,
                                              int32_t* x_sum, int64_t M, int64_t K, int x_dt,
                                              int scale_out_dt, int overflow_policy, void* stream) {
  if (!x || !x_q || !x_scale) return qmm_fail(XLA_AMD_QMM_EINVAL, "quantize_per_token: null pointer");
  if (M < 0 || K <= 0 || M > 0x7fffffffLL)
    return qmm_fail(XLA_AMD_QMM_EINVAL, "quantize_per_token: bad sizes M=%lld K=%lld", (long long)M, (long long)K);
  if (!qmm_valid_dt(x_dt) || !qmm_valid_dt(scale_out_dt))
    return qmm_fail(XLA_AMD_QMM_EINVAL, "quantize_per_token: bad dtype enum");
  if (overflow_policy != XLA_AMD_OVERFLOW_SATURATE && overflow_policy != XLA_AMD_OVERFLOW_WRAP)
    return qmm_fail(XLA_AMD_QMM_EINVAL, "quantize_per_token: bad overflow policy %d", overflow_policy);
  if (M == 0) return XLA_AMD_QMM_OK;
  bool vec = (K % 8 == 0) && (((uintptr_t)x & 15) == 0) && (((uintptr_t)x_q & 7) == 0);
  hipStream_t s = (hipStream_t)stream;
  if (x_dt == XLA_AMD_DT_BF16) return launch<XLA_AMD_DT_BF16>(x, x_q, x_scale, x_sum, M, K, scale_out_dt, overflow_policy, vec, s);
  if (x_dt == XLA_AMD_DT_F16) return launch<XLA_AMD_DT_F16>(x, x_q, x_scale, x_sum, M, K, scale_out_dt, overflow_policy, vec, s);
  return launch<XLA_AMD_DT_F32>(x, x_q, x_scale, x_sum, M, K, scale_out_dt, overflow_policy, vec, s);
}
