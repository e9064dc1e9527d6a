// Affine quantize / dequantize of whole tensors (per tensor or per channel):
// HBM-bound elementwise kernels for the quantized_decomposed operators that
// sit on either side of a quantized matmul in PT2E flows.
//
// A contiguous tensor is addressed as [outer, channels, inner]; element
// (o, c, i) uses parameter c (channels == 1: per tensor).  The arithmetic is
// torch's decomposition (torch/ao/quantization/fx/_decomposed.py), op by op in
// f32:  q = cast(clamp(rint(f32(x) * inv_scale[c]) + zp[c], qmin, qmax))
// (rint: half to even); NaN maps to 0.
#include "qmm_common.h"

namespace {

__device__ __forceinline__ int qdq_load_q(const void* q, int64_t i, int q_dt) {
  switch (q_dt) {
    case XLA_AMD_QDT_I8: return ((const int8_t*)q)[i];
    case XLA_AMD_QDT_U8: return ((const uint8_t*)q)[i];
    case XLA_AMD_QDT_I16: return ((const int16_t*)q)[i];
    default: return ((const int32_t*)q)[i];
  }
}
__device__ __forceinline__ void qdq_store_q(void* q, int64_t i, int v, int q_dt) {
  switch (q_dt) {
    case XLA_AMD_QDT_I8: ((int8_t*)q)[i] = (int8_t)v; break;
    case XLA_AMD_QDT_U8: ((uint8_t*)q)[i] = (uint8_t)v; break;
    case XLA_AMD_QDT_I16: ((int16_t*)q)[i] = (int16_t)v; break;
    default: ((int32_t*)q)[i] = v; break;
  }
}

__device__ __forceinline__ int quantize_value(float x, float inv_scale, float zp, float qmin, float qmax) {
  float r = rintf(x * inv_scale) + zp;
  r = fminf(fmaxf(r, qmin), qmax);  // NaN -> qmin by fmaxf/fminf; mapped to 0 below
  return (x != x) ? 0 : (int)r;
}

// One thread per 8 consecutive elements of a row of `inner` (inner % 8 == 0,
// 16-byte aligned x, 8-byte aligned q, 1-byte q) or per element otherwise.
template <int XT, bool VEC>
__global__ void __launch_bounds__(256)
qdq_quantize_kernel(const void* __restrict__ x, void* __restrict__ q, const float* __restrict__ inv_scale,
                    const int32_t* __restrict__ zp, int64_t total, int64_t channels, int64_t inner,
                    int q_dt, float qmin, float qmax) {
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if constexpr (VEC) {
    const int64_t e0 = t * 8;
    if (e0 >= total) return;
    const int64_t c = (e0 / inner) % channels;
    const float is = inv_scale[c], z = (float)zp[c];
    float f[8];
    if constexpr (XT == XLA_AMD_DT_F32) {
      const f32x4 a = ((const f32x4*)((const float*)x + e0))[0], b = ((const f32x4*)((const float*)x + e0))[1];
#pragma unroll
      for (int i = 0; i < 4; ++i) { f[i] = a[i]; f[4 + i] = b[i]; }
    } else {
      const i32x4 a = *(const i32x4*)((const uint16_t*)x + e0);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t d = (uint32_t)a[i];
        f[2 * i] = XT == XLA_AMD_DT_BF16 ? __uint_as_float(d << 16) : qmm_f16_to_f32((uint16_t)(d & 0xffffu));
        f[2 * i + 1] = XT == XLA_AMD_DT_BF16 ? __uint_as_float(d & 0xffff0000u) : qmm_f16_to_f32((uint16_t)(d >> 16));
      }
    }
    uint32_t lo = 0, hi = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      lo |= ((uint32_t)(uint8_t)quantize_value(f[i], is, z, qmin, qmax)) << (8 * i);
      hi |= ((uint32_t)(uint8_t)quantize_value(f[4 + i], is, z, qmin, qmax)) << (8 * i);
    }
    *(i32x2*)((uint8_t*)q + e0) = i32x2{(int)lo, (int)hi};
  } else {
    if (t >= total) return;
    const int64_t c = (t / inner) % channels;
    qdq_store_q(q, t, quantize_value(qmm_load(x, t, XT), inv_scale[c], (float)zp[c], qmin, qmax), q_dt);
  }
}

// int_subtract != 0: out = cast(f32(q - zp[c]) * scale[c])            (per-channel form)
// int_subtract == 0: out = round(round(cast(q) - zp[c]) * scale[c])   (per-tensor form, tensor ops in out's dtype)
__device__ __forceinline__ float dequantize_value(int qv, int z, float sc, int out_dt, int int_subtract) {
  if (int_subtract) return (float)(qv - z) * sc;
  // (zero point and scale are host scalars there: they enter the arithmetic as f32)
  const float a = qmm_round_dt((float)qv, out_dt);
  const float d = qmm_round_dt(a - (float)z, out_dt);
  return d * sc;
}

// VEC: one thread per 8 consecutive 1-byte elements of a row of `inner`
// (inner % 8 == 0, 8-byte aligned q, 32-byte aligned out), else one per element.
template <bool VEC>
__global__ void __launch_bounds__(256)
qdq_dequantize_kernel(const void* __restrict__ q, void* __restrict__ out, const float* __restrict__ scale,
                      const int32_t* __restrict__ zp, int64_t total, int64_t channels, int64_t inner,
                      int q_dt, int out_dt, int int_subtract) {
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if constexpr (VEC) {
    const int64_t e0 = t * 8;
    if (e0 >= total) return;
    const int64_t c = (e0 / inner) % channels;
    const int z = zp ? zp[c] : 0;
    const float sc = scale[c];
    const i32x2 raw = *(const i32x2*)((const uint8_t*)q + e0);
    float r[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t b = ((uint32_t)raw[i >> 2] >> (8 * (i & 3))) & 0xffu;
      const int qv = q_dt == XLA_AMD_QDT_I8 ? (int)(int8_t)b : (int)b;
      r[i] = dequantize_value(qv, z, sc, out_dt, int_subtract);
    }
    if (out_dt == XLA_AMD_DT_F32) {
      f32x4* o = (f32x4*)((float*)out + e0);
      o[0] = f32x4{r[0], r[1], r[2], r[3]};
      o[1] = f32x4{r[4], r[5], r[6], r[7]};
    } else {
      i32x4 pk;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t lo = out_dt == XLA_AMD_DT_BF16 ? qmm_f32_to_bf16(r[2 * i]) : qmm_f32_to_f16(r[2 * i]);
        const uint32_t hi = out_dt == XLA_AMD_DT_BF16 ? qmm_f32_to_bf16(r[2 * i + 1]) : qmm_f32_to_f16(r[2 * i + 1]);
        pk[i] = (int)(lo | (hi << 16));
      }
      *(i32x4*)((uint16_t*)out + e0) = pk;
    }
  } else {
    if (t >= total) return;
    const int64_t c = (t / inner) % channels;
    const int z = zp ? zp[c] : 0;
    qmm_store(out, t, dequantize_value(qdq_load_q(q, t, q_dt), z, scale[c], out_dt, int_subtract), out_dt);
  }
}

bool valid_qdt(int q_dt) { return q_dt >= XLA_AMD_QDT_I8 && q_dt <= XLA_AMD_QDT_I32; }

}  // namespace

extern "C" int xla_amd_qmm_quantize_affine(const void* x, void* q, const float* inv_scale,
                                           const int32_t* zp, int64_t outer, int64_t channels,
                                           int64_t inner, int x_dt, int q_dt, int32_t qmin,
                                           int32_t qmax, void* stream) {
  if (!x || !q || !inv_scale || !zp) return qmm_fail(XLA_AMD_QMM_EINVAL, "quantize_affine: null pointer");
  if (outer < 0 || channels <= 0 || inner < 0) return qmm_fail(XLA_AMD_QMM_EINVAL, "quantize_affine: bad sizes");
  if (!qmm_valid_dt(x_dt) || !valid_qdt(q_dt) || qmin > qmax)
    return qmm_fail(XLA_AMD_QMM_EINVAL, "quantize_affine: bad dtype enum or bounds");
  const int64_t total = outer * channels * inner;
  if (total == 0) return XLA_AMD_QMM_OK;
  const bool vec = (q_dt == XLA_AMD_QDT_I8 || q_dt == XLA_AMD_QDT_U8) && inner % 8 == 0 &&
                   (((uintptr_t)x & 15) == 0) && (((uintptr_t)q & 7) == 0);
  const int64_t threads = vec ? total / 8 : total;
  const int64_t blocks = (threads + 255) / 256;
  if (blocks > 0x7fffffffLL) return qmm_fail(XLA_AMD_QMM_EUNSUPPORTED, "quantize_affine: tensor too large");
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)blocks), block(256);
  const float fmin = (float)qmin, fmax = (float)qmax;
#define QDQ_LAUNCH(XT)                                                                                          \
  do {                                                                                                          \
    if (vec) hipLaunchKernelGGL((qdq_quantize_kernel<XT, true>), grid, block, 0, s, x, q, inv_scale, zp, total, \
                                channels, inner, q_dt, fmin, fmax);                                             \
    else hipLaunchKernelGGL((qdq_quantize_kernel<XT, false>), grid, block, 0, s, x, q, inv_scale, zp, total,    \
                            channels, inner, q_dt, fmin, fmax);                                                 \
  } while (0)
  if (x_dt == XLA_AMD_DT_BF16) QDQ_LAUNCH(XLA_AMD_DT_BF16);
  else if (x_dt == XLA_AMD_DT_F16) QDQ_LAUNCH(XLA_AMD_DT_F16);
  else QDQ_LAUNCH(XLA_AMD_DT_F32);
#undef QDQ_LAUNCH
  return QMM_CHECK_LAUNCH("quantize_affine launch");
}

extern "C" int xla_amd_qmm_dequantize_affine(const void* q, void* out, const float* scale,
                                             const int32_t* zp, int64_t outer, int64_t channels,
                                             int64_t inner, int q_dt, int out_dt, int int_subtract,
                                             void* stream) {
  if (!q || !out || !scale) return qmm_fail(XLA_AMD_QMM_EINVAL, "dequantize_affine: null pointer");
  if (outer < 0 || channels <= 0 || inner < 0) return qmm_fail(XLA_AMD_QMM_EINVAL, "dequantize_affine: bad sizes");
  if (!qmm_valid_dt(out_dt) || !valid_qdt(q_dt)) return qmm_fail(XLA_AMD_QMM_EINVAL, "dequantize_affine: bad dtype enum");
  const int64_t total = outer * channels * inner;
  if (total == 0) return XLA_AMD_QMM_OK;
  const bool vec = (q_dt == XLA_AMD_QDT_I8 || q_dt == XLA_AMD_QDT_U8) && inner % 8 == 0 &&
                   (((uintptr_t)q & 7) == 0) && (((uintptr_t)out & 31) == 0);
  const int64_t threads = vec ? total / 8 : total;
  const int64_t blocks = (threads + 255) / 256;
  if (blocks > 0x7fffffffLL) return qmm_fail(XLA_AMD_QMM_EUNSUPPORTED, "dequantize_affine: tensor too large");
  if (vec)
    hipLaunchKernelGGL(qdq_dequantize_kernel<true>, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, q, out,
                       scale, zp, total, channels, inner, q_dt, out_dt, int_subtract);
  else
    hipLaunchKernelGGL(qdq_dequantize_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, q, out,
                       scale, zp, total, channels, inner, q_dt, out_dt, int_subtract);
  return QMM_CHECK_LAUNCH("dequantize_affine launch");
}
