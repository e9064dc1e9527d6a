// Always-correct kernels for any shape (one thread per output element) and the
// one-time weight re-layout.  They define the arithmetic the fast kernels must
// reproduce: fp32 accumulation inside a reduction, one rounding to the tensor
// dtype wherever the reference materialises a tensor.
#include "qmm_common.h"

// out[m,n] for weight-only quantization.
//   p_s   = round_x( sum_c x[m,s,c] * w[s,c,n] )
//   o     = round_o( sum_s scale[s,n] * p_s )
//   zpo   = round_z( sum_s round_x(sum_c x[m,s,c]) * zp[s,n] ),  o = round_o(o - zpo)
// With S == 1 this is the per-channel formula round_o(round_x(dot) * scale[n]).
// dot_dt replaces x's dtype in the rounding of p_s (f32: the dot product is not rounded);
// the result is stored as store_dt (out_dt, or a final cast of it).
__global__ void __launch_bounds__(256)
qmm_weight_only_generic_kernel(const void* __restrict__ x, const int8_t* __restrict__ w,
                               const void* __restrict__ scale, const void* __restrict__ zp,
                               void* __restrict__ out, int64_t M, int64_t N, int64_t K, int64_t C,
                               int w_layout, int x_dt, int scale_dt, int zp_dt, int dot_dt, int out_dt,
                               int store_dt) {
  int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= M * N) return;
  int64_t m = idx / N, n = idx % N;
  int64_t S = K / C;
  int zpo_dt = qmm_promote(x_dt, zp_dt);
  float o = 0.f, zacc = 0.f;
  for (int64_t s = 0; s < S; ++s) {
    float acc = 0.f, xs = 0.f;
    for (int64_t c = 0; c < C; ++c) {
      int64_t k = s * C + c;
      float xv = qmm_load(x, m * K + k, x_dt);
      int8_t wv = (w_layout == XLA_AMD_W_NK) ? w[n * K + k] : w[k * N + n];
      acc = fmaf(xv, (float)wv, acc);
      xs += xv;
    }
    float p = qmm_round_dt(acc, dot_dt);
    o = fmaf(qmm_load(scale, s * N + n, scale_dt), p, o);
    if (zp) zacc = fmaf(qmm_round_dt(xs, x_dt), qmm_load(zp, s * N + n, zp_dt), zacc);
  }
  o = qmm_round_dt(o, out_dt);
  if (zp) o = qmm_round_dt(o - qmm_round_dt(zacc, zpo_dt), out_dt);
  qmm_store(out, idx, o, store_dt);
}

extern "C" int xla_amd_qmm_weight_only_generic(const void* x, const int8_t* w, const void* scale,
                                               const void* zp, void* out, int64_t M, int64_t N,
                                               int64_t K, int64_t C, int w_layout, int x_dt,
                                               int scale_dt, int zp_dt, int dot_dt, int out_dt,
                                               int store_dt, void* stream) {
  if (!x || !w || !scale || !out) return qmm_fail(XLA_AMD_QMM_EINVAL, "weight_only_generic: null pointer");
  if (M < 0 || N <= 0 || K <= 0 || C <= 0 || K % C != 0)
    return qmm_fail(XLA_AMD_QMM_EINVAL, "weight_only_generic: bad sizes M=%lld N=%lld K=%lld C=%lld",
                    (long long)M, (long long)N, (long long)K, (long long)C);
  if (!qmm_valid_dt(x_dt) || !qmm_valid_dt(scale_dt) || !qmm_valid_dt(out_dt) || !qmm_valid_dt(dot_dt) ||
      !qmm_valid_dt(store_dt) || (zp && !qmm_valid_dt(zp_dt)))
    return qmm_fail(XLA_AMD_QMM_EINVAL, "weight_only_generic: bad dtype enum");
  if (dot_dt != x_dt && (dot_dt != XLA_AMD_DT_F32 || C != K))
    return qmm_fail(XLA_AMD_QMM_EINVAL, "weight_only_generic: dot dtype must be x's, or f32 for per-channel weights");
  if (w_layout != XLA_AMD_W_NK && w_layout != XLA_AMD_W_SCN)
    return qmm_fail(XLA_AMD_QMM_EINVAL, "weight_only_generic: bad weight layout %d", w_layout);
  if (w_layout == XLA_AMD_W_NK && C != K)
    return qmm_fail(XLA_AMD_QMM_EINVAL, "weight_only_generic: [N,K] layout is per-channel (C must equal K)");
  if (out_dt != qmm_promote(x_dt, scale_dt))
    return qmm_fail(XLA_AMD_QMM_EINVAL, "weight_only_generic: out dtype must be promote(x, scale)");
  if (M == 0) return XLA_AMD_QMM_OK;
  int64_t total = M * N;
  int64_t blocks = (total + 255) / 256;
  if (blocks > 0x7fffffffLL) return qmm_fail(XLA_AMD_QMM_EUNSUPPORTED, "weight_only_generic: too many outputs");
  hipLaunchKernelGGL(qmm_weight_only_generic_kernel, dim3((unsigned)blocks), dim3(256), 0,
                     (hipStream_t)stream, x, w, scale, zp, out, M, N, K, C, w_layout, x_dt,
                     scale_dt, zp_dt, dot_dt, out_dt, store_dt);
  return QMM_CHECK_LAUNCH("weight_only_generic launch");
}

// W8A8 for any K: exact int32 dot, then the epilogue chain documented at
// xla_amd_qmm_w8a8_gemm.
__device__ __forceinline__ float qmm_w8a8_epilogue(int acc, int xsum, float ws, float zpv, bool has_zp,
                                                   float xs, int cvt_dt, int mid_dt, int zpo_dt,
                                                   int out_dt) {
  float v = qmm_round_dt((float)acc, cvt_dt);
  v = qmm_round_dt(v * ws, mid_dt);
  if (has_zp) {
    float z = qmm_round_dt(qmm_round_dt((float)xsum, zpo_dt) * zpv, zpo_dt);
    v = qmm_round_dt(v - z, mid_dt);
  }
  return qmm_round_dt(v * xs, out_dt);
}

__global__ void __launch_bounds__(256)
qmm_w8a8_generic_kernel(const int8_t* __restrict__ xq, const int8_t* __restrict__ w,
                        const void* __restrict__ x_scale, const void* __restrict__ w_scale,
                        const void* __restrict__ zp, const int32_t* __restrict__ x_sum,
                        void* __restrict__ out, int32_t* __restrict__ acc_out, int64_t M,
                        int64_t N, int64_t K,
                        int x_scale_dt, int w_scale_dt, int zp_dt, int cvt_dt, int mid_dt,
                        int zpo_dt, int out_dt) {
  int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= M * N) return;
  int64_t m = idx / N, n = idx % N;
  int acc = 0;
  for (int64_t k = 0; k < K; ++k) acc += (int)xq[m * K + k] * (int)w[n * K + k];
  int xsum = zp ? x_sum[m] : 0;
  if (acc_out) acc_out[idx] = acc;
  if (out) {
    float v = qmm_w8a8_epilogue(acc, xsum, qmm_load(w_scale, n, w_scale_dt),
                                zp ? qmm_load(zp, n, zp_dt) : 0.f, zp != nullptr,
                                qmm_load(x_scale, m, x_scale_dt), cvt_dt, mid_dt, zpo_dt, out_dt);
    qmm_store(out, idx, v, out_dt);
  }
}

int qmm_w8a8_generic_launch(const int8_t* xq, const int8_t* w, const void* x_scale,
                            const void* w_scale, const void* zp, const int32_t* x_sum, void* out,
                            int32_t* acc_out, int64_t M, int64_t N, int64_t K, int x_scale_dt,
                            int w_scale_dt,
                            int zp_dt, int cvt_dt, int mid_dt, int zpo_dt, int out_dt,
                            hipStream_t stream) {
  int64_t blocks = (M * N + 255) / 256;
  if (blocks > 0x7fffffffLL) return qmm_fail(XLA_AMD_QMM_EUNSUPPORTED, "w8a8 generic: too many outputs");
  hipLaunchKernelGGL(qmm_w8a8_generic_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, xq, w,
                     x_scale, w_scale, zp, x_sum, out, acc_out, M, N, K, x_scale_dt, w_scale_dt, zp_dt,
                     cvt_dt, mid_dt, zpo_dt, out_dt);
  return QMM_CHECK_LAUNCH("w8a8 generic launch");
}

// ---- one-time weight re-layout ----------------------------------------------
// One thread produces one 32-bit word of the packed row: 4 weights (bits 8) or
// 8 weights (bits 4).  Consecutive threads take consecutive n so that reads of
// the [S,C,N] source coalesce.
__global__ void __launch_bounds__(256)
qmm_pack_kernel(const int8_t* __restrict__ w, uint32_t* __restrict__ packed, int64_t N, int64_t K,
                int src_layout, int bits) {
  int per = bits == 4 ? 8 : 4;
  int64_t words_per_row = K / per;
  int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= N * words_per_row) return;
  int64_t n = idx % N, g = idx / N;
  int64_t k0 = g * per;
  uint32_t word = 0;
  if (bits == 8) {
    for (int j = 0; j < 4; ++j) {
      int64_t k = k0 + j;
      int8_t v = src_layout == XLA_AMD_W_NK ? w[n * K + k] : w[k * N + n];
      word |= ((uint32_t)(uint8_t)v) << (8 * j);
    }
  } else {
    const int P[8] = {0, 2, 4, 6, 1, 3, 5, 7};
    for (int j = 0; j < 8; ++j) {
      int64_t k = k0 + P[j];
      int v = src_layout == XLA_AMD_W_NK ? w[n * K + k] : w[k * N + n];
      word |= ((uint32_t)((v + 8) & 15)) << (4 * j);
    }
  }
  packed[n * words_per_row + g] = word;
}

// Tiled copy for the streaming kernel: one thread writes the 16 bytes that one
// lane of one load will receive.  G channels per group (16, or fewer for some
// per-channel int8 weights): a block holds, for each half h and quarter q of its
// 128 columns, G rows of 16 bytes.
struct TileIndex {
  int64_t n, k0;
};
__device__ __forceinline__ TileIndex qmm_tile_index(int64_t idx, int64_t K, int bits, int G) {
  const int halves = bits == 8 ? 2 : 1;
  const int chunks = halves * 4 * G;  // 16-byte chunks per block
  const int c = (int)(idx % chunks);
  const int64_t blk = idx / chunks;
  const int64_t n_blk = K / 128;
  const int64_t t = blk % n_blk, p = blk / n_blk;
  const int h = c / (4 * G), q = (c % (4 * G)) / G, r = c % G;
  return TileIndex{(int64_t)G * p + r, 128 * t + 32 * q + 16 * h};
}

__global__ void __launch_bounds__(256)
qmm_tile_kernel(const int8_t* __restrict__ w, i32x4* __restrict__ tiled, int64_t N, int64_t K,
                int src_layout, int bits, int G, int64_t total) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const TileIndex ti = qmm_tile_index(idx, K, bits, G);
  const int64_t n = ti.n, k0 = ti.k0;
  auto at = [&](int64_t k) -> int { return src_layout == XLA_AMD_W_NK ? w[n * K + k] : w[k * N + n]; };
  i32x4 v = {0, 0, 0, 0};
  if (n < N) {
    if (bits == 8) {
      for (int i = 0; i < 4; ++i) {
        uint32_t word = 0;
        for (int j = 0; j < 4; ++j) word |= ((uint32_t)(uint8_t)at(k0 + 4 * i + j)) << (8 * j);
        v[i] = (int)word;
      }
    } else {
      const int P[8] = {0, 2, 4, 6, 1, 3, 5, 7};
      for (int i = 0; i < 4; ++i) {
        uint32_t word = 0;
        for (int j = 0; j < 8; ++j) word |= ((uint32_t)((at(k0 + 8 * i + P[j]) + 8) & 15)) << (4 * j);
        v[i] = (int)word;
      }
    }
  }
  tiled[idx] = v;
}

// 16-byte chunks of the tiled copy (one thread each)
static int64_t qmm_tile_chunks(int64_t N, int64_t K, int bits, int G) {
  return ((N + G - 1) / G) * (K / 128) * (bits == 8 ? 8 : 4) * G;
}

extern "C" int xla_amd_qmm_tile_weight(const int8_t* w, void* tiled, int64_t S, int64_t C, int64_t N,
                                       int src_layout, int bits, void* stream) {
  if (!w || !tiled) return qmm_fail(XLA_AMD_QMM_EINVAL, "tile_weight: null pointer");
  if (S <= 0 || C <= 0 || N <= 0) return qmm_fail(XLA_AMD_QMM_EINVAL, "tile_weight: bad sizes");
  if (bits != 4 && bits != 8) return qmm_fail(XLA_AMD_QMM_EINVAL, "tile_weight: bits must be 4 or 8");
  if (src_layout != XLA_AMD_W_NK && src_layout != XLA_AMD_W_SCN)
    return qmm_fail(XLA_AMD_QMM_EINVAL, "tile_weight: bad layout %d", src_layout);
  const int64_t K = S * C;
  if (K % 128 != 0) return qmm_fail(XLA_AMD_QMM_EUNSUPPORTED, "tile_weight: K=%lld not a multiple of 128", (long long)K);
  const int G = xla_amd_qmm_tile_group(N, K, S == 1 ? K : C, bits);
  const int64_t total = qmm_tile_chunks(N, K, bits, G);
  const int64_t blocks = (total + 255) / 256;
  if (blocks > 0x7fffffffLL) return qmm_fail(XLA_AMD_QMM_EUNSUPPORTED, "tile_weight: weight too large");
  hipLaunchKernelGGL(qmm_tile_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, w,
                     (i32x4*)tiled, N, K, src_layout, bits, G, total);
  return QMM_CHECK_LAUNCH("tile_weight launch");
}

// Inverse of qmm_tile_kernel: one thread reads the 16 bytes of one lane fragment and writes
// the 16 (bits 8) or 32 (bits 4) weights they hold back into the operator's layout.
__global__ void __launch_bounds__(256)
qmm_untile_kernel(const i32x4* __restrict__ tiled, int8_t* __restrict__ w, int64_t N, int64_t K,
                  int dst_layout, int bits, int G, int64_t total) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const TileIndex ti = qmm_tile_index(idx, K, bits, G);
  const int64_t n = ti.n, k0 = ti.k0;
  if (n >= N) return;
  const i32x4 v = tiled[idx];
  auto put = [&](int64_t k, int val) {
    if (dst_layout == XLA_AMD_W_NK) w[n * K + k] = (int8_t)val;
    else w[k * N + n] = (int8_t)val;
  };
  if (bits == 8) {
    for (int i = 0; i < 4; ++i)
      for (int j = 0; j < 4; ++j) put(k0 + 4 * i + j, (int)(int8_t)((uint32_t)v[i] >> (8 * j)));
  } else {
    const int P[8] = {0, 2, 4, 6, 1, 3, 5, 7};
    for (int i = 0; i < 4; ++i)
      for (int j = 0; j < 8; ++j) put(k0 + 8 * i + P[j], (int)(((uint32_t)v[i] >> (4 * j)) & 15u) - 8);
  }
}

extern "C" int xla_amd_qmm_untile_weight(const void* tiled, int8_t* w, int64_t S, int64_t C, int64_t N,
                                         int dst_layout, int bits, void* stream) {
  if (!w || !tiled) return qmm_fail(XLA_AMD_QMM_EINVAL, "untile_weight: null pointer");
  if (S <= 0 || C <= 0 || N <= 0) return qmm_fail(XLA_AMD_QMM_EINVAL, "untile_weight: bad sizes");
  if (bits != 4 && bits != 8) return qmm_fail(XLA_AMD_QMM_EINVAL, "untile_weight: bits must be 4 or 8");
  if (dst_layout != XLA_AMD_W_NK && dst_layout != XLA_AMD_W_SCN)
    return qmm_fail(XLA_AMD_QMM_EINVAL, "untile_weight: bad layout %d", dst_layout);
  const int64_t K = S * C;
  if (K % 128 != 0) return qmm_fail(XLA_AMD_QMM_EUNSUPPORTED, "untile_weight: K=%lld not a multiple of 128", (long long)K);
  const int G = xla_amd_qmm_tile_group(N, K, S == 1 ? K : C, bits);
  const int64_t total = qmm_tile_chunks(N, K, bits, G);
  const int64_t blocks = (total + 255) / 256;
  if (blocks > 0x7fffffffLL) return qmm_fail(XLA_AMD_QMM_EUNSUPPORTED, "untile_weight: weight too large");
  hipLaunchKernelGGL(qmm_untile_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                     (const i32x4*)tiled, w, N, K, dst_layout, bits, G, total);
  return QMM_CHECK_LAUNCH("untile_weight launch");
}

extern "C" int xla_amd_qmm_pack_weight(const int8_t* w, void* packed, int64_t S, int64_t C, int64_t N,
                                       int src_layout, int bits, void* stream) {
  if (!w || !packed) return qmm_fail(XLA_AMD_QMM_EINVAL, "pack_weight: null pointer");
  if (S <= 0 || C <= 0 || N <= 0) return qmm_fail(XLA_AMD_QMM_EINVAL, "pack_weight: bad sizes");
  if (bits != 4 && bits != 8) return qmm_fail(XLA_AMD_QMM_EINVAL, "pack_weight: bits must be 4 or 8");
  if (src_layout != XLA_AMD_W_NK && src_layout != XLA_AMD_W_SCN)
    return qmm_fail(XLA_AMD_QMM_EINVAL, "pack_weight: bad layout %d", src_layout);
  int64_t K = S * C;
  int per = bits == 4 ? 8 : 4;
  if (K % per != 0) return qmm_fail(XLA_AMD_QMM_EUNSUPPORTED, "pack_weight: K=%lld not a multiple of %d", (long long)K, per);
  int64_t total = N * (K / per);
  int64_t blocks = (total + 255) / 256;
  if (blocks > 0x7fffffffLL) return qmm_fail(XLA_AMD_QMM_EUNSUPPORTED, "pack_weight: weight too large");
  // Values outside [-8,7] are stored modulo 16 (two's-complement truncation),
  // as a reinterpreting cast to a 4-bit type would.
  hipLaunchKernelGGL(qmm_pack_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, w,
                     (uint32_t*)packed, N, K, src_layout, bits);
  return QMM_CHECK_LAUNCH("pack_weight launch");
}
