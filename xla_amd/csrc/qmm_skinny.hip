// Weight-streaming GEMV / skinny GEMM for weight-only quantized linear layers
// on gfx950.  HBM-bound: every weight byte is read once with 128-bit loads,
// converted in registers and fed to MFMA against up to 64 rows of x that stay
// in registers; K is split over the waves of a workgroup and reduced in LDS.
//
// Thread/data mapping.  A workgroup owns 16*RG consecutive output channels
// (rows n of the K-major weight).  Lane l of a wave is (r = l%16, g = l/16):
// in one k-iteration of 128 columns it loads, for row n0+r, the 32 weights at
// columns k0+32g..k0+32g+31 (32 bytes for int8, 16 bytes for int4), and for x
// row m = r of each 16-row tile the same 32 columns.  The 32 columns go
// through four 16x16x32 MFMAs (A = weights: 16 channels x 32 k, B = x^T:
// 32 k x 16 rows), each lane contributing 8 k per MFMA for both operands, so
// any k-order the hardware uses inside the instruction pairs the same
// elements.  D[i][j] lands in lane (j + 16*(i/4)), register i%4:
// channel n0 + 4g + v, x row r.
#include "qmm_common.h"

namespace {

constexpr int kWaves = 4;    // waves per workgroup (K is split over them)
constexpr int kKIter = 128;  // k columns per wave iteration

// ---- operand fragments --------------------------------------------------------
__device__ __forceinline__ uint32_t pack_hi16(float lo, float hi) {
  // {bf16(lo), bf16(hi)} by truncation: exact for integers of magnitude <= 256.
  return __builtin_amdgcn_perm(__float_as_uint(hi), __float_as_uint(lo), 0x07060302u);
}

__device__ __forceinline__ uint32_t pack_f16(float lo, float hi) {
  typedef _Float16 h2 __attribute__((ext_vector_type(2)));
  h2 v = __builtin_bit_cast(h2, __builtin_amdgcn_cvt_pkrtz(lo, hi));  // exact for small integers
  return __builtin_bit_cast(uint32_t, v);
}

// 8 int8 weights (two dwords) -> 8 elements of the x dtype.
template <int XT>
__device__ __forceinline__ i32x4 cvt_w8(uint32_t d0, uint32_t d1) {
  float f[8];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f[i] = (float)(int8_t)(d0 >> (8 * i));
    f[4 + i] = (float)(int8_t)(d1 >> (8 * i));
  }
  i32x4 o;
  if constexpr (XT == XLA_AMD_DT_BF16) {
    o[0] = pack_hi16(f[0], f[1]); o[1] = pack_hi16(f[2], f[3]);
    o[2] = pack_hi16(f[4], f[5]); o[3] = pack_hi16(f[6], f[7]);
  } else {
    o[0] = pack_f16(f[0], f[1]); o[1] = pack_f16(f[2], f[3]);
    o[2] = pack_f16(f[4], f[5]); o[3] = pack_f16(f[6], f[7]);
  }
  return o;
}

// 8 packed int4 weights (one dword, nibble j = column P[j] + 8 biased) -> 8
// elements (1 + u/16) of the x dtype, u = w + 8 in 0..15.  The caller undoes
// the affine map with the exact x sum: sum w*x = 16*(sum a*x - 1.5*sum x).
template <int XT>
__device__ __forceinline__ i32x4 cvt_w4(uint32_t d) {
  i32x4 o;
  if constexpr (XT == XLA_AMD_DT_BF16) {
    const uint32_t mask = 0x00780078u, one = 0x3F803F80u;  // mantissa bits 3..6 of bf16
    o[0] = ((d << 3) & mask) | one;
    o[1] = ((d >> 1) & mask) | one;
    o[2] = ((d >> 5) & mask) | one;
    o[3] = ((d >> 9) & mask) | one;
  } else {
    const uint32_t mask = 0x03C003C0u, one = 0x3C003C00u;  // mantissa bits 6..9 of f16
    o[0] = ((d << 6) & mask) | one;
    o[1] = ((d << 2) & mask) | one;
    o[2] = ((d >> 2) & mask) | one;
    o[3] = ((d >> 6) & mask) | one;
  }
  return o;
}

template <int XT>
__device__ __forceinline__ f32x4 mfma16(i32x4 a, i32x4 b, f32x4 c) {
  if constexpr (XT == XLA_AMD_DT_BF16)
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

template <int XT> __device__ __forceinline__ i32x4 ones_frag() {
  uint32_t one2 = XT == XLA_AMD_DT_BF16 ? 0x3F803F80u : 0x3C003C00u;
  i32x4 o = {(int)one2, (int)one2, (int)one2, (int)one2};
  return o;
}

struct SkinnyArgs {
  const void* x;
  const uint8_t* w;  // K-major packed weight
  const void* scale;
  const void* zp;
  void* out;
  int M, N, K, C;  // M = rows of this pass (<= 16*MT)
  int scale_dt, zp_dt, out_dt;
};

// XT: dtype of x.  BITS: 8 or 4.  MT: 16-row tiles of x.  RG: 16-channel
// groups per wave.  D: k-iterations whose loads are in flight per wave (a
// register ring: iteration j lives in stage j % D).  PERCH: per-channel
// (C == K): waves interleave over k and raw dot products are reduced;
// otherwise each wave owns whole blocks and the reduction is over scaled block
// results.  HASZP: a zero point is given.
template <int XT, int BITS, int MT, int RG, int D, bool PERCH, bool HASZP>
__global__ void __launch_bounds__(kWaves * 64)
qmm_skinny_kernel(SkinnyArgs a) {
  constexpr bool kMfma = XT != XLA_AMD_DT_F32;
  constexpr bool NEEDXS = HASZP || (BITS == 4 && kMfma);  // x sums: zero point, int4 affine map
  constexpr int kSlots = RG * MT * 4;                 // accumulators per lane
  constexpr int kXsSlots = NEEDXS ? MT : 0;           // x sums per lane (PERCH reduce)
  constexpr int kRedSlots = PERCH ? kSlots + kXsSlots : (HASZP ? 2 * kSlots : kSlots);
  constexpr int WQ = BITS == 8 ? 2 : 1;               // 16-byte weight loads per lane per iteration
  constexpr int XQ = kMfma ? 4 : 8;                   // 16-byte x loads per lane per iteration
  __shared__ float red[kWaves][kRedSlots][64];

  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int n_base = blockIdx.x * (16 * RG);
  const int K = a.K, N = a.N, M = a.M;
  const int x_dt = XT;

  // Row pointers (clamped so that tail lanes read valid memory; their results
  // are never stored).
  const uint8_t* wrow[RG];
#pragma unroll
  for (int rg = 0; rg < RG; ++rg) {
    int n = min(n_base + 16 * rg + r, N - 1);
    wrow[rg] = a.w + (size_t)n * (BITS == 8 ? (size_t)K : (size_t)K / 2) + (BITS == 8 ? 32 * g : 16 * g);
  }
  const char* xrow[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    int m = min(16 * mt + r, M - 1);
    xrow[mt] = (const char*)a.x + ((size_t)m * K + 32 * g) * (XT == XLA_AMD_DT_F32 ? 4 : 2);
  }

  f32x4 acc[RG][MT];
  f32x4 xs[MT];
  f32x4 sacc[RG][MT], zacc[RG][MT];
#pragma unroll
  for (int rg = 0; rg < RG; ++rg)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      acc[rg][mt] = f32x4{0, 0, 0, 0};
      sacc[rg][mt] = f32x4{0, 0, 0, 0};
      zacc[rg][mt] = f32x4{0, 0, 0, 0};
    }
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) xs[mt] = f32x4{0, 0, 0, 0};

  // Iteration j of this wave -> first column k0.  Per-channel: iterations are
  // dealt round-robin to the waves.  Blockwise: blocks are dealt round-robin
  // and a wave walks its block's C/128 iterations consecutively.
  const int ipb = PERCH ? 1 : a.C / kKIter;  // iterations per block
  const int units = PERCH ? K / kKIter : K / a.C;     // iterations resp. blocks in total
  const int my_units = units > wv ? (units - wv + kWaves - 1) / kWaves : 0;
  const int n_it = my_units * ipb;
  // Workgroups start at different k (rotation `rot`): rows are K bytes apart,
  // so without it every wave of the grid would begin in the same few hundred
  // bytes of each row and crowd the same memory channels.
  const int rot = (int)((blockIdx.x * 5u) % (unsigned)units);
  auto unit_of = [&](int u) -> int {  // u-th unit of this wave -> global unit index
    int t = wv + u * kWaves + rot;
    return t >= units ? t - units : t;
  };
  auto k0_of = [&](int j) -> int {
    if constexpr (PERCH) return unit_of(j) * kKIter;
    const int b = j / ipb, i = j - b * ipb;
    return unit_of(b) * a.C + i * kKIter;
  };

  // Register ring of D stages.
  i32x4 wq[D][RG][WQ];
  i32x4 xq[D][MT][XQ];
  auto load_stage = [&](auto dc, int j) {
    constexpr int d = dc;
    const int k0 = k0_of(j);
#pragma unroll
    for (int rg = 0; rg < RG; ++rg) {
      const i32x4* p = (const i32x4*)(wrow[rg] + (BITS == 8 ? k0 : k0 / 2));
#pragma unroll
      for (int q = 0; q < WQ; ++q) wq[d][rg][q] = __builtin_nontemporal_load(p + q);
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const i32x4* p = (const i32x4*)(xrow[mt] + (size_t)k0 * (XT == XLA_AMD_DT_F32 ? 4 : 2));
#pragma unroll
      for (int q = 0; q < XQ; ++q) xq[d][mt][q] = p[q];
    }
  };

  auto compute_stage = [&](auto dc) {
    constexpr int d = dc;
    if constexpr (kMfma) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
#pragma unroll
        for (int rg = 0; rg < RG; ++rg) {
          i32x4 af;
          if constexpr (BITS == 8)
            af = cvt_w8<XT>((uint32_t)wq[d][rg][j >> 1][(j & 1) * 2], (uint32_t)wq[d][rg][j >> 1][(j & 1) * 2 + 1]);
          else
            af = cvt_w4<XT>((uint32_t)wq[d][rg][0][j]);
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) acc[rg][mt] = mfma16<XT>(af, xq[d][mt][j], acc[rg][mt]);
        }
        if constexpr (NEEDXS) {
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) xs[mt] = mfma16<XT>(ones_frag<XT>(), xq[d][mt][j], xs[mt]);
        }
      }
    } else {
      // f32 x: 16x16x4 f32 MFMA, one k per lane per instruction.
#pragma unroll
      for (int kk = 0; kk < 32; ++kk) {  // 0..31 within the lane's columns
#pragma unroll
        for (int rg = 0; rg < RG; ++rg) {
          float wf;
          if constexpr (BITS == 8) {
            uint32_t dw = (uint32_t)wq[d][rg][kk >> 4][(kk >> 2) & 3];
            wf = (float)(int8_t)(dw >> (8 * (kk & 3)));
          } else {
            // column kk = 8*word + P[nibble]: nibble = (c&1)*4 + (c>>1), c = kk % 8
            uint32_t dw = (uint32_t)wq[d][rg][0][kk >> 3];
            int c = kk & 7, nib = (c & 1) * 4 + (c >> 1);
            wf = (float)(int)((dw >> (4 * nib)) & 15u) - 8.0f;
          }
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
            acc[rg][mt] = __builtin_amdgcn_mfma_f32_16x16x4f32(
                wf, __builtin_bit_cast(float, xq[d][mt][kk >> 2][kk & 3]), acc[rg][mt], 0, 0, 0);
        }
        if constexpr (NEEDXS) {
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
            xs[mt] = __builtin_amdgcn_mfma_f32_16x16x4f32(
                1.0f, __builtin_bit_cast(float, xq[d][mt][kk >> 2][kk & 3]), xs[mt], 0, 0, 0);
        }
      }
    }
  };

  // Undo the int4 affine map (MFMA path only): dot = 16 * (acc - 1.5 * xsum).
  auto true_dot = [&](float accv, float xsv) -> float {
    if constexpr (BITS == 4 && kMfma) return 16.0f * (accv - 1.5f * xsv);
    return accv;
  };

  // Block epilogue (blockwise only): p = round_x(dot); sacc += scale[s,n] * p;
  // zacc += round_x(xsum) * zp[s,n]; then the block accumulators restart.
  auto block_epilogue = [&](int sblk) {
#pragma unroll
    for (int rg = 0; rg < RG; ++rg)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        int n = min(n_base + 16 * rg + 4 * g + v, N - 1);
        float sc = qmm_load(a.scale, (int64_t)sblk * N + n, a.scale_dt);
        float zv = 0.f;
        if constexpr (HASZP) zv = qmm_load(a.zp, (int64_t)sblk * N + n, a.zp_dt);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          float xsv = NEEDXS ? xs[mt][v] : 0.f;
          float p = qmm_round_dt(true_dot(acc[rg][mt][v], xsv), x_dt);
          sacc[rg][mt][v] = fmaf(sc, p, sacc[rg][mt][v]);
          if constexpr (HASZP) zacc[rg][mt][v] = fmaf(qmm_round_dt(xsv, x_dt), zv, zacc[rg][mt][v]);
        }
      }
#pragma unroll
    for (int rg = 0; rg < RG; ++rg)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) acc[rg][mt] = f32x4{0, 0, 0, 0};
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) xs[mt] = f32x4{0, 0, 0, 0};
  };

  // Software pipeline: D iterations of loads stay in flight.
  qmm_static_for<D>([&](auto dc) {
    if (dc < n_it) load_stage(dc, dc);
  });
  for (int j0 = 0; j0 < n_it; j0 += D) {
    qmm_static_for<D>([&](auto dc) {
      const int j = j0 + dc;
      if (j < n_it) {
        compute_stage(dc);
        if (j + D < n_it) load_stage(dc, j + D);
        if constexpr (!PERCH) {
          if ((j + 1) % ipb == 0) block_epilogue(unit_of(j / ipb));
        }
      }
    });
  }

  if constexpr (PERCH) {
    // Reduce raw partial sums over the waves.
#pragma unroll
    for (int rg = 0; rg < RG; ++rg)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int v = 0; v < 4; ++v) red[wv][(rg * MT + mt) * 4 + v][lane] = acc[rg][mt][v];
    if constexpr (NEEDXS) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) red[wv][kSlots + mt][lane] = xs[mt][0];
    }
  } else {
#pragma unroll
    for (int rg = 0; rg < RG; ++rg)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          red[wv][(rg * MT + mt) * 4 + v][lane] = sacc[rg][mt][v];
          if constexpr (HASZP) red[wv][kSlots + (rg * MT + mt) * 4 + v][lane] = zacc[rg][mt][v];
        }
  }
  __syncthreads();

  // Final epilogue: thread (wv, lane) finishes slots wv, wv + kWaves, ...
  const int zpo_dt = qmm_promote(x_dt, a.zp_dt);
  for (int slot = wv; slot < kSlots; slot += kWaves) {
    int v = slot & 3, mt = (slot >> 2) % MT, rg = (slot >> 2) / MT;
    int n = n_base + 16 * rg + 4 * g + v;
    int m = 16 * mt + r;
    float tot = 0.f, aux = 0.f;
#pragma unroll
    for (int w2 = 0; w2 < kWaves; ++w2) tot += red[w2][slot][lane];
    float o;
    if constexpr (PERCH) {
      if constexpr (NEEDXS) {
#pragma unroll
        for (int w2 = 0; w2 < kWaves; ++w2) aux += red[w2][kSlots + mt][lane];
      }
      if (n >= N || m >= M) continue;
      float p = qmm_round_dt(true_dot(tot, aux), x_dt);
      o = qmm_round_dt(p * qmm_load(a.scale, n, a.scale_dt), a.out_dt);
      if constexpr (HASZP) {
        float z = qmm_round_dt(qmm_round_dt(aux, x_dt) * qmm_load(a.zp, n, a.zp_dt), zpo_dt);
        o = qmm_round_dt(o - z, a.out_dt);
      }
    } else {
      if constexpr (HASZP) {
#pragma unroll
        for (int w2 = 0; w2 < kWaves; ++w2) aux += red[w2][kSlots + slot][lane];
      }
      if (n >= N || m >= M) continue;
      o = qmm_round_dt(tot, a.out_dt);
      if constexpr (HASZP) o = qmm_round_dt(o - qmm_round_dt(aux, zpo_dt), a.out_dt);
    }
    qmm_store(a.out, (int64_t)m * N + n, o, a.out_dt);
  }
}

#ifndef QMM_SKINNY_RG
#define QMM_SKINNY_RG 1
#endif
#ifndef QMM_SKINNY_D
#define QMM_SKINNY_D 0
#endif

// Pipeline depth: as many iterations in flight as ~150 VGPRs of staging allow.
constexpr int pipeline_depth(int xt, int mt) {
  if (QMM_SKINNY_D > 0) return QMM_SKINNY_D;
  if (xt == XLA_AMD_DT_F32) return mt <= 2 ? 2 : 1;
  return mt == 1 ? 4 : (mt == 2 ? 3 : 2);
}

template <int XT, int BITS, int MT, bool PERCH, bool HASZP>
int launch_rg(const SkinnyArgs& a, hipStream_t stream) {
  constexpr int RG = QMM_SKINNY_RG;
  constexpr int D = pipeline_depth(XT, MT);
  unsigned blocks = (unsigned)((a.N + 16 * RG - 1) / (16 * RG));
  hipLaunchKernelGGL((qmm_skinny_kernel<XT, BITS, MT, RG, D, PERCH, HASZP>), dim3(blocks),
                     dim3(kWaves * 64), 0, stream, a);
  return QMM_CHECK_LAUNCH("weight_only_skinny launch");
}

template <int XT, int BITS, int MT>
int launch_mode(const SkinnyArgs& a, bool perch, bool haszp, hipStream_t stream) {
  if (perch) return haszp ? launch_rg<XT, BITS, MT, true, true>(a, stream) : launch_rg<XT, BITS, MT, true, false>(a, stream);
  return haszp ? launch_rg<XT, BITS, MT, false, true>(a, stream) : launch_rg<XT, BITS, MT, false, false>(a, stream);
}

template <int XT, int BITS>
int launch_mt(const SkinnyArgs& a, bool perch, bool haszp, hipStream_t stream) {
  if (a.M <= 16) return launch_mode<XT, BITS, 1>(a, perch, haszp, stream);
  if (a.M <= 32) return launch_mode<XT, BITS, 2>(a, perch, haszp, stream);
  return launch_mode<XT, BITS, 4>(a, perch, haszp, stream);
}

template <int XT>
int launch_bits(const SkinnyArgs& a, int bits, bool perch, bool haszp, hipStream_t stream) {
  return bits == 8 ? launch_mt<XT, 8>(a, perch, haszp, stream) : launch_mt<XT, 4>(a, perch, haszp, stream);
}

}  // namespace

extern "C" int xla_amd_qmm_weight_only_skinny(const void* x, const void* w_packed, const void* scale,
                                              const void* zp, void* out, int64_t M, int64_t N,
                                              int64_t K, int64_t C, int bits, int x_dt, int scale_dt,
                                              int zp_dt, int out_dt, void* stream) {
  if (!x || !w_packed || !scale || !out) return qmm_fail(XLA_AMD_QMM_EINVAL, "weight_only_skinny: null pointer");
  if (M < 0 || N <= 0 || K <= 0 || C <= 0 || K % C != 0)
    return qmm_fail(XLA_AMD_QMM_EINVAL, "weight_only_skinny: bad sizes M=%lld N=%lld K=%lld C=%lld",
                    (long long)M, (long long)N, (long long)K, (long long)C);
  if (bits != 4 && bits != 8) return qmm_fail(XLA_AMD_QMM_EINVAL, "weight_only_skinny: bits must be 4 or 8");
  if (!qmm_valid_dt(x_dt) || !qmm_valid_dt(scale_dt) || !qmm_valid_dt(out_dt) || (zp && !qmm_valid_dt(zp_dt)))
    return qmm_fail(XLA_AMD_QMM_EINVAL, "weight_only_skinny: bad dtype enum");
  if (out_dt != qmm_promote(x_dt, scale_dt))
    return qmm_fail(XLA_AMD_QMM_EINVAL, "weight_only_skinny: out dtype must be promote(x, scale)");
  if (K % kKIter != 0 || C % kKIter != 0)
    return qmm_fail(XLA_AMD_QMM_EUNSUPPORTED, "weight_only_skinny: K=%lld and C=%lld must be multiples of %d",
                    (long long)K, (long long)C, kKIter);
  if (N > (1 << 30) || K > (1 << 30) || M > (1 << 30))
    return qmm_fail(XLA_AMD_QMM_EUNSUPPORTED, "weight_only_skinny: dimension too large");
  if (((uintptr_t)x | (uintptr_t)w_packed) & 15)
    return qmm_fail(XLA_AMD_QMM_EUNSUPPORTED, "weight_only_skinny: x and w must be 16-byte aligned");
  if (M == 0) return XLA_AMD_QMM_OK;
  const bool perch = (C == K);
  const int xsz = qmm_dt_size(x_dt), osz = qmm_dt_size(out_dt);
  // Up to 64 rows of x per pass over the weight.
  for (int64_t m0 = 0; m0 < M; m0 += 64) {
    SkinnyArgs a;
    a.x = (const char*)x + (size_t)m0 * K * xsz;
    a.w = (const uint8_t*)w_packed;
    a.scale = scale;
    a.zp = zp;
    a.out = (char*)out + (size_t)m0 * N * osz;
    a.M = (int)((M - m0) < 64 ? (M - m0) : 64);
    a.N = (int)N; a.K = (int)K; a.C = (int)C;
    a.scale_dt = scale_dt; a.zp_dt = zp ? zp_dt : x_dt; a.out_dt = out_dt;
    int rc;
    if (x_dt == XLA_AMD_DT_BF16) rc = launch_bits<XLA_AMD_DT_BF16>(a, bits, perch, zp != nullptr, (hipStream_t)stream);
    else if (x_dt == XLA_AMD_DT_F16) rc = launch_bits<XLA_AMD_DT_F16>(a, bits, perch, zp != nullptr, (hipStream_t)stream);
    else rc = launch_bits<XLA_AMD_DT_F32>(a, bits, perch, zp != nullptr, (hipStream_t)stream);
    if (rc != XLA_AMD_QMM_OK) return rc;
  }
  return XLA_AMD_QMM_OK;
}
