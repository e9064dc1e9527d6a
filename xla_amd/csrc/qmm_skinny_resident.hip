// Weight-streaming GEMV for outputs of more than one round of channel groups: persistent waves
// with all of x resident in LDS.
//
// The weight-streaming kernel of qmm_skinny.hip gives every wave one channel group; a launch
// with more groups than the chip has wave slots (1024 = 256 compute units x 4 computing waves)
// runs in rounds of workgroups, and every round pays the kernel's prologue again: the first,
// cold weight loads, the copy of x into LDS, the meetings of the workgroup.  Here one workgroup
// per compute unit stays: each of its four computing waves owns a contiguous run of channel
// groups - a contiguous region of the tiled weight - and streams through it without a break
// (the register ring of weight loads simply runs on from one group into the next), while x,
// up to 16 rows x K columns of 2-byte activations (at most 144 KB), is copied into LDS once
// and stays.  Per-channel int8 weights, scale / zero point / result of x's dtype, K a multiple
// of 512, N even.
//
// Arithmetic, MFMA mapping and rounding points are those of qmm_skinny.hip (per-channel case):
//   p = round_x(sum_k x*w); out = round_x(scale * p);
//   zero point: out = round_x(out - round_x(round_x(sum_k x) * zp)).
// A group of G channels (xla_amd_qmm_tile_group) occupies MFMA rows 0 .. G-1; rows from G on
// read the group's last row again and their results are dropped.
//
// This file is compiled once per activation dtype (-DQMM_SKINNY_XT=1|2).
#include "qmm_common.h"

#ifndef QMM_SKINNY_XT
#error "compile with -DQMM_SKINNY_XT=<XLA_AMD_DT_BF16|XLA_AMD_DT_F16 value>"
#endif

#include "qmm_frag.h"
#include "qmm_skinny.h"

namespace {

using namespace qmm_frag;

#ifndef QMM_RESIDENT_WAVES
#define QMM_RESIDENT_WAVES 4
#endif
constexpr int kWaves = QMM_RESIDENT_WAVES;      // computing waves per workgroup
constexpr int kCopiers = 4;    // waves that copy x (and the scales) into LDS
constexpr int kKS = 512;       // columns per step
constexpr int kSub = 4;        // 128-column sub-steps per step
constexpr int kXRow = kKS * 2; // bytes of one x row per step
constexpr int kXTile = 16 * kXRow;
constexpr int kNld = 8;        // 1 KB weight loads per wave and step (the ring: one step in flight)
constexpr int kChunk = 4;      // x tiles (steps) per copy chunk: the workgroup meets once per chunk while x arrives

template <int XT, bool HASZP>
__global__ void __launch_bounds__((kWaves + kCopiers) * 64)
qmm_skinny_resident_kernel(SkinnyArgs a) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  typedef __attribute__((address_space(3))) void* lds_ptr_t;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r = lane & 15, g = lane >> 4;
  const int N = a.N, K = a.K, M = a.M, G = a.G;
  const int steps = K / kKS;
  const int n_chunks = (steps + kChunk - 1) / kChunk;
  const int groups = (N + G - 1) / G;
  // channel groups of this workgroup and of each of its computing waves: contiguous, balanced to one group
  const int n_waves = (int)gridDim.x * kWaves;
  auto first_group = [&](int w) { return (int)((int64_t)w * groups / n_waves); };
  const int wg_g0 = first_group((int)blockIdx.x * kWaves), wg_g1 = first_group((int)blockIdx.x * kWaves + kWaves);
  const int wg_ch0 = wg_g0 * G;                       // first channel of the workgroup (even)
  // LDS: [x: steps tiles][scales of the workgroup's channels][zero points]
  char* const xsm = smem;
  constexpr int SE = 2;
  char* const scl = smem + steps * kXTile;
  const int scl_bytes = ((wg_g1 - wg_g0) * G * SE + 255) & ~255;
  char* const zpl = scl + scl_bytes;

  if (__builtin_expect(wave >= kWaves, 0)) {
    // ---- copying waves: the scales, then x chunk after chunk; the workgroup meets after each chunk ----
    const int cw = wave - kWaves;
    const int x_rows = min(M, 16);
    // scales / zero points: 4 bytes (two channels) per lane and instruction, 256 bytes per instruction
    for (int i = cw; i * 256 < scl_bytes * (HASZP ? 2 : 1); i += kCopiers) {
      const bool is_zp = i * 256 >= scl_bytes;
      const int off = (is_zp ? i * 256 - scl_bytes : i * 256) + lane * 4;
      int ch = wg_ch0 + off / SE;
      if (ch + 2 > N) ch = N - 2;  // past the last channel: any valid address (never used)
      const char* src = (const char*)(is_zp ? a.zp : a.scale) + (size_t)ch * SE;
      char* dst = (is_zp ? zpl : scl) + (is_zp ? i * 256 - scl_bytes : i * 256);
      __builtin_amdgcn_global_load_lds((const void*)src, (lds_ptr_t)dst, 4, 0, 0);
    }
    for (int c = 0; c < n_chunks; ++c) {
      const int t0 = c * kChunk, t1 = min(steps, t0 + kChunk);
      for (int row = cw; row < x_rows; row += kCopiers) {
        const char* xrow = (const char*)a.x + (size_t)row * ((size_t)K * 2);
        const uint32_t col = (uint32_t)((lane ^ (row & 15)) * 16);  // LDS slot l of a row holds the row's 16-byte piece l ^ (row % 16)
        for (int t = t0; t < t1; ++t)
          __builtin_amdgcn_global_load_lds((const void*)(xrow + (size_t)t * kXRow + col),
                                           (lds_ptr_t)(xsm + t * kXTile + row * kXRow), 16, 0, 0);
      }
      __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's copies have landed
      qmm_bare_barrier();                  // chunk c is there
    }
    return;
  }

  // ---- computing waves ----
  const int wave_id = (int)blockIdx.x * kWaves + wave;
  const int g_begin = first_group(wave_id), g_end = first_group(wave_id + 1);
  const int n_blk = K / 128;
  const int blk_bytes = G * 128, half_bytes = G * 64;
  const int64_t last_blk = (int64_t)max(g_end - g_begin, 1) * n_blk - 1;  // of this wave's region
  const uint8_t* const w_base = a.w + (size_t)min(g_begin, groups - 1) * n_blk * blk_bytes + (g * G + min(r, G - 1)) * 16;
  i32x4 wreg[kNld];
  // the fragments of sub-step t of the wave's step `lin` (steps counted through all its groups); past the
  // end of the region the last block is read again (loaded to keep the loads in flight the same, never used)
  auto load_sub = [&](int64_t lin, auto tc) __attribute__((always_inline)) {
    constexpr int t = tc;
    int64_t blk = lin * kSub + t;
    blk = blk < last_blk ? blk : last_blk;
    const uint8_t* const wp = w_base + blk * blk_bytes;
    wreg[2 * t] = __builtin_nontemporal_load((const i32x4*)wp);
    wreg[2 * t + 1] = __builtin_nontemporal_load((const i32x4*)(wp + half_bytes));
  };
  qmm_static_for<kSub>([&](auto tc) { load_sub(0, tc); });
  __builtin_amdgcn_sched_barrier(0);

  f32x4 acc, accb, xs;
  // one step: the ring's weights against x tile s; every sub-step's registers are re-loaded with the same
  // sub-step of the next step as soon as they have been used
  auto step = [&](int s, int64_t lin) __attribute__((always_inline)) {
    const char* xb = xsm + s * kXTile + r * kXRow;
    auto read_frags = [&](auto tc, i32x4 (&xq)[4]) __attribute__((always_inline)) {
      constexpr int t = tc;
      qmm_static_for<4>([&](auto qc) {
        constexpr int q = qc;
        xq[q] = *(const i32x4*)(xb + (((16 * t + 4 * g + q) ^ r) * 16));
      });
    };
    i32x4 xq[2][4];
    read_frags(qmm_const<0>{}, xq[0]);
    qmm_static_for<kSub>([&](auto tc) {
      constexpr int t = tc;
      constexpr int cur = t & 1, nxt = cur ^ 1;
      if constexpr (t + 1 < kSub) read_frags(qmm_const<t + 1>{}, xq[nxt]);
      __builtin_amdgcn_sched_barrier(0);
      qmm_static_for<4>([&](auto jc) {
        constexpr int j = jc;
        const i32x4 src = (j >> 1) ? wreg[2 * t + 1] : wreg[2 * t];
        const i32x4 af = cvt_w8<XT>((uint32_t)src[(j & 1) * 2], (uint32_t)src[(j & 1) * 2 + 1]);
        if constexpr (j & 1) accb = mfma16<XT>(af, xq[cur][j], accb);
        else acc = mfma16<XT>(af, xq[cur][j], acc);
        if constexpr (HASZP) xs = mfma16<XT>(ones_frag<XT>(), xq[cur][j], xs);
      });
      load_sub(lin + 1, tc);
      __builtin_amdgcn_sched_barrier(0);
    });
  };

  qmm_bare_barrier();  // the first chunk of x (and the scales) is there
  int chunks_seen = 1;
  int64_t lin = 0;
  for (int grp = g_begin; grp < g_end; ++grp) {
    acc = f32x4{0, 0, 0, 0};
    accb = f32x4{0, 0, 0, 0};
    xs = f32x4{0, 0, 0, 0};
    // The group's first step stands outside the loop: it follows the previous group's stores in straight-line
    // code, so the compiler counts them and its waits for the ring stay exact; in a loop their count would be
    // merged with the loop's own and every group would begin with a wait for its predecessor's stores.
    step(0, lin);
    ++lin;
    for (int s = 1; s < steps; ++s, ++lin) {
      if (chunks_seen < n_chunks && s == chunks_seen * kChunk) {  // (first group only: x is still arriving)
        qmm_bare_barrier();
        ++chunks_seen;
      }
      step(s, lin);
    }
    // ---- the group's results: lane (r, g) holds row r of x, channels G grp + 4g .. + 3 ----
    const int n = grp * G + 4 * g;
    const int cnt = min(min(G - 4 * g, N - n), 4);  // channels of this lane that exist (<= 0: none)
    if (r < M && cnt > 0) {
      const char* sc = scl + (n - wg_ch0) * SE;
      const char* zc = zpl + (n - wg_ch0) * SE;
      const float xsum = HASZP ? qmm_round_dt(xs[0], XT) : 0.f;
      float res4[4];
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const float p = qmm_round_dt(acc[v] + accb[v], XT);
        float res = qmm_round_dt(qmm_from_raw(*(const uint16_t*)(sc + min(v, cnt - 1) * SE), XT) * p, XT);
        if constexpr (HASZP) {
          const float z = qmm_round_dt(xsum * qmm_from_raw(*(const uint16_t*)(zc + min(v, cnt - 1) * SE), XT), XT);
          res = qmm_round_dt(res - z, XT);
        }
        res4[v] = res;
      }
      // two channels per store (n and N are even), four where the lane's channels are four-aligned
      uint16_t* o = (uint16_t*)a.out + (size_t)r * N + n;
      const uint32_t lo = XT == XLA_AMD_DT_BF16 ? qmm_f32x2_to_bf16x2(res4[0], res4[1]) : qmm_f32x2_to_f16x2(res4[0], res4[1]);
      const uint32_t hi = XT == XLA_AMD_DT_BF16 ? qmm_f32x2_to_bf16x2(res4[2], res4[3]) : qmm_f32x2_to_f16x2(res4[2], res4[3]);
      if (cnt == 4 && ((N | n) & 3) == 0) {
        *(i32x2*)o = i32x2{(int)lo, (int)hi};
      } else {
        if (cnt >= 2) *(uint32_t*)o = lo;
        else o[0] = (uint16_t)lo;
        if (cnt == 4) *(uint32_t*)(o + 2) = hi;
        else if (cnt == 3) o[2] = (uint16_t)hi;
      }
    }
  }
  // (a launch with fewer steps than chunks to wait for, or a wave without groups: the meetings still take place)
  for (; chunks_seen < n_chunks; ++chunks_seen) qmm_bare_barrier();
}

template <int XT>
int launch(const SkinnyArgs& a, bool haszp, int workgroups, hipStream_t stream) {
  const int steps = a.K / kKS;
  const int groups = (a.N + a.G - 1) / a.G;
  // scales (and zero points) of the most channels a workgroup can get
  const int per_wg = ((groups + workgroups - 1) / workgroups + kWaves) * a.G;
  const int scl_bytes = (per_wg * 2 + 255) & ~255;
  const int lds = steps * kXTile + scl_bytes * (haszp ? 2 : 1);
  auto go = [&](auto kern) -> int {
    static std::atomic<uint64_t> lds_set{0};
    const int rc = qmm_set_max_lds((const void*)kern, 160 * 1024, lds_set, "weight_only_skinny (resident) hipFuncSetAttribute");
    if (rc != XLA_AMD_QMM_OK) return rc;
    hipLaunchKernelGGL(kern, dim3((unsigned)workgroups), dim3((kWaves + kCopiers) * 64), lds, stream, a);
    return QMM_CHECK_LAUNCH("weight_only_skinny (resident) launch");
  };
  return haszp ? go(qmm_skinny_resident_kernel<XT, true>) : go(qmm_skinny_resident_kernel<XT, false>);
}

}  // namespace

#if QMM_SKINNY_XT == XLA_AMD_DT_BF16
// Whether a launch can take this kernel, and with how many workgroups (0: it cannot).
int qmm_skinny_resident_workgroups(const SkinnyArgs& a, int x_dt, int bits) {
  if (bits != 8 || a.C != a.K || a.slices != 1 || a.M > 16 || (x_dt != XLA_AMD_DT_BF16 && x_dt != XLA_AMD_DT_F16)) return 0;
  if (a.scale_dt != x_dt || a.zp_dt != x_dt || a.out_dt != x_dt || a.dot_dt != x_dt || a.store_dt != x_dt) return 0;
  if (a.K % kKS != 0 || (a.N & 1) != 0) return 0;
  const int steps = a.K / kKS;
  const int groups = (a.N + a.G - 1) / a.G;
  constexpr int kWorkgroups = 256;  // one per compute unit
  // Up to two groups per wave slot the kernel of qmm_skinny.hip is as fast or faster (one round of four or of
  // eight one-group waves per workgroup; 28672 x 4096 at M = 16, cold: 21.1 us against 21.7 here); from there on
  // the rounds' prologues add up (128256 x 4096: M = 1 91.7 -> 84 us, M = 16 95 -> 91).
  if (groups <= kWorkgroups * 8) return 0;
  const int per_wg = ((groups + kWorkgroups - 1) / kWorkgroups + kWaves) * a.G;
  const int scl_bytes = (per_wg * 2 + 255) & ~255;
  if (steps * kXTile + 2 * scl_bytes > 160 * 1024) return 0;
  return kWorkgroups;
}
#endif

#if QMM_SKINNY_XT == XLA_AMD_DT_F16
int qmm_skinny_resident_launch_f16(const SkinnyArgs& a, bool haszp, int workgroups, hipStream_t stream) {
  return launch<XLA_AMD_DT_F16>(a, haszp, workgroups, stream);
}
#else
int qmm_skinny_resident_launch_bf16(const SkinnyArgs& a, bool haszp, int workgroups, hipStream_t stream) {
  return launch<XLA_AMD_DT_BF16>(a, haszp, workgroups, stream);
}
#endif
