// Weight-only quantized matmul for many rows of x: a tiled bf16/f16 MFMA GEMM whose B
// operand is the int8 weight, converted to x's dtype in registers (exact).
//
// The weight-streaming kernel (qmm_skinny.hip) keeps up to 32 rows of x per pass and
// re-reads the whole weight for every further 32 rows; its workgroups also each copy all
// of x, which for a long K and few output channels is several times the weight itself.
// This kernel covers those cases: a workgroup owns a tile of 16*MT rows x 64*NG channels,
// every weight fragment is used against all row tiles from registers, and K can be split
// over workgroups (each then copies only its slice of x); the partial sums of a split
// go to a workspace and a second kernel adds them in a fixed order and finishes them.
//
// Operands.  Weights come from the tiled copy (xla_amd_qmm_tile_weight): per group of G <= 16 channels and 128
// columns one block, already in MFMA operand order, so a wave loads its fragments straight into registers: no
// LDS traffic and no transposition for weights.  An MFMA row set is 16 consecutive channels whatever G is
// (channel n = row n % G of group n / G; every lane keeps the offset of its row, the base is scalar), so the
// kernel wastes no MFMA rows on groups narrower than 16.  Per row set a wave keeps a ring of three or five half
// blocks (64 columns) in registers and asks for a half again as soon as it has been used.
// x goes through LDS: the workgroup's rows, one step (128 columns) per tile, in a ring of 3 to 8 tiles (what
// fits); four extra waves copy (global -> LDS without registers) up to R - 1 tiles ahead of the four computing
// waves, and the workgroup meets once per step.  (The computing waves must not issue such copies themselves: with
// copies in flight the compiler can no longer count their register loads in flight and turns every wait of the
// loop into a wait for all of them.)  The 128 x 256 tile's results leave through LDS as well: the computing waves
// put the rounded dot products there and go on, the copying waves scale them and write them out meanwhile.
//
// MFMA mapping (v_mfma_f32_16x16x32_bf16/f16, A = weights, B = x^T), as in the streaming
// kernel: lane l is (r = l%16, g = l/16); for a block of 128 columns the lane supplies, for
// weight channel r and for x row r of each 16-row tile, the columns 32g..32g+31 as four
// instructions of 8 columns each.  D[i][j] lands in lane (j + 16*(i/4)), register i%4:
// channel 4g + v, x row r: four consecutive channels of one row per lane.
//
// Arithmetic: the reference's per-channel sequence with its rounding points
//   p = round_dot(sum_k x*w); out = round_out(scale * p);
//   zero point: out = round_out(out - round_zpo(round_x(sum_k x) * zp)); stored as store_dt.
//
// This file is compiled once per (activation dtype, row tile) pair (-DQMM_WO_XT=1|2 for bf16 | f16,
// -DQMM_WO_MT=4|8) so that the units build in parallel; the unit of bf16 with MT = 8 also
// holds the second kernel of a K split and the C entry points.
#include "qmm_common.h"
#include "qmm_frag.h"
#include "qmm_skinny.h"
#include "qmm_wo_bw.h"

#if !defined(QMM_WO_XT) || !defined(QMM_WO_MT)
#error "compile with -DQMM_WO_XT=<XLA_AMD_DT_BF16|XLA_AMD_DT_F16 value> -DQMM_WO_MT=<4|8>"
#endif

struct WoGemmArgs {
  const void* x;       // [M, K]
  const uint8_t* w;    // tiled weight, 8 bits
  const void* scale;   // [N]
  const void* zp;      // [N] or null
  void* out;           // [M, N] of store_dt (split == 1)
  float* part;         // [split][M][N] partial dot products (split > 1)
  float* part_xs;      // [split][M] partial row sums of x (split > 1, zero point)
  int M, N, K;
  int G;               // channels per group of the tiled weight (xla_amd_qmm_tile_group)
  int k_per_split;     // columns per K slice (a multiple of 128)
  int split;
  int scale_dt, zp_dt, dot_dt, out_dt, store_dt;
  int Kw;    // columns of the weight: K, or K / 3 when x is an f32 matrix split into three bf16 parts side by side
  int x_dt;  // the caller's x dtype (the row sums of x are rounded to it): the kernel's, or f32 for split f32 rows
  int stage_out;  // 128 x 256 tile: results leave through LDS, written out by the copying waves during the next item
};

// one launcher per unit: row tile of 16 * MT rows, ng = 2 or 4 channel groups per computing wave
int qmm_wo_launch_bf16_mt4(const WoGemmArgs& a, int ng, hipStream_t stream);
int qmm_wo_launch_bf16_mt8(const WoGemmArgs& a, int ng, hipStream_t stream);
int qmm_wo_launch_f16_mt4(const WoGemmArgs& a, int ng, hipStream_t stream);
int qmm_wo_launch_f16_mt8(const WoGemmArgs& a, int ng, hipStream_t stream);

namespace {

constexpr int kComputeWaves = 4;
constexpr int kCopyWaves = 4;
constexpr int kLds = 160 * 1024;

using namespace qmm_frag;

// Half blocks of weights (64 columns) in flight per wave and MFMA row set: a ring of registers.  A half is
// requested again as soon as it has been used, so it has (H - 1) / 2 steps to arrive.  The 128 x 256 tile
// (128 accumulator registers) has room for three, and so has the 64 x 256 tile with a zero point and dtypes
// known only at run time; the others hold five: their steps are short.
template <int MT, int NG, bool HASZP, bool UNI> constexpr int wo_ring_halves() {
  return ((MT == 8 && NG == 4) || (MT == 4 && NG == 4 && HASZP && !UNI)) ? 3 : 5;
}

template <int MT, int NG> struct WoCfg {
  static constexpr int BM = 16 * MT;
  static constexpr int X_TILE = BM * 256;  // bytes of the x columns of one step (128 columns, 2-byte x)
  // The 128 x 256 tile keeps room for its 2-byte results in LDS (64 KB): the computing waves leave them there and
  // go on with the next item, and the copying waves write them out a little per step.  Stored by the computing
  // waves themselves, the 16.8 MB that all workgroups finish at the same moment cost 6 - 8 us per item, during which
  // nothing is computed (a build without the stores: 249 -> 223 us).
  static constexpr int kStage = (MT == 8 && NG == 4) ? BM * 64 * NG * 2 : 0;
  // x tiles (one step each) in LDS: a ring that the copying waves fill R - 1 tiles ahead of the computing waves
  static constexpr int kFit = (kLds - kStage) / X_TILE;
  static constexpr int R = kFit < 8 ? kFit : 8;
  static_assert(R >= 3, "the x ring needs room to run ahead");
  static constexpr int lds_bytes(int steps) { return kStage + (steps < R ? steps : R) * X_TILE; }
};

// The dtypes of the epilogue: those of the call, or (UNI) all equal to x's dtype and known at
// compile time, which is the common case and removes every branch on a dtype.
template <int XT, bool UNI> struct WoDts {
  int scale_dt, zp_dt, dot_dt, out_dt, store_dt, x_dt;
  __device__ __forceinline__ explicit WoDts(const WoGemmArgs& a)
      : scale_dt(UNI ? XT : a.scale_dt), zp_dt(UNI ? XT : a.zp_dt), dot_dt(UNI ? XT : a.dot_dt),
        out_dt(UNI ? XT : a.out_dt), store_dt(UNI ? XT : a.store_dt), x_dt(UNI ? XT : a.x_dt) {}
};

// Scale (or zero point) of four consecutive channels as raw bits; channels past N repeat the last one.
__device__ __forceinline__ void wo_load4_raw(const void* p, int n, int N, int dt, uint32_t raw[4]) {
#pragma unroll
  for (int v = 0; v < 4; ++v) raw[v] = qmm_load_raw(p, min(n + v, N - 1), dt);
}

// The reference's epilogue for four consecutive channels of one row:
//   p = round_dot(dot); r = round_out(scale * p); with a zero point r = round_out(r - round_zpo(round_x(xsum) * zp)).
template <class Dts>
__device__ __forceinline__ void wo_finish4(const Dts& d, const uint32_t sraw[4], const uint32_t zraw[4], bool has_zp,
                                           f32x4 dot, float xsum, int x_dt, float o[4]) {
#pragma unroll
  for (int v = 0; v < 4; ++v) {
    const float p = qmm_round_dt(dot[v], d.dot_dt);
    float r = qmm_round_dt(qmm_from_raw(sraw[v], d.scale_dt) * p, d.out_dt);
    if (has_zp) {
      const int zpo_dt = qmm_promote(x_dt, d.zp_dt);
      const float z = qmm_round_dt(qmm_round_dt(xsum, x_dt) * qmm_from_raw(zraw[v], d.zp_dt), zpo_dt);
      r = qmm_round_dt(r - z, d.out_dt);
    }
    o[v] = r;
  }
}

// Stores four consecutive channels of row m starting at channel n (n % 4 == 0).  VEC: N is a
// multiple of 4, so the four channels exist and their address is aligned for one store.
template <bool VEC>
__device__ __forceinline__ void wo_store4(void* out, int m, int n, int N, const float o[4], int store_dt) {
  const size_t idx = (size_t)m * N + n;
  if constexpr (VEC) {
    if (store_dt == XLA_AMD_DT_F32) {
      *(f32x4*)((float*)out + idx) = f32x4{o[0], o[1], o[2], o[3]};
    } else {
      const bool bf = store_dt == XLA_AMD_DT_BF16;
      const uint32_t lo = bf ? qmm_f32x2_to_bf16x2(o[0], o[1]) : qmm_f32x2_to_f16x2(o[0], o[1]);
      const uint32_t hi = bf ? qmm_f32x2_to_bf16x2(o[2], o[3]) : qmm_f32x2_to_f16x2(o[2], o[3]);
      *(i32x2*)((uint16_t*)out + idx) = i32x2{(int)lo, (int)hi};
    }
  } else {
#pragma unroll
    for (int v = 0; v < 4; ++v)
      if (n + v < N) qmm_store(out, idx + v, o[v], store_dt);
  }
}

// Stores the first cnt (1 .. 4) of four consecutive channels of row m starting at channel n, n even: in
// pairs where the row length allows it (rows whose length is no multiple of 4).
__device__ __forceinline__ void wo_store_some(void* out, int m, int n, int N, int cnt, const float o[4], int store_dt) {
  const size_t idx = (size_t)m * N + n;
  if ((N & 1) == 0) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      if (cnt >= 2 * h + 2) {
        if (store_dt == XLA_AMD_DT_F32) {
          typedef float f32x2_t __attribute__((ext_vector_type(2)));
          *(f32x2_t*)((float*)out + idx + 2 * h) = f32x2_t{o[2 * h], o[2 * h + 1]};
        } else {
          *(uint32_t*)((uint16_t*)out + idx + 2 * h) = store_dt == XLA_AMD_DT_BF16 ? qmm_f32x2_to_bf16x2(o[2 * h], o[2 * h + 1])
                                                                                  : qmm_f32x2_to_f16x2(o[2 * h], o[2 * h + 1]);
        }
      } else if (cnt == 2 * h + 1) {
        qmm_store(out, idx + 2 * h, o[2 * h], store_dt);
      }
    }
  } else {
#pragma unroll
    for (int v = 0; v < 4; ++v)
      if (v < cnt) qmm_store(out, idx + v, o[v], store_dt);
  }
}

// The same epilogue and store when every dtype is bf16 and there is no zero point: two
// values per conversion, and the rounded product is already the stored bit pattern.
__device__ __forceinline__ void wo_finish_pack_bf16(const uint32_t sraw[4], f32x4 dot, uint32_t res[2]) {
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const uint32_t p = qmm_f32x2_to_bf16x2(dot[2 * h], dot[2 * h + 1]);
    const float p0 = __uint_as_float(p << 16), p1 = __uint_as_float(p & 0xffff0000u);
    res[h] = qmm_f32x2_to_bf16x2(__uint_as_float(sraw[2 * h] << 16) * p0, __uint_as_float(sraw[2 * h + 1] << 16) * p1);
  }
}
__device__ __forceinline__ void wo_finish_store_bf16(void* out, int m, int n, int N, const uint32_t sraw[4], f32x4 dot) {
  uint32_t res[2];
  wo_finish_pack_bf16(sraw, dot, res);
  *(i32x2*)((uint16_t*)out + (size_t)m * N + n) = i32x2{(int)res[0], (int)res[1]};
}

// One unit of work: a tile of rows x channels over one K slice.
struct WoItem {
  int m0, n0, ks, k_begin, steps, rows;  // n0: first channel of the column tile
};

// The kernel is persistent: workgroup b takes the work items b, b + gridDim.x, ... one after the
// other.  The ring of x tiles simply runs on across items, so the copying waves fetch the first
// tiles of the next item while the computing waves finish and store the current one, and the
// computing waves request the next item's first weights before they store.
template <int XT, int MT, int NG, bool HASZP, bool UNI>
__global__ void __launch_bounds__((kComputeWaves + kCopyWaves) * 64)
qmm_wo_gemm_kernel(WoGemmArgs a) {
  using Cfg = WoCfg<MT, NG>;
  constexpr int BM = Cfg::BM, X_TILE = Cfg::X_TILE;
  constexpr int BN = 64 * NG;  // channels per workgroup: NG MFMA row sets of 16 per computing wave
  extern __shared__ __attribute__((aligned(16))) char smem[];
  char* const ring = smem + Cfg::kStage;  // the x tiles; before them the results on their way out
  const bool stage_out = Cfg::kStage > 0 && a.stage_out != 0;
  typedef __attribute__((address_space(3))) void* lds_ptr_t;

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r = lane & 15, g = lane >> 4;
  const int M = a.M, N = a.N, K = a.K, G = a.G;
  const int tiles_n = (N + BN - 1) / BN;
  const int tiles = tiles_n * ((M + BM - 1) / BM);
  const int n_items = tiles * a.split;
  // item -> (K slice, row tile, column tile), column tiles fastest: workgroups that run together share x rows
  auto item_of = [&](int it) __attribute__((always_inline)) {
    WoItem w;
    const int tile = it % tiles;
    w.ks = it / tiles;
    w.m0 = (tile / tiles_n) * BM;
    w.n0 = (tile % tiles_n) * BN;
    w.k_begin = w.ks * a.k_per_split;
    w.steps = (min(K, w.k_begin + a.k_per_split) - w.k_begin) / 128;  // >= 1
    w.rows = min(BM, M - w.m0);  // live rows of this tile
    return w;
  };

  if (__builtin_expect(wave >= kComputeWaves, 0)) {
    // ---- copying waves: the x tiles of this workgroup's steps, one after the other (across items), into
    // the slots of the ring in turn; tile t lives in slot t % R.  D = R - 1 tiles are requested ahead: the
    // loads of a wave return in order, so tile n is there once no more than the loads of the D - 1 tiles
    // after it are in flight, whatever the memory latency (up to D - 1 steps of it are hidden).
    const int cw = wave - kComputeWaves;
    constexpr int R = Cfg::R, D = R - 1;
    constexpr int L = BM / (4 * kCopyWaves);  // loads per tile and wave: an instruction copies four rows of 256 bytes
    static_assert((D - 1) * L < 64, "the loads in flight must fit the counter");
    int total = 0;  // steps of this workgroup
    for (int i = blockIdx.x; i < n_items; i += gridDim.x) total += item_of(i).steps;
    int q_it = blockIdx.x, q_s = 0, issued = 0;  // the next tile to request: step q_s of item q_it
    WoItem q = item_of(q_it);
    // this lane's part of each of its L loads of a tile, from the tile's first byte (less than 2^32: 128 rows of at
    // most 2^24 bytes): lane l copies row l / 16 of four, 16-byte chunk l % 16, swizzled on the source side; rows
    // past the end repeat the last one.  Kept across the steps of an item: the base of a tile is then scalar.
    uint32_t x_off[L];
    auto set_offsets = [&]() __attribute__((always_inline)) {
#pragma unroll
      for (int i = 0; i < L; ++i) {
        const int row = min((cw + i * kCopyWaves) * 4 + (lane >> 4), q.rows - 1);
        x_off[i] = (uint32_t)row * ((uint32_t)K * 2u) + (uint32_t)(((lane & 15) ^ (row & 15)) * 16);
      }
    };
    set_offsets();
    auto issue = [&]() __attribute__((always_inline)) {
      if (issued >= total) return;
      char* const dst = ring + (issued % R) * X_TILE;
      const char* const xb = (const char*)a.x + ((size_t)q.m0 * K + q.k_begin) * 2 + (size_t)q_s * 256;
#pragma unroll
      for (int i = 0; i < L; ++i)
        __builtin_amdgcn_global_load_lds((const void*)(xb + (size_t)x_off[i]), (lds_ptr_t)(dst + (cw + i * kCopyWaves) * 1024), 16, 0, 0);
      ++issued;
      if (++q_s == q.steps) {
        q_s = 0;
        q_it += gridDim.x;
        if (q_it < n_items) {
          const int rows_before = q.rows;
          q = item_of(q_it);
          if (q.rows != rows_before) set_offsets();
        }
      }
    };
    // Results that the computing waves left in LDS (stage_out): the dot products rounded to the dot dtype,
    // [128 rows][256 channels] of 2 bytes, the 16-byte chunks of a row swizzled by the row.  The copying waves
    // multiply them by the channels' scales and write them out: an instruction two rows (512 bytes each: whole
    // lines); a wave has 16 of them per item and does two per step from the next item's first step on.  A lane
    // always handles the same eight channels of the tile and keeps their scales in registers.  These reach it
    // through LDS as well (a load into registers here would make the compiler wait for every x tile in flight):
    // with the results written out, four steps before the item's end, the first copying wave requests the item's
    // 256 scales into the first row of the results' area; two steps later, a barrier after they have arrived, every
    // copying wave reads its lanes' scales, and another barrier later the computing waves may overwrite them.
    // The host asks for this path from 12 steps per item up.
    constexpr int kDrainPerWave = BM / 2 / kCopyWaves;
    static_assert(Cfg::kStage == 0 || D == 2, "the waits below count what is issued within one step");
    int c_it = blockIdx.x, c_s = 0, drain_left = 0;  // the step the computing waves begin after the next barrier
    WoItem c_item = item_of(c_it), d_item = c_item;  // d_item: the item whose results are in LDS
    float sc[8] = {0, 0, 0, 0, 0, 0, 0, 0};          // scales of the channels n0 + 8 (lane % 32) .. + 7 of d_item
    // (the LDS reads are written as assembly: the compiler would put a wait for every load of x in flight before
    // an LDS read that follows them in the same wave, since those loads write LDS)
    auto lds_read16 = [&](const char* p) __attribute__((always_inline)) {
      i32x4 v;
      asm volatile("ds_read_b128 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"((uint32_t)(uintptr_t)(lds_ptr_t)p) : "memory");
      return v;
    };
    // Writes out up to two pairs of rows and returns the number of store instructions issued (a pair of rows
    // past M issues none).
    auto drain = [&]() __attribute__((always_inline)) {
      int stores = 0;
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        if (drain_left > 0) {
          const int pair = cw * kDrainPerWave + (kDrainPerWave - drain_left);  // uniform over the wave
          --drain_left;
          if (d_item.m0 + 2 * pair < M) {
            const int row = 2 * pair + (lane >> 5), c = lane & 31;
            const i32x4 v = lds_read16(smem + row * 512 + ((c ^ (row & 31)) * 16));
            i32x4 o;
#pragma unroll
            for (int h = 0; h < 4; ++h) {
              const uint32_t d = (uint32_t)v[h];
              const float r0 = sc[2 * h] * qmm_from_raw(d & 0xffffu, XT), r1 = sc[2 * h + 1] * qmm_from_raw(d >> 16, XT);
              o[h] = (int)(XT == XLA_AMD_DT_BF16 ? qmm_f32x2_to_bf16x2(r0, r1) : qmm_f32x2_to_f16x2(r0, r1));
            }
            const int m = d_item.m0 + row, n = d_item.n0 + 8 * c;
            if (m < M && n < N) *(i32x4*)((uint16_t*)a.out + (size_t)m * N + n) = o;
            ++stores;
          }
        }
      }
      return stores;
    };
    for (int d = 0; d < D; ++d) issue();
    int ops_before = 0;  // memory instructions issued between the loads of tile n and those of tile n + 1
    for (int n = 0; n < total; ++n) {
      // the tiles n + 1 .. n + D - 1 may be in flight, and what was issued between them (the memory instructions
      // of a wave complete in the order of their issue)
      if (issued - n == D) {
        if (ops_before == 0) qmm_wait_vmcnt<(D - 1) * L>();
        else if (ops_before == 1) qmm_wait_vmcnt<(D - 1) * L + 1>();
        else qmm_wait_vmcnt<(D - 1) * L + 2>();
      } else {
        qmm_wait_vmcnt<0>();  // (the first and the last tiles of the workgroup)
      }
      qmm_bare_barrier();  // tile n is there; the computing waves have read tile n - 1
      ops_before = 0;
      if (stage_out) {
        if (c_s < c_item.steps - 4) {
          ops_before = drain();
        } else if (c_s == c_item.steps - 4) {
          if (cw == 0) {  // (lanes 32 .. 63 fetch the same 512 bytes again, into the second row)
            const int n8 = min(c_item.n0 + 8 * (lane & 31), N - 8);
            __builtin_amdgcn_global_load_lds((const void*)((const uint16_t*)a.scale + n8), (lds_ptr_t)smem, 16, 0, 0);
            ops_before = 1;
          }
        } else if (c_s == c_item.steps - 2) {
          const i32x4 v = lds_read16(smem + (lane & 31) * 16);
#pragma unroll
          for (int h = 0; h < 4; ++h) {
            sc[2 * h] = qmm_from_raw((uint32_t)v[h] & 0xffffu, XT);
            sc[2 * h + 1] = qmm_from_raw((uint32_t)v[h] >> 16, XT);
          }
        }
        if (++c_s == c_item.steps) {  // after this step the computing waves leave this item's results in LDS
          d_item = c_item;
          drain_left = kDrainPerWave;
          c_s = 0;
          c_it += gridDim.x;
          if (c_it < n_items) c_item = item_of(c_it);
        }
      }
      issue();  // tile n + D into the slot of tile n - 1
    }
    if (stage_out) {
      qmm_bare_barrier();  // the last item's results are in LDS
      while (drain_left > 0) drain();
    }
    return;
  }

  // ---- computing waves ----
  // wave w owns the channels n0 + 64 w .. + 63 of the item's column tile as NG MFMA row sets of 16 consecutive
  // channels, whatever the width G of the channel groups of the tiled weight: channel n lies in group n / G at
  // row n % G, so the 16 rows of a set come out of one or two groups and every lane keeps its own offset
  // (channels past N read the last one again; their results are dropped).
  const int n_blk = a.Kw / 128;  // blocks per channel group in the tiled weight
  const int w_halves = 2 * n_blk;  // the item's halves wrap round the weight's (x in three parts: three trips)
  const int blk_bytes = G * 128, half_bytes = G * 64;
  constexpr int H = wo_ring_halves<MT, NG, HASZP, UNI>(), R = Cfg::R;
  static_assert(H % 2 == 1, "a step uses two halves: an odd ring visits every phase in H steps");
  const uint8_t* wp;     // wave-uniform: the first half block of the item in the tile's first channel group
  uint32_t w_lane[NG];   // from there to this lane's 16 bytes of row set gi (less than 2^32: 270 channels of K columns)
  i32x4 wreg[H][NG];     // ring: half q of the item (block q / 2, columns 64 (q % 2) ..) lives in slot q % H
  // (divisions by G without a divide: the channel is at most 271 past the first channel of the tile's first
  // group, and for t < 272 and G <= 16, t / G == (t * ceil(65536 / G)) >> 16)
  const uint32_t g_magic = (65536u + (uint32_t)G - 1u) / (uint32_t)G;
  auto set_weights = [&](const WoItem& w) __attribute__((always_inline)) {
    const int p0 = w.n0 / G, a0 = w.n0 - p0 * G;
    wp = a.w + ((size_t)p0 * n_blk + w.k_begin / 128) * blk_bytes;
    qmm_static_for<NG>([&](auto gc) {
      constexpr int gi = gc;
      const uint32_t t = (uint32_t)(a0 + min((wave * NG + gi) * 16 + r, N - 1 - w.n0));
      const uint32_t pd = (t * g_magic) >> 16, row = t - pd * (uint32_t)G;
      w_lane[gi] = pd * ((uint32_t)n_blk * (uint32_t)blk_bytes) + ((uint32_t)(g * G) + row) * 16u;
    });
  };
  // half q of the item into its slot (a half past the end is the last one again: never used, and no branch
  // around the loads: the counts of loads in flight stay known at compile time on every path)
  auto request = [&](int q, int last, auto slotc) __attribute__((always_inline)) {
    constexpr int slot = slotc;
    int qq = min(q, last);
    if (qq >= w_halves) qq -= w_halves;
    if (qq >= w_halves) qq -= w_halves;
    qmm_static_for<NG>([&](auto gc) {
      constexpr int gi = gc;
      const uint8_t* half = wp + (size_t)qq * half_bytes;  // uniform: scalar base + lane offset
      // (an ordinary load, not a streaming one: the other row tiles read the same block out of L2; measured 5 % apart)
      wreg[slot][gi] = *(const i32x4*)(half + (size_t)w_lane[gi]);
    });
  };
  auto load_first = [&](const WoItem& w) __attribute__((always_inline)) {
    qmm_static_for<H>([&](auto hc) { request((int)hc, 2 * w.steps - 1, hc); });
  };

  f32x4 acc[NG][MT], xs[MT];
  // The converted weight fragments of one j (columns 32 g + 8 j .. + 7 of the step, one fragment per row set gi):
  // those in use and those of the next j, which are converted meanwhile; the fragments of a step's first j are
  // converted during the step before (or, for an item's first step, by prime()).
  i32x4 af[2][NG];
  auto prime = [&]() __attribute__((always_inline)) {
    qmm_static_for<NG>([&](auto gc) {
      const i32x4 src = wreg[0][(int)gc];
      af[0][(int)gc] = cvt_w8<XT>((uint32_t)src[0], (uint32_t)src[1]);
    });
  };
  // One step (128 columns): step s of an item of S steps, x out of LDS slot `xslot`, weights out of the ring
  // slots PH (columns 0 .. 63) and PH + 1 (columns 64 .. 127); each slot is requested again (half + H of the
  // item) as soon as its last fragment has been converted.
  // The order is j, row tile mt, row set gi: an x fragment (one LDS read) serves NG MFMAs in a row and is read two
  // row tiles ahead into one of three registers in turn, so the LDS reads of the four computing waves, which run
  // in step, come one per NG MFMAs instead of MT at once (that burst, 32 KB per compute unit, took longer than
  // the MFMAs it fed: a quarter of the step went to waiting for LDS).  Between the MFMAs sit the conversions of
  // the next j's fragments, a quarter of a fragment (three instructions) after every MT / 4 th MFMA.  A
  // scheduling fence after each MFMA keeps that order: left to itself the compiler emits the conversions and
  // the MFMAs as separate runs, and with one computing wave per SIMD nothing else fills the gaps.
  auto compute = [&](int xslot, int s, int S, auto phc) __attribute__((always_inline)) {
    constexpr int PH = phc;
    const char* xrow = ring + xslot * X_TILE + r * 256;  // this lane's row of each 16-row tile
    const int last = 2 * S - 1;
    auto xfrag = [&](int idx) __attribute__((always_inline)) {  // idx = j * MT + mt
      return *(const i32x4*)(xrow + (idx % MT) * (16 * 256) + (((4 * g + idx / MT) ^ r) * 16));
    };
    i32x4 xq[3];
    xq[0] = xfrag(0);
    xq[1] = xfrag(1);
    __builtin_amdgcn_sched_barrier(0);
    constexpr int kEvery = MT / 4;  // a quarter of a fragment of the next j after every kEvery th MFMA
    qmm_static_for<4 * MT>([&](auto ic) {
      constexpr int idx = ic, j = idx / MT, mt = idx % MT, jn = j + 1;
      if constexpr (idx + 2 < 4 * MT) xq[(idx + 2) % 3] = xfrag(idx + 2);
      qmm_static_for<NG>([&](auto gc) {
        constexpr int gi = gc, u = mt * NG + gi;
        acc[gi][mt] = mfma16<XT>(af[j & 1][gi], xq[idx % 3], acc[gi][mt]);
        if constexpr (HASZP && gi == NG - 1) xs[mt] = mfma16<XT>(ones_frag<XT>(), xq[idx % 3], xs[mt]);
        if constexpr (u % kEvery == 0) {
          // element q of fragment gn of the next j (of the next step's first j during the last one): bytes
          // 2 (q & 1), 2 (q & 1) + 1 of dword q / 2 of its half's second or first 32 columns
          constexpr int gn = (u / kEvery) / 4, q = (u / kEvery) % 4;
          af[jn & 1][gn][q] = (int)cvt_w2<XT>((uint32_t)wreg[(PH + (jn >> 1)) % H][gn][(jn & 1) * 2 + q / 2], qmm_const<(q & 1)>{});
        }
        __builtin_amdgcn_sched_barrier(0);
      });
      // the half whose last fragments have just been converted (columns 0 .. 63 during j = 0, 64 .. 127 during j = 2)
      if constexpr (mt == MT - 1 && (j & 1) == 0) {
        request(2 * s + (j >> 1) + H, last, qmm_const<(PH + (j >> 1)) % H>{});
        __builtin_amdgcn_sched_barrier(0);
      }
    });
  };

  int it = blockIdx.x;
  WoItem cur = item_of(it);
  set_weights(cur);
  load_first(cur);
  int xslot = 0;  // LDS slot of the next x tile: the tiles of all items of the workgroup follow each other round the ring
  auto step = [&](int s, int S, auto phc) __attribute__((always_inline)) {
    qmm_bare_barrier();  // the tile is there (the copying waves waited for it); the tile before it has been read
    compute(xslot, s, S, phc);
    xslot = xslot + 1 == R ? 0 : xslot + 1;
  };
  for (;;) {
    qmm_static_for<MT>([&](auto mc) {
      constexpr int mt = mc;
      xs[mt] = f32x4{0, 0, 0, 0};
      qmm_static_for<NG>([&](auto gc) { acc[(int)gc][mt] = f32x4{0, 0, 0, 0}; });
    });
    prime();
    // H steps visit the H phases of the weight ring (step s starts at half 2 s, slot 2 s % H): unrolled, so that
    // every register of the ring is named at compile time; the last S % H steps follow one by one
    const int S = cur.steps;
    int s = 0;
    for (; s + H <= S; s += H)
      qmm_static_for<H>([&](auto kc) { step(s + (int)kc, S, qmm_const<(2 * (int)kc) % H>{}); });
    qmm_static_for<H - 1>([&](auto kc) {
      if (s + (int)kc < S) step(s + (int)kc, S, qmm_const<(2 * (int)kc) % H>{});
    });

    // the next item's first weights are requested before this item's results are stored: a wait
    // for them then does not include the stores
    const WoItem done = cur;
    const int it_next = it + (int)gridDim.x;
    const bool more = it_next < n_items;
    if (more) {
      it = it_next;
      cur = item_of(it);
      set_weights(cur);
      load_first(cur);
    }

    // ---- results: four consecutive channels of one row per lane ----
    const int m0 = done.m0;
    // channels of this lane for row set gi of its wave: n .. n + cnt - 1, n a multiple of 4 (cnt <= 4, or <= 0 past N;
    // computed where they are used: the 128 x 256 tile has no register to keep them in)
    const int n_first = done.n0 + wave * (NG * 16) + 4 * g;
    auto chan = [&](int gi, int& n, int& cnt) __attribute__((always_inline)) {
      n = n_first + gi * 16;
      cnt = min(N - n, 4);
    };
    if (stage_out) {
      // the dot products, rounded, into LDS: row 16 mt + r, 16-byte chunk 8 wave + 2 gi + g / 2 (swizzled by the
      // row), half g % 2; the copying waves scale them and write them out
      qmm_static_for<MT>([&](auto mc) {
        constexpr int mt = mc;
        const int row = 16 * mt + r;
        qmm_static_for<NG>([&](auto gc) {
          constexpr int gi = gc;
          const f32x4 d = acc[gi][mt];
          const uint32_t lo = XT == XLA_AMD_DT_BF16 ? qmm_f32x2_to_bf16x2(d[0], d[1]) : qmm_f32x2_to_f16x2(d[0], d[1]);
          const uint32_t hi = XT == XLA_AMD_DT_BF16 ? qmm_f32x2_to_bf16x2(d[2], d[3]) : qmm_f32x2_to_f16x2(d[2], d[3]);
          const int chunk = (wave * 8 + gi * 2 + (g >> 1)) ^ (row & 31);
          *(i32x2*)(smem + row * 512 + chunk * 16 + (g & 1) * 8) = i32x2{(int)lo, (int)hi};
        });
      });
    } else if (a.split == 1) {
      const WoDts<XT, UNI> dts(a);
      // scales (and zero points) of this lane's channels first, all at once: loads inside the
      // loop over row tiles would be waited for one after the other
      uint32_t sraw[NG][4], zraw[NG][4];
      qmm_static_for<NG>([&](auto gc) {
        constexpr int gi = gc;
        int n, cnt;
        chan(gi, n, cnt);
        n = min(n, N - 1);
        wo_load4_raw(a.scale, n, N, dts.scale_dt, sraw[gi]);
        if constexpr (HASZP) wo_load4_raw(a.zp, n, N, dts.zp_dt, zraw[gi]);
      });
      // the two store forms as two straight-line copies of the whole epilogue, chosen once
      auto emit = [&](auto vecc) __attribute__((always_inline)) {
        constexpr bool kVec = vecc != 0;
        qmm_static_for<MT>([&](auto mc) {
          constexpr int mt = mc;
          const int m = m0 + 16 * mt + r;
          qmm_static_for<NG>([&](auto gc) {
            constexpr int gi = gc;
            int n, cnt;
            chan(gi, n, cnt);
            if (m < M && cnt > 0) {
              if (kVec && cnt == 4) {  // four channels (n is a multiple of 4): one store
                if constexpr (kVec && UNI && !HASZP && XT == XLA_AMD_DT_BF16) {
                  wo_finish_store_bf16(a.out, m, n, N, sraw[gi], acc[gi][mt]);
                } else {
                  float o[4];
                  wo_finish4(dts, sraw[gi], zraw[gi], HASZP, acc[gi][mt], HASZP ? xs[mt][0] : 0.f, dts.x_dt, o);
                  wo_store4<kVec>(a.out, m, n, N, o, dts.store_dt);
                }
              } else {
                float o[4];
                wo_finish4(dts, sraw[gi], zraw[gi], HASZP, acc[gi][mt], HASZP ? xs[mt][0] : 0.f, dts.x_dt, o);
                wo_store_some(a.out, m, n, N, cnt, o, dts.store_dt);
              }
            }
          });
        });
      };
      if ((N & 3) == 0) {
        emit(qmm_const<1>{});
      } else {
        emit(qmm_const<0>{});
      }
    } else {
      const bool vec = (N & 3) == 0;
      qmm_static_for<NG>([&](auto gc) {
        constexpr int gi = gc;
        int n, cnt;
        chan(gi, n, cnt);
        qmm_static_for<MT>([&](auto mc) {
          constexpr int mt = mc;
          const int m = m0 + 16 * mt + r;
          if (m < M && cnt > 0) {
            float* p = a.part + ((size_t)done.ks * M + m) * N + n;
            if (vec && cnt == 4 && (n & 3) == 0) *(f32x4*)p = acc[gi][mt];
            else for (int v = 0; v < 4; ++v) if (v < cnt) p[v] = acc[gi][mt][v];
          }
        });
      });
      if constexpr (HASZP) {
        // partial row sums of x: once per row tile and K slice (the first column tile's first wave, channel lanes 0..15)
        if (done.n0 == 0 && wave == 0 && g == 0) {
          qmm_static_for<MT>([&](auto mc) {
            constexpr int mt = mc;
            const int m = m0 + 16 * mt + r;
            if (m < M) a.part_xs[(size_t)done.ks * M + m] = xs[mt][0];
          });
        }
      }
    }
    if (!more) break;
  }
  if (stage_out) qmm_bare_barrier();  // the copying waves may write out the last item's results
}

// Compute units of the current device (asked once per device).
int cu_count() {
  static std::atomic<int> cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  int n = cached[dev].load(std::memory_order_relaxed);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cached[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}

template <int XT, int MT, int NG>
int launch(const WoGemmArgs& a, hipStream_t stream) {
  using Cfg = WoCfg<MT, NG>;
  const int64_t items = (int64_t)((a.M + Cfg::BM - 1) / Cfg::BM) * (((int64_t)a.N + 64 * NG - 1) / (64 * NG)) * a.split;
  const int steps = a.k_per_split / 128;
  // one workgroup per compute unit (its LDS and registers leave room for no second one); each walks its share of
  // the items.  No more workgroups than give every one the same number of items: 896 items are four rounds on
  // 256 compute units as on 224, and the chip, which runs this kernel at the clock its power allows, is faster
  // with 32 of them idle throughout than with 128 idle in the last round (193.5 -> 191.5 us).
  const int cus = cu_count();
  const int64_t rounds = (items + cus - 1) / cus;
  const dim3 grid((unsigned)((items + rounds - 1) / rounds)), block((kComputeWaves + kCopyWaves) * 64);
  auto go = [&](auto kern) -> int {
    static std::atomic<uint64_t> lds_set{0};
    const int rc = qmm_set_max_lds((const void*)kern, Cfg::lds_bytes(1 << 20), lds_set, "weight_only_gemm hipFuncSetAttribute");
    if (rc != XLA_AMD_QMM_OK) return rc;
    // a workgroup with several items keeps the whole ring of x tiles whatever the slice length
    hipLaunchKernelGGL(kern, grid, block, Cfg::lds_bytes(items > cus ? (1 << 20) : steps), stream, a);
    return QMM_CHECK_LAUNCH("weight_only_gemm launch");
  };
  // one dtype throughout (x, scale, zero point, dot, out, store): the epilogue's dtypes fold at compile time
  const bool uni = a.scale_dt == XT && a.zp_dt == XT && a.dot_dt == XT && a.out_dt == XT && a.store_dt == XT;
  if constexpr (MT == 8 && NG == 4) {
    // (the 128 x 256 tile fits the register file neither with the row sums of x nor with dtypes known only at run
    // time: the plan never asks for the first, and the second takes the 128 x 128 tile)
    if (a.zp) return qmm_fail(XLA_AMD_QMM_EUNSUPPORTED, "weight_only_gemm: no 128 x 256 tile with a zero point");
    if (!uni) return launch<XT, MT, 2>(a, stream);
    return go(qmm_wo_gemm_kernel<XT, MT, NG, false, true>);
  } else {
    if (uni) return a.zp ? go(qmm_wo_gemm_kernel<XT, MT, NG, true, true>) : go(qmm_wo_gemm_kernel<XT, MT, NG, false, true>);
    return a.zp ? go(qmm_wo_gemm_kernel<XT, MT, NG, true, false>) : go(qmm_wo_gemm_kernel<XT, MT, NG, false, false>);
  }
}

}  // namespace

#define QMM_WO_CAT2(a, b, c) a##b##c
#define QMM_WO_CAT(a, b, c) QMM_WO_CAT2(a, b, c)
#if QMM_WO_XT == XLA_AMD_DT_BF16
#define QMM_WO_UNIT_NAME QMM_WO_CAT(qmm_wo_launch_bf16_mt, QMM_WO_MT, )
#else
#define QMM_WO_UNIT_NAME QMM_WO_CAT(qmm_wo_launch_f16_mt, QMM_WO_MT, )
#endif
int QMM_WO_UNIT_NAME(const WoGemmArgs& a, int ng, hipStream_t stream) {
  return ng == 4 ? launch<QMM_WO_XT, QMM_WO_MT, 4>(a, stream) : launch<QMM_WO_XT, QMM_WO_MT, 2>(a, stream);
}

#if QMM_WO_XT == XLA_AMD_DT_BF16 && QMM_WO_MT == 8
namespace {

// Adds the partial sums of a K split in slice order and finishes them: one thread per four
// consecutive channels of one row.
__global__ void __launch_bounds__(256) qmm_wo_gemm_finish_kernel(WoGemmArgs a, int x_dt) {
  const int n4 = (a.N + 3) / 4;
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (int64_t)a.M * n4) return;
  const int m = (int)(idx / n4), n = (int)(idx % n4) * 4;
  const WoDts<0, false> dts(a);
  uint32_t sraw[4], zraw[4] = {0, 0, 0, 0};
  wo_load4_raw(a.scale, n, a.N, dts.scale_dt, sraw);
  if (a.zp) wo_load4_raw(a.zp, n, a.N, dts.zp_dt, zraw);
  f32x4 dot = {0, 0, 0, 0};
  float xsum = 0.f;
  const size_t slice = (size_t)a.M * a.N;
  const float* p = a.part + (size_t)m * a.N + n;
  int s = 0;
  if ((a.N & 3) == 0) {
    // four slices' loads in flight at a time (the slices come from memory: one load after the
    // other would cost a memory latency each); the additions stay in slice order
    for (; s + 4 <= a.split; s += 4) {
      const f32x4 p0 = *(const f32x4*)(p + (size_t)s * slice), p1 = *(const f32x4*)(p + (size_t)(s + 1) * slice);
      const f32x4 p2 = *(const f32x4*)(p + (size_t)(s + 2) * slice), p3 = *(const f32x4*)(p + (size_t)(s + 3) * slice);
      dot += p0; dot += p1; dot += p2; dot += p3;
    }
    for (; s < a.split; ++s) dot += *(const f32x4*)(p + (size_t)s * slice);
  } else {
    for (; s < a.split; ++s)
      for (int v = 0; v < 4; ++v) if (n + v < a.N) dot[v] += p[(size_t)s * slice + v];
  }
  if (a.zp)
    for (int t = 0; t < a.split; ++t) xsum += a.part_xs[(size_t)t * a.M + m];
  float o[4];
  wo_finish4(dts, sraw, zraw, a.zp != nullptr, dot, xsum, x_dt, o);
  if ((a.N & 3) == 0) wo_store4<true>(a.out, m, n, a.N, o, dts.store_dt);
  else wo_store4<false>(a.out, m, n, a.N, o, dts.store_dt);
}

// The second kernel of K slices over blockwise weights: every slice left its sum over blocks of
// scale * round(block dot) in part and of round(block sum of x) * zero point in part_z (or null);
// out = round_out(sum), with a zero point round_out(out - round_zpo(sum of part_z)).
// One thread per four consecutive channels of one row (N % 4 == 0).
__global__ void __launch_bounds__(256) qmm_wo_bw_finish_kernel(const float* part, const float* part_z, void* out, int M,
                                                               int N, int split, int out_dt, int zpo_dt, int store_dt) {
  const int n4 = N / 4;
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (int64_t)M * n4) return;
  const int m = (int)(idx / n4), n = (int)(idx % n4) * 4;
  const size_t slice = (size_t)M * N, at = (size_t)m * N + n;
  auto sum = [&](const float* p) {
    f32x4 t = {0, 0, 0, 0};
    int s = 0;
    for (; s + 4 <= split; s += 4) {  // four loads in flight, additions in slice order
      const f32x4 p0 = *(const f32x4*)(p + (size_t)s * slice), p1 = *(const f32x4*)(p + (size_t)(s + 1) * slice);
      const f32x4 p2 = *(const f32x4*)(p + (size_t)(s + 2) * slice), p3 = *(const f32x4*)(p + (size_t)(s + 3) * slice);
      t += p0; t += p1; t += p2; t += p3;
    }
    for (; s < split; ++s) t += *(const f32x4*)(p + (size_t)s * slice);
    return t;
  };
  const f32x4 t = sum(part + at);
  float o[4];
#pragma unroll
  for (int v = 0; v < 4; ++v) o[v] = qmm_round_dt(t[v], out_dt);
  if (part_z) {
    const f32x4 z = sum(part_z + at);
#pragma unroll
    for (int v = 0; v < 4; ++v) o[v] = qmm_round_dt(o[v] - qmm_round_dt(z[v], zpo_dt), out_dt);
  }
  wo_store4<true>(out, m, n, N, o, store_dt);
}

struct Plan {
  int mt, ng, split, k_per_split;
};

// floats of workspace for K slices of the weight-streaming kernel
size_t slice_workspace_floats(int slices, int64_t M, int64_t N, bool blockwise) {
  const size_t mn = (size_t)slices * (size_t)M * (size_t)N;
  return blockwise ? 2 * mn : mn + (size_t)slices * (size_t)M;  // blockwise: room for the zero-point sums
}

// Tile and K split by shape.  Row tiles of 64 / 128 rows; 256 channels per workgroup, or 128 when the wide tiles
// leave a quarter of the chip idle and the narrow ones still fit one round of workgroups (three row tiles against
// 14336 channels: 168 wide tiles in one round take 48 us, 336 narrow ones in two rounds 59); K split over
// workgroups while the items still fit one round (a part-full second round costs a whole one, and the second
// kernel's partial sums grow with the split: 128 rows against 14336 x 4096 took 36 us in three slices, 336 items,
// and take 28 in two), in slices of at least 512 columns.
// (with a zero point the 128-row tile keeps 128 channels per workgroup: the row sums of x take
// the registers that the wider tile would need)
Plan make_plan(int64_t M, int64_t N, int64_t K, bool has_zp) {
  Plan p;
  p.mt = M <= 64 ? 4 : 8;
  const int64_t bm = 16 * p.mt;
  const int64_t tiles_m = (M + bm - 1) / bm;
  const int64_t groups = (N + 15) / 16;  // MFMA row sets of 16 channels: a column tile is 4 * ng of them
  const int64_t wide = tiles_m * ((groups + 15) / 16), narrow = tiles_m * ((groups + 7) / 8);
  p.ng = 4;
  if ((wide < 192 && narrow <= 256 && N > 128) || (has_zp && p.mt == 8)) p.ng = 2;
  const int64_t tiles = p.ng == 2 ? narrow : wide;
  int64_t split = 1;
  if (tiles <= 128) split = 256 / tiles;
  const int64_t blocks = K / 128;
  int64_t per = (blocks + split - 1) / split;
  if (per < 4) per = blocks < 4 ? blocks : 4;
  split = (blocks + per - 1) / per;
  p.split = (int)split;
  p.k_per_split = (int)per * 128;
  return p;
}

}  // namespace

namespace {

// x f32 [M, K] -> [M, 3 K] bf16: hi | mid | lo side by side, hi = bf16(x), mid = bf16(x - hi), lo = bf16(x - hi - mid)
// (round to nearest even; the differences are exact in f32): hi + mid + lo = x to the last bit of f32 for finite x,
// and every product of a part with an int8 weight is exact in the f32 accumulator of the MFMA.  An infinity or a
// NaN stays in hi alone.
__global__ void __launch_bounds__(256) qmm_split3_kernel(const float* x, uint16_t* out, int64_t quads, int K) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= quads) return;
  const int kq = K / 4;
  const int64_t m = i / kq;
  const int c = (int)(i - m * kq) * 4;
  const f32x4 v = *(const f32x4*)(x + m * K + c);
  uint16_t part[3][4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const uint16_t hi = qmm_f32_to_bf16(v[e]);
    const float fh = qmm_bf16_to_f32(hi);
    const bool finite = (__float_as_uint(fh) & 0x7f800000u) != 0x7f800000u;
    const float r1 = finite ? v[e] - fh : 0.f;
    const uint16_t mid = qmm_f32_to_bf16(r1);
    const float r2 = r1 - qmm_bf16_to_f32(mid);
    part[0][e] = hi; part[1][e] = mid; part[2][e] = qmm_f32_to_bf16(r2);
  }
  uint16_t* o = out + m * (3 * (int64_t)K) + c;
#pragma unroll
  for (int t = 0; t < 3; ++t)
    *(i32x2*)(o + (int64_t)t * K) = i32x2{(int)(part[t][0] | ((uint32_t)part[t][1] << 16)), (int)(part[t][2] | ((uint32_t)part[t][3] << 16))};
}

}  // namespace

extern "C" size_t xla_amd_qmm_weight_only_gemm_f32_workspace_bytes(int64_t M, int64_t N, int64_t K) {
  if (M <= 0 || N <= 0 || K <= 0 || K % 128 != 0) return 0;
  return (size_t)M * (size_t)K * 3 * sizeof(uint16_t);
}

extern "C" int xla_amd_qmm_weight_only_gemm_f32(const float* x, const void* w_tiled, const void* scale, const void* zp,
                                                float* out, void* workspace, size_t workspace_bytes, int64_t M, int64_t N,
                                                int64_t K, int scale_dt, int zp_dt, void* stream) {
  if (!x || !w_tiled || !scale || !out) return qmm_fail(XLA_AMD_QMM_EINVAL, "weight_only_gemm_f32: null pointer");
  if (M < 0 || N <= 0 || K <= 0) return qmm_fail(XLA_AMD_QMM_EINVAL, "weight_only_gemm_f32: bad sizes");
  if (!qmm_valid_dt(scale_dt) || (zp && !qmm_valid_dt(zp_dt))) return qmm_fail(XLA_AMD_QMM_EINVAL, "weight_only_gemm_f32: bad dtype enum");
  if (K % 128 != 0) return qmm_fail(XLA_AMD_QMM_EUNSUPPORTED, "weight_only_gemm_f32: K=%lld must be a multiple of 128", (long long)K);
  if (N > (1 << 30) || 3 * K > (1 << 23) || M > (1 << 24))
    return qmm_fail(XLA_AMD_QMM_EUNSUPPORTED, "weight_only_gemm_f32: dimension too large");
  if ((((uintptr_t)x | (uintptr_t)w_tiled | (uintptr_t)out | (uintptr_t)workspace) & 15))
    return qmm_fail(XLA_AMD_QMM_EUNSUPPORTED, "weight_only_gemm_f32: x, w, out and workspace must be 16-byte aligned");
  if (M == 0) return XLA_AMD_QMM_OK;
  const size_t need = xla_amd_qmm_weight_only_gemm_f32_workspace_bytes(M, N, K);
  if (!workspace || workspace_bytes < need)
    return qmm_fail(XLA_AMD_QMM_EINVAL, "weight_only_gemm_f32: workspace of %zu bytes, need %zu", workspace ? workspace_bytes : (size_t)0, need);
  hipStream_t s = (hipStream_t)stream;
  const int64_t quads = M * (K / 4);
  hipLaunchKernelGGL(qmm_split3_kernel, dim3((unsigned)((quads + 255) / 256)), dim3(256), 0, s, x, (uint16_t*)workspace, quads, (int)K);
  int rc = QMM_CHECK_LAUNCH("weight_only_gemm_f32 split launch");
  if (rc != XLA_AMD_QMM_OK) return rc;
  // the bf16 GEMM over 3 K columns of x against the weight's K columns three times over, f32 from the dot product on
  Plan p = make_plan(M, N, 3 * K, zp != nullptr);
  WoGemmArgs a;
  a.x = workspace; a.w = (const uint8_t*)w_tiled; a.scale = scale; a.zp = zp; a.out = out;
  a.part = nullptr; a.part_xs = nullptr;
  a.M = (int)M; a.N = (int)N; a.K = (int)(3 * K);
  a.Kw = (int)K; a.x_dt = XLA_AMD_DT_F32; a.stage_out = 0;
  a.G = xla_amd_qmm_tile_group(N, K, K, 8);
  a.k_per_split = (int)(3 * K); a.split = 1;  // (no K split: a slice would have to wrap round the weight)
  a.scale_dt = scale_dt; a.zp_dt = zp ? zp_dt : XLA_AMD_DT_F32;
  a.dot_dt = XLA_AMD_DT_F32; a.out_dt = XLA_AMD_DT_F32; a.store_dt = XLA_AMD_DT_F32;
  return p.mt == 4 ? qmm_wo_launch_bf16_mt4(a, p.ng, s) : qmm_wo_launch_bf16_mt8(a, p.ng, s);
}

extern "C" size_t xla_amd_qmm_weight_only_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K, int64_t C, int bits) {
  if (M <= 0 || N <= 0 || K <= 0 || K % 128 != 0) return 0;
  if (C <= 0) C = K;
  if (K % C != 0) return 0;
  if (M <= 32) {  // the weight-streaming kernel over K slices
    int per;
    const int slices = qmm_skinny_k_slices(M, N, K, C, bits, &per);
    if (slices > 1) return slice_workspace_floats(slices, M, N, C != K) * sizeof(float);
  }
  if (C != K || bits != 8) return 0;  // blockwise / int4 weights: the tiled GEMM splits no K and needs no workspace
  size_t need = 0;
  for (int zp = 0; zp < 2; ++zp) {  // the larger of the two plans: the size does not depend on the zero point
    const Plan p = make_plan(M, N, K, zp != 0);
    if (p.split > 1) {
      const size_t b = ((size_t)p.split * (size_t)M * (size_t)N + (size_t)p.split * (size_t)M) * sizeof(float);
      need = b > need ? b : need;
    }
  }
  return need;
}

extern "C" int xla_amd_qmm_weight_only_gemm(const void* x, const void* w_tiled, const void* scale, const void* zp,
                                            void* out, void* workspace, size_t workspace_bytes, int64_t M, int64_t N,
                                            int64_t K, int64_t C, int bits, int x_dt, int scale_dt, int zp_dt,
                                            int dot_dt, int out_dt, int store_dt, void* stream) {
  if (!x || !w_tiled || !scale || !out) return qmm_fail(XLA_AMD_QMM_EINVAL, "weight_only_gemm: null pointer");
  if (M < 0 || N <= 0 || K <= 0 || C <= 0 || K % C != 0)
    return qmm_fail(XLA_AMD_QMM_EINVAL, "weight_only_gemm: bad sizes M=%lld N=%lld K=%lld C=%lld", (long long)M,
                    (long long)N, (long long)K, (long long)C);
  if (bits != 4 && bits != 8) return qmm_fail(XLA_AMD_QMM_EINVAL, "weight_only_gemm: bits must be 4 or 8");
  if (!qmm_valid_dt(x_dt) || !qmm_valid_dt(scale_dt) || !qmm_valid_dt(out_dt) || !qmm_valid_dt(dot_dt) ||
      !qmm_valid_dt(store_dt) || (zp && !qmm_valid_dt(zp_dt)))
    return qmm_fail(XLA_AMD_QMM_EINVAL, "weight_only_gemm: bad dtype enum");
  if (out_dt != qmm_promote(x_dt, scale_dt))
    return qmm_fail(XLA_AMD_QMM_EINVAL, "weight_only_gemm: out dtype must be promote(x, scale)");
  if (dot_dt != x_dt && dot_dt != XLA_AMD_DT_F32)
    return qmm_fail(XLA_AMD_QMM_EINVAL, "weight_only_gemm: dot dtype must be x's or f32");
  if (x_dt == XLA_AMD_DT_F32) return qmm_fail(XLA_AMD_QMM_EUNSUPPORTED, "weight_only_gemm: x must be bf16 or f16");
  if (K % 128 != 0) return qmm_fail(XLA_AMD_QMM_EUNSUPPORTED, "weight_only_gemm: K=%lld must be a multiple of 128", (long long)K);
  if (N > (1 << 30) || K > (1 << 23) || M > (1 << 24))
    return qmm_fail(XLA_AMD_QMM_EUNSUPPORTED, "weight_only_gemm: dimension too large");
  if (((uintptr_t)x | (uintptr_t)w_tiled) & 15)
    return qmm_fail(XLA_AMD_QMM_EUNSUPPORTED, "weight_only_gemm: x and w must be 16-byte aligned");
  if (((uintptr_t)out & 15) && (N & 3) == 0)
    return qmm_fail(XLA_AMD_QMM_EUNSUPPORTED, "weight_only_gemm: out must be 16-byte aligned");
  if (M == 0) return XLA_AMD_QMM_OK;
  const bool blockwise = C != K;
  // (blockwise weights in the weight-streaming kernel: every dtype but the stored one is x's, at least 8 scales)
  const bool bw_ok = !blockwise || (scale_dt == x_dt && (!zp || zp_dt == x_dt) && dot_dt == x_dt && (K / C) * N >= 8 &&
                                    (((uintptr_t)scale | (uintptr_t)zp) & 3) == 0);
  if (M <= 32 && bw_ok) {
    // few rows: the weight-streaming kernel over K slices, when that is what its plan says and the workspace is there
    int per;
    const int slices = qmm_skinny_k_slices(M, N, K, C, bits, &per);
    const size_t need = slice_workspace_floats(slices, M, N, blockwise) * sizeof(float);
    if (slices > 1 && workspace && workspace_bytes >= need && (((uintptr_t)workspace) & 15) == 0) {
      SkinnyArgs k;
      k.x = x; k.w = (const uint8_t*)w_tiled; k.scale = scale; k.zp = zp; k.out = out;
      k.M = (int)M; k.N = (int)N; k.K = (int)K; k.C = (int)C;
      k.G = xla_amd_qmm_tile_group(N, K, C, bits);
      k.scale_dt = scale_dt; k.zp_dt = zp ? zp_dt : x_dt; k.out_dt = out_dt; k.dot_dt = dot_dt; k.store_dt = store_dt;
      k.k_per_slice = per; k.slices = slices;
      k.part = (float*)workspace;
      const size_t mn = (size_t)slices * (size_t)M * (size_t)N;
      k.part_xs = blockwise ? nullptr : k.part + mn;
      k.part_z = blockwise && zp ? k.part + mn : nullptr;
      int rc = x_dt == XLA_AMD_DT_BF16 ? qmm_skinny_launch_bf16(k, bits, zp != nullptr, (hipStream_t)stream)
                                       : qmm_skinny_launch_f16(k, bits, zp != nullptr, (hipStream_t)stream);
      if (rc != XLA_AMD_QMM_OK) return rc;
      if (blockwise) {
        const int64_t threads = M * (N / 4);
        hipLaunchKernelGGL(qmm_wo_bw_finish_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0,
                           (hipStream_t)stream, k.part, k.part_z, out, (int)M, (int)N, slices, out_dt,
                           qmm_promote(x_dt, k.zp_dt), store_dt);
        return QMM_CHECK_LAUNCH("weight_only_gemm blockwise finish launch");
      }
      WoGemmArgs f;
      f.x = x; f.w = (const uint8_t*)w_tiled; f.scale = scale; f.zp = zp; f.out = out;
      f.part = k.part; f.part_xs = k.part_xs;
      f.M = (int)M; f.N = (int)N; f.K = (int)K; f.G = k.G; f.k_per_split = per; f.split = slices;
      f.scale_dt = scale_dt; f.zp_dt = zp ? zp_dt : x_dt; f.dot_dt = dot_dt; f.out_dt = out_dt; f.store_dt = store_dt;
      const int64_t threads = M * ((N + 3) / 4);
      hipLaunchKernelGGL(qmm_wo_gemm_finish_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0,
                         (hipStream_t)stream, f, x_dt);
      return QMM_CHECK_LAUNCH("weight_only_gemm finish launch");
    }
  }
  if (C != K || bits != 8) {
    // blockwise and int4 weights: the tiled GEMM with per-block rounding points (every dtype x's)
    if (!qmm_valid_dt(x_dt) || x_dt == XLA_AMD_DT_F32)
      return qmm_fail(XLA_AMD_QMM_EUNSUPPORTED, "weight_only_gemm: x must be bf16 or f16");
    if (scale_dt != x_dt || (zp && zp_dt != x_dt) || dot_dt != x_dt || out_dt != x_dt || store_dt != x_dt)
      return qmm_fail(XLA_AMD_QMM_EUNSUPPORTED, "weight_only_gemm: blockwise / int4 weights need every dtype to be x's");
    if (K % 128 != 0 || C % 128 != 0 || N % 4 != 0)
      return qmm_fail(XLA_AMD_QMM_EUNSUPPORTED, "weight_only_gemm: blockwise / int4 weights need K %% 128 == 0, C %% 128 == 0, N %% 4 == 0");
    if (N > (1 << 30) || K > (1 << 24) || M > (1 << 24))
      return qmm_fail(XLA_AMD_QMM_EUNSUPPORTED, "weight_only_gemm: dimension too large");
    if ((((uintptr_t)x | (uintptr_t)w_tiled) & 15) || ((uintptr_t)out & 7) || ((uintptr_t)scale & 3) || ((uintptr_t)zp & 3))
      return qmm_fail(XLA_AMD_QMM_EUNSUPPORTED, "weight_only_gemm: x and w must be 16-byte, out 8-byte, scale / zero point 4-byte aligned");
    if (M == 0) return XLA_AMD_QMM_OK;
    WoBwArgs b;
    b.x = x; b.w = (const uint8_t*)w_tiled; b.scale = scale; b.zp = zp; b.out = out;
    b.M = (int)M; b.N = (int)N; b.K = (int)K; b.C = (int)C;
    return x_dt == XLA_AMD_DT_BF16 ? qmm_wo_bw_launch_bf16(b, bits, (hipStream_t)stream)
                                   : qmm_wo_bw_launch_f16(b, bits, (hipStream_t)stream);
  }
  const Plan p = make_plan(M, N, K, zp != nullptr);
  WoGemmArgs a;
  a.x = x; a.w = (const uint8_t*)w_tiled; a.scale = scale; a.zp = zp; a.out = out;
  a.part = nullptr; a.part_xs = nullptr;
  a.M = (int)M; a.N = (int)N; a.K = (int)K;
  a.Kw = (int)K; a.x_dt = x_dt;
  a.G = xla_amd_qmm_tile_group(N, K, K, 8);
  a.k_per_split = p.k_per_split; a.split = p.split;
  // (results through LDS: the 128 x 256 tile with one 2-byte dtype throughout, whole 16-byte chunks per row of the
  // output and of the scales, and enough steps per item for the copying waves to write an item's results out during
  // the next one and to fetch the scales after that)
  a.stage_out = p.mt == 8 && p.ng == 4 && p.split == 1 && !zp && scale_dt == x_dt && dot_dt == x_dt && out_dt == x_dt &&
                store_dt == x_dt && N % 8 == 0 && K / 128 >= 12 && ((((uintptr_t)out) | ((uintptr_t)scale)) & 15) == 0;
  a.scale_dt = scale_dt; a.zp_dt = zp ? zp_dt : x_dt; a.dot_dt = dot_dt; a.out_dt = out_dt; a.store_dt = store_dt;
  if (p.split > 1) {
    const size_t need = ((size_t)p.split * (size_t)M * (size_t)N + (size_t)p.split * (size_t)M) * sizeof(float);
    if (!workspace || workspace_bytes < need)
      return qmm_fail(XLA_AMD_QMM_EINVAL, "weight_only_gemm: workspace of %zu bytes, need %zu", workspace ? workspace_bytes : (size_t)0, need);
    if ((uintptr_t)workspace & 15) return qmm_fail(XLA_AMD_QMM_EINVAL, "weight_only_gemm: workspace must be 16-byte aligned");
    a.part = (float*)workspace;
    a.part_xs = a.part + (size_t)p.split * (size_t)M * (size_t)N;
  }
  hipStream_t s = (hipStream_t)stream;
  int rc;
  if (x_dt == XLA_AMD_DT_BF16) rc = p.mt == 4 ? qmm_wo_launch_bf16_mt4(a, p.ng, s) : qmm_wo_launch_bf16_mt8(a, p.ng, s);
  else rc = p.mt == 4 ? qmm_wo_launch_f16_mt4(a, p.ng, s) : qmm_wo_launch_f16_mt8(a, p.ng, s);
  if (rc != XLA_AMD_QMM_OK) return rc;
  if (p.split > 1) {
    const int64_t threads = M * ((N + 3) / 4);
    hipLaunchKernelGGL(qmm_wo_gemm_finish_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, s, a, x_dt);
    rc = QMM_CHECK_LAUNCH("weight_only_gemm finish launch");
  }
  return rc;
}
#endif  // the unit with the entry points
