// W8A8 GEMM for gfx950: out[m,n] = epilogue( sum_k x_q[m,k] * w[n,k] ), int8
// operands, int32 accumulation on the matrix cores (v_mfma_i32_32x32x32_i8),
// both operands K-contiguous, tiles staged through LDS with a pipeline of two
// or three stages, scale epilogue fused.
//
// Tiling.  A workgroup of WM x WN waves owns a BM x BN tile of the output and
// walks K in steps of kBK = 128 bytes.  Each wave owns (BM/WM) x (BN/WN)
// outputs as a grid of 32x32 MFMA tiles whose int32 accumulators never leave
// registers.  LDS holds, per stage, the A tile [BM][128] and the B tile
// [BN][128] as 16-byte chunks with an XOR swizzle (chunk ^= (row/2) % 8) so
// that the 16 rows x 16 bytes read by a quarter wave for an MFMA operand land
// in 64 distinct banks, and so do the 2 rows x 8 chunks a quarter wave writes.
//
// MFMA operand/result mapping (A = x_q rows, B = w rows):
//   operand: lane l supplies row l%32, 16 bytes of k at chunk l/32 of a 32-byte step
//   result : acc[v] of lane l is D[8*(v/4) + 4*(l/32) + v%4][l%32]  (row = m, col = n)
// so one result register of a wave is 32 consecutive n of a row: coalesced stores.
#include "qmm_common.h"

int qmm_w8a8_generic_launch(const int8_t* xq, const int8_t* w, const void* x_scale,
                            const void* w_scale, const void* zp, const int32_t* x_sum, void* out,
                            int32_t* acc_out, int64_t M, int64_t N, int64_t K, int x_scale_dt,
                            int w_scale_dt, int zp_dt, int cvt_dt, int mid_dt, int zpo_dt,
                            int out_dt, hipStream_t stream);

namespace {

constexpr int kBK = 128;  // bytes (= int8 elements) of K per pipeline stage

struct GemmArgs {
  const int8_t* a;  // x_q [M,K]
  const int8_t* b;  // w   [N,K]
  const void* x_scale;
  const void* w_scale;
  const void* zp;
  const int32_t* x_sum;
  void* out;
  int32_t* acc_out;
  int M, N, K;
  int ldo;  // elements between rows of out / acc_out (N, or more when this launch covers a column range)
  int x_scale_dt, w_scale_dt, zp_dt, cvt_dt, mid_dt, zpo_dt, out_dt;
  int tiles_m, tiles_n;
};

__device__ __forceinline__ int swz(int row, int chunk) { return chunk ^ ((row >> 1) & 7); }

// EPI selects the epilogue: 0 = general (any dtype chain, zero point, raw
// accumulator output, partial tiles); 1/2/3 = all-f32 scale chain with bf16 /
// f16 / f32 output and nothing else, which whole tiles finish with a short
// branch-free loop (partial tiles of such a launch still take the general code).

// s_waitcnt immediate for "at most n vector-memory operations outstanding" (n < 64),
// leaving expcnt and lgkmcnt alone
constexpr int vmcnt_imm(int n) { return (n & 15) | ((n >> 4) << 14) | 0x0F70; }

// NS = LDS pipeline stages: the copies of NS - 1 K steps are in flight while one is
// computed.
// KG = K groups: the workgroup holds KG sets of WM x WN waves; set kg runs the whole
// pipeline (its own LDS stages) over the K steps kg, kg + KG, ..., and the sets' int32
// accumulators are added through LDS before the epilogue (exact in any order).  For
// launches with at most one small tile per CU, whose time is the length of the K loop.
template <int BM, int BN, int WM, int WN, int EPI, int NS, int KG>
__global__ void __launch_bounds__(KG * WM * WN * 64)
qmm_w8a8_gemm_kernel(GemmArgs g) {
  constexpr int T = WM * WN * 64;  // threads of one K group
  constexpr int TM = BM / WM, TN = BN / WN;  // wave tile
  constexpr int MI = TM / 32, NI = TN / 32;  // 32x32 MFMA tiles per wave
  constexpr int A_CH = BM * 8 / T, B_CH = BN * 8 / T;  // 16-byte chunks per thread per stage
  static_assert(BM % (WM * 32) == 0 && BN % (WN * 32) == 0, "wave tile must be a multiple of 32");
  static_assert((BM * 8) % T == 0 && (BN * 8) % T == 0, "tile rows must divide over the threads");
  extern __shared__ __attribute__((aligned(16))) char smem[];
  // wave-uniform values through readfirstlane: keeps LDS bases in scalar registers
  const int wave_all = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
  const int kg = KG > 1 ? wave_all / (WM * WN) : 0;  // K group of this wave
  const int wave = wave_all - kg * (WM * WN);         // wave, thread within the group
  const int tid = (int)threadIdx.x - kg * T, lane = tid & 63;
  char* sA = smem + kg * (NS * (BM + BN) * kBK);  // [NS][BM][128]
  char* sB = sA + NS * BM * kBK;                  // [NS][BN][128]
  const int wm = wave / WN, wn = wave % WN;

  // Workgroup -> tile.  Consecutive workgroup ids go to different XCDs (8 of
  // them, each with its own L2), so give every XCD a contiguous run of tiles
  // and walk a run down M first: the workgroups an XCD runs together then
  // share a few B (weight) panels and all A panels through its L2.
  int bid = blockIdx.x;
  const int ntiles = g.tiles_m * g.tiles_n;
  {
    const int per = (ntiles + 7) / 8;
    const int xcd = bid & 7, loc = bid >> 3;
    bid = xcd * per + loc;  // the grid has 8 * per workgroups; the excess ones have no tile
  }
  if (bid >= ntiles) return;
  const int tile_m = bid % g.tiles_m, tile_n = bid / g.tiles_m;
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int K = g.K;

  // Global -> LDS copies bypass registers (global_load_lds_dwordx4): a wave
  // instruction writes 64 x 16 bytes to consecutive LDS addresses (lane l at
  // base + 16 l), i.e. 8 rows x 8 chunks of a stage.  The XOR swizzle of the
  // LDS layout is therefore applied on the source side: LDS slot (row, c')
  // receives global chunk c' ^ (row/2 % 8) of that row.  Rows are clamped
  // into the matrix; chunks past K are zero-filled with a plain LDS store.
  const int8_t* ga[A_CH];
  const int8_t* gb[B_CH];
  int a_col[A_CH], b_col[B_CH];  // byte column of this lane's source chunk
  const int cslot = tid & 7;     // chunk slot within the 128-byte LDS row
  qmm_static_for<A_CH>([&](auto ic) {
    constexpr int i = ic;
    const int row = (i * T + tid) >> 3;
    a_col[i] = swz(row, cslot) * 16;
    ga[i] = g.a + (size_t)min(m0 + row, g.M - 1) * K + a_col[i];
  });
  qmm_static_for<B_CH>([&](auto ic) {
    constexpr int i = ic;
    const int row = (i * T + tid) >> 3;
    b_col[i] = swz(row, cslot) * 16;
    gb[i] = g.b + (size_t)min(n0 + row, g.N - 1) * K + b_col[i];
  });
  typedef __attribute__((address_space(3))) void* lds_ptr_t;
  auto stage_load = [&](int stage, int k0) __attribute__((always_inline)) {
    char* const wa = sA + stage * BM * kBK + wave * 1024;  // this wave's 1 KB slices: + i * T * 16
    char* const wb = sB + stage * BN * kBK + wave * 1024;
    if (k0 + kBK <= K) {  // whole step inside K (uniform): no per-lane conditions
      qmm_static_for<A_CH>([&](auto ic) {
        constexpr int i = ic;
        __builtin_amdgcn_global_load_lds((const void*)(ga[i] + k0), (lds_ptr_t)(wa + i * (T * 16)), 16, 0, 0);
      });
      qmm_static_for<B_CH>([&](auto ic) {
        constexpr int i = ic;
        __builtin_amdgcn_global_load_lds((const void*)(gb[i] + k0), (lds_ptr_t)(wb + i * (T * 16)), 16, 0, 0);
      });
    } else {  // last, partial step: chunks past K are zero-filled
      qmm_static_for<A_CH>([&](auto ic) {
        constexpr int i = ic;
        char* const dst = wa + i * (T * 16);
        if (k0 + a_col[i] < K) __builtin_amdgcn_global_load_lds((const void*)(ga[i] + k0), (lds_ptr_t)dst, 16, 0, 0);
        else *(i32x4*)(dst + lane * 16) = i32x4{0, 0, 0, 0};
      });
      qmm_static_for<B_CH>([&](auto ic) {
        constexpr int i = ic;
        char* const dst = wb + i * (T * 16);
        if (k0 + b_col[i] < K) __builtin_amdgcn_global_load_lds((const void*)(gb[i] + k0), (lds_ptr_t)dst, 16, 0, 0);
        else *(i32x4*)(dst + lane * 16) = i32x4{0, 0, 0, 0};
      });
    }
  };
  // This wave's copies of a stage have landed in LDS (they count as vector-memory
  // operations, which complete in order: at most the copies of the `later` full
  // stages issued after it may be outstanding), then the workgroup meets.
  constexpr int kStageOps = A_CH + B_CH;
  static_assert((NS - 2) * kStageOps < 64, "vmcnt is a 6-bit counter");
  // (A workgroup-scope release fence would make the compiler wait for every copy in
  // flight, since the copies are LDS writes; the asm barrier with a memory clobber keeps
  // the order of the LDS accesses around it, and the explicit counts do the waiting.)
  auto stage_sync = [&](bool later_stages_all_full) __attribute__((always_inline)) {
    if (NS > 2 && later_stages_all_full) __builtin_amdgcn_s_waitcnt(vmcnt_imm((NS - 2) * kStageOps));
    else __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
  };

  // Scales of this tile are fetched now so that their latency is hidden by the
  // main loop: thread t keeps x_scale[m0+t] and w_scale[n0+t] (BM, BN <= T).
  static_assert(BM <= T && BN <= T, "one scale per thread");
  const bool has_zp = g.zp != nullptr;
  const bool want_out = g.out != nullptr, want_acc = g.acc_out != nullptr;
  // (raw bits, loaded without a branch on the dtype: converting here would make
  // the kernel wait for each of these loads in turn before its first copy)
  uint32_t pre_xs = 0u, pre_ws = 0u, pre_zp = 0u;
  int pre_xsum = 0;
  if (want_out) {
    const int m = min(m0 + min(tid, BM - 1), g.M - 1);
    const int n = min(n0 + min(tid, BN - 1), g.N - 1);
    pre_xs = qmm_load_raw(g.x_scale, m, g.x_scale_dt);
    pre_ws = qmm_load_raw(g.w_scale, n, g.w_scale_dt);
    if (has_zp) {
      pre_xsum = g.x_sum[m];
      pre_zp = qmm_load_raw(g.zp, n, g.zp_dt);
    }
  }

  i32x16 acc[MI][NI];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NI; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0;

  const int lrow = lane & 31, lchunk = lane >> 5;
  // Copy `piece` (a 1 KB slice of this wave: A slices first) of a whole step into `stage`.
  auto copy_piece = [&](int stage, int k0, auto pc) __attribute__((always_inline)) {
    constexpr int p = pc;
    if constexpr (p < A_CH)
      __builtin_amdgcn_global_load_lds((const void*)(ga[p] + k0), (lds_ptr_t)(sA + stage * BM * kBK + wave * 1024 + p * (T * 16)), 16, 0, 0);
    else
      __builtin_amdgcn_global_load_lds((const void*)(gb[p - A_CH] + k0), (lds_ptr_t)(sB + stage * BN * kBK + wave * 1024 + (p - A_CH) * (T * 16)), 16, 0, 0);
  };
  // One K step out of LDS: 4 sub-steps of 32 bytes.  The operand fragments of sub-step ks+1 are read while the
  // MFMAs of sub-step ks run (two register sets), one read after each MFMA, and the copies of the step NS - 1
  // ahead are issued the same way, one after each of the step's first MFMAs.  A wave issues in order: issued as
  // a run (6 reads before a sub-step's MFMAs, 8 copies with their addresses at the start of the step) they keep
  // the wave from issuing MFMAs for that long, and the two waves of a SIMD, which leave the step's barrier
  // together, do it at the same moment.
  // COPY: 0 = no copies, 1 = a whole step (spread), 2 = the last, partial step (as a run: its chunks past K are
  // zero-filled under per-lane conditions).
  // Tiles with few MFMAs per step are bound by the latency of their copies and keep the runs (compute_runs below:
  // the copies go out at once, as early as possible; 32 x 32 tiles at M = 32 against 4096 x 14336 take 15.2 us so
  // and 16.6 - 18.7 us with any part of this order).
  constexpr int kPerSub = MI * NI;
  constexpr bool kSpread = kStageOps <= 2 * kPerSub;
  auto compute = [&](int stage, int COPY, int cstage, int ck0) __attribute__((always_inline)) {
    const char* a_base = sA + stage * BM * kBK + (wm * TM) * kBK;
    const char* b_base = sB + stage * BN * kBK + (wn * TN) * kBK;
    i32x4 af[2][MI], bf[2][NI];
    auto read_frag = [&](auto setc, auto ksc, auto nc) __attribute__((always_inline)) {  // fragment n: A tiles, then B tiles
      constexpr int set = setc, ks = ksc, n = nc;
      const int c = 2 * ks + lchunk;
      if constexpr (n < MI) {
        const int row = n * 32 + lrow;
        af[set][n] = *(const i32x4*)(a_base + row * kBK + swz(wm * TM + row, c) * 16);
      } else {
        const int row = (n - MI) * 32 + lrow;
        bf[set][n - MI] = *(const i32x4*)(b_base + row * kBK + swz(wn * TN + row, c) * 16);
      }
    };
    qmm_static_for<MI + NI>([&](auto nc) { read_frag(qmm_const<0>{}, qmm_const<0>{}, nc); });
    __builtin_amdgcn_sched_barrier(0);
    if (COPY == 2) stage_load(cstage, ck0);
    qmm_static_for<kBK / 32>([&](auto ksc) {
      constexpr int ks = ksc, set = ks & 1;
      constexpr bool kMore = ks + 1 < kBK / 32;
      qmm_static_for<MI>([&](auto ic) {
        constexpr int i = ic;
        qmm_static_for<NI>([&](auto jc) {
          constexpr int j = jc, n = i * NI + j, at = ks * kPerSub + n;
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[set][i], bf[set][j], acc[i][j], 0, 0, 0);
          if constexpr (kMore && n < MI + NI) read_frag(qmm_const<set ^ 1>{}, qmm_const<ks + 1>{}, qmm_const<n>{});
          if constexpr (at < kStageOps) { if (COPY == 1) copy_piece(cstage, ck0, qmm_const<at>{}); }
          __builtin_amdgcn_sched_barrier(0);
        });
      });
      // (tiles with fewer MFMAs than fragments per sub-step: the rest of the reads)
      if constexpr (kMore && kPerSub < MI + NI) {
        qmm_static_for<MI + NI - kPerSub>([&](auto nc) { read_frag(qmm_const<set ^ 1>{}, qmm_const<ks + 1>{}, qmm_const<kPerSub + (int)nc>{}); });
        __builtin_amdgcn_sched_barrier(0);
      }
    });
  };

  auto compute_runs = [&](int stage, auto&& after_first_reads) __attribute__((always_inline)) {
    const char* a_base = sA + stage * BM * kBK + (wm * TM) * kBK;
    const char* b_base = sB + stage * BN * kBK + (wn * TN) * kBK;
    i32x4 af[2][MI], bf[2][NI];
    auto read_frags = [&](auto setc, auto ksc) __attribute__((always_inline)) {
      constexpr int set = setc, ks = ksc;
      const int c = 2 * ks + lchunk;
      qmm_static_for<MI>([&](auto ic) {
        constexpr int i = ic;
        const int row = i * 32 + lrow;
        af[set][i] = *(const i32x4*)(a_base + row * kBK + swz(wm * TM + row, c) * 16);
      });
      qmm_static_for<NI>([&](auto jc) {
        constexpr int j = jc;
        const int row = j * 32 + lrow;
        bf[set][j] = *(const i32x4*)(b_base + row * kBK + swz(wn * TN + row, c) * 16);
      });
    };
    read_frags(qmm_const<0>{}, qmm_const<0>{});
    __builtin_amdgcn_sched_barrier(0);
    after_first_reads();  // the next stage's copies are issued while those reads are in flight
    qmm_static_for<kBK / 32>([&](auto ksc) {
      constexpr int ks = ksc, set = ks & 1;
      if constexpr (ks + 1 < kBK / 32) read_frags(qmm_const<set ^ 1>{}, qmm_const<ks + 1>{});
      // keep those reads ahead of this sub-step's MFMAs (the scheduler would
      // otherwise sink each read next to its first use to save registers)
      __builtin_amdgcn_sched_barrier(0);
      qmm_static_for<MI>([&](auto ic) {
        constexpr int i = ic;
        qmm_static_for<NI>([&](auto jc) {
          constexpr int j = jc;
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[set][i], bf[set][j], acc[i][j], 0, 0, 0);
        });
      });
    });
  };

  // Steps 0 .. NS-2 are copied ahead; step kt then computes stage kt % NS while the
  // copy of step kt + NS - 1 goes into the stage that step kt - 1 read, which every
  // wave has left at the barrier of step kt.  When step kt is waited for, the steps
  // issued after it are kt+1 .. min(kt + NS - 2, last): they are NS - 2 full stages
  // unless they include the last step, which may be partial (fewer copies per wave).
  // With K groups, "step kt" below is the group's own kt-th step, global step
  // kt * KG + kg; every wave of the workgroup runs the same number of iterations (and
  // barriers), a group that has run out of steps just meets the others.
  const int ksteps_all = (K + kBK - 1) / kBK;
  const int ksteps = (ksteps_all - kg + KG - 1) / KG;   // this group's steps
  const int kiters = (ksteps_all + KG - 1) / KG;        // iterations of every group
  auto step_k0 = [&](int kt) { return (kt * KG + kg) * kBK; };
#pragma unroll
  for (int s = 0; s < NS - 1; ++s)
    if (s < ksteps) stage_load(s, step_k0(s));
  int cur = 0, nxt = NS - 1;
  for (int kt = 0; kt < kiters; ++kt) {
    stage_sync(kt + NS - 2 < ksteps - 1);
    if (KG == 1 || kt < ksteps) {
      const int ck0 = step_k0(kt + NS - 1);
      if constexpr (kSpread) {
        compute(cur, kt + NS - 1 >= ksteps ? 0 : ck0 + kBK <= K ? 1 : 2, nxt, ck0);
      } else {
        compute_runs(cur, [&]() __attribute__((always_inline)) {
          if (kt + NS - 1 < ksteps) stage_load(nxt, ck0);
        });
      }
    }
    cur = cur + 1 == NS ? 0 : cur + 1;
    nxt = nxt + 1 == NS ? 0 : nxt + 1;
  }

  // Epilogue, staged through LDS so that (a) the code stays small (the
  // accumulators are register-indexed by constants only in the 16*MI*NI
  // ds_write instructions; everything else is a rolled loop) and (b) global
  // stores are row-contiguous vectors instead of one element per lane.
  constexpr int kEpStride = TN + 8;  // ints per staged row: +8 keeps rows 16-byte aligned and
                                     // shifts the second half-wave (4 rows down) by 32 banks
  static_assert(4 * WM * WN * 32 * kEpStride + 4 * 4 * (BM + BN) <= NS * (BM + BN) * kBK,
                "epilogue staging must fit in the pipeline's LDS");
  __syncthreads();  // every wave is done reading the last pipeline stage
  if constexpr (KG > 1) {
    // Groups 1 .. KG-1 hand their accumulators to group 0, one after the other, through
    // LDS ([register][thread]: consecutive lanes, consecutive words).  Every wave takes
    // part in every barrier; the groups other than 0 leave after the last one.
    static_assert(MI * NI * 16 * T * 4 <= NS * (BM + BN) * kBK, "reduction buffer must fit in one group's stages");
    int* s_red = (int*)smem + tid;
    for (int src = 1; src < KG; ++src) {
      if (kg == src) {
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
          for (int j = 0; j < NI; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) s_red[((i * NI + j) * 16 + v) * T] = acc[i][j][v];
      }
      __syncthreads();
      if (kg == 0) {
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
          for (int j = 0; j < NI; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] += s_red[((i * NI + j) * 16 + v) * T];
      }
      __syncthreads();
    }
  }
  float* s_xs = (float*)smem;          // [BM] activation scale
  float* s_xsum = s_xs + BM;           // [BM] round_zpo(float(x_sum))
  float* s_ws = s_xsum + BM;           // [BN] weight scale
  float* s_zp = s_ws + BN;             // [BN] zero point
  int* s_ep = (int*)(s_zp + BN) + wave * (32 * kEpStride);  // per-wave [32][kEpStride]
  if (kg == 0 && tid < BM) {
    s_xs[tid] = qmm_from_raw(pre_xs, g.x_scale_dt);
    s_xsum[tid] = has_zp ? qmm_round_dt((float)pre_xsum, g.zpo_dt) : 0.f;
  }
  if (kg == 0 && tid < BN) {
    s_ws[tid] = qmm_from_raw(pre_ws, g.w_scale_dt);
    s_zp[tid] = has_zp ? qmm_from_raw(pre_zp, g.zp_dt) : 0.f;
  }
  __syncthreads();
  if (KG > 1 && kg != 0) return;  // no barrier below this line
  constexpr int kLanesPerRow = TN / 4;               // each lane finishes 4 consecutive n
  constexpr int kPasses = 32 * kLanesPerRow / 64;    // passes over a 32-row block
  constexpr int kRowsPerPass = 64 / kLanesPerRow;

  if constexpr (EPI != 0) {
    if (m0 + BM <= g.M && n0 + BN <= g.N) {
      // Whole tile, f32 chain: out = cast((float(acc) * w_scale) * x_scale).  The lane's
      // 4 columns are the same in every pass, so their scales stay in registers.
      // (when the lanes of a row divide the wave, a lane's 4 columns are the same
      // in every pass and their scales stay in registers)
      constexpr bool kFixedCols = 64 % kLanesPerRow == 0;
      const int c4f = lane % kLanesPerRow, prow = lane / kLanesPerRow;
      const f32x4 wsf = *(const f32x4*)(s_ws + wn * TN + c4f * 4);
      qmm_static_for<MI>([&](auto ic) {
        constexpr int i = ic;
        qmm_static_for<NI>([&](auto jc) {
          constexpr int j = jc;
          qmm_static_for<16>([&](auto vc) {
            constexpr int v = vc;
            s_ep[(8 * (v >> 2) + 4 * lchunk + (v & 3)) * kEpStride + j * 32 + lrow] = acc[i][j][v];
          });
        });
        const int rbase = wm * TM + i * 32;
#pragma unroll 4
        for (int p = 0; p < kPasses; ++p) {
          int row, c4;
          f32x4 ws;
          if constexpr (kFixedCols) {
            row = p * kRowsPerPass + prow; c4 = c4f; ws = wsf;
          } else {
            const int idx = p * 64 + lane;
            row = idx / kLanesPerRow; c4 = idx % kLanesPerRow;
            ws = *(const f32x4*)(s_ws + wn * TN + c4 * 4);
          }
          const i32x4 a = *(const i32x4*)(s_ep + row * kEpStride + c4 * 4);
          const float xs = s_xs[rbase + row];
          const float v0 = ((float)a[0] * ws[0]) * xs, v1 = ((float)a[1] * ws[1]) * xs;
          const float v2 = ((float)a[2] * ws[2]) * xs, v3 = ((float)a[3] * ws[3]) * xs;
          const size_t idx0 = (size_t)(m0 + rbase + row) * g.ldo + (n0 + wn * TN + c4 * 4);
          // (streaming stores: the output is written once and not read here, it should
          // not push the operands out of L2)
          if constexpr (EPI == 3) {
            __builtin_nontemporal_store(f32x4{v0, v1, v2, v3}, (f32x4*)((float*)g.out + idx0));
          } else if constexpr (EPI == 1) {
            const uint32_t lo = qmm_f32_to_bf16(v0) | ((uint32_t)qmm_f32_to_bf16(v1) << 16);
            const uint32_t hi = qmm_f32_to_bf16(v2) | ((uint32_t)qmm_f32_to_bf16(v3) << 16);
            __builtin_nontemporal_store(i32x2{(int)lo, (int)hi}, (i32x2*)((uint16_t*)g.out + idx0));
          } else {
            const uint32_t lo = qmm_f32_to_f16(v0) | ((uint32_t)qmm_f32_to_f16(v1) << 16);
            const uint32_t hi = qmm_f32_to_f16(v2) | ((uint32_t)qmm_f32_to_f16(v3) << 16);
            __builtin_nontemporal_store(i32x2{(int)lo, (int)hi}, (i32x2*)((uint16_t*)g.out + idx0));
          }
        }
      });
      return;
    }
  }
  const bool simple = g.cvt_dt == XLA_AMD_DT_F32 && g.mid_dt == XLA_AMD_DT_F32 && !has_zp;
  const bool n_vec = (g.ldo % 4) == 0 && (g.N % 4) == 0;  // rows of out start 8/16-byte aligned, no ragged last group
  // Finishes one staged 32 x TN block whose first row is global row mb.
  auto finish_block = [&](int mb, int row_off) {
    for (int p = 0; p < kPasses; ++p) {
      const int idx = p * 64 + lane;
      const int row = idx / kLanesPerRow, c4 = idx % kLanesPerRow;
      const int m = mb + row, n = n0 + wn * TN + c4 * 4;
      if (m >= g.M || n >= g.N) continue;
      const i32x4 a = *(const i32x4*)(s_ep + row * kEpStride + c4 * 4);
      const size_t idx0 = (size_t)m * g.ldo + n;
      const int nvalid = min(4, g.N - n);
      if (want_acc) {
        if (n_vec) *(i32x4*)(g.acc_out + idx0) = a;
        else for (int e = 0; e < nvalid; ++e) g.acc_out[idx0 + e] = a[e];
      }
      if (!want_out) continue;
      const float xs = s_xs[row_off + row];
      const f32x4 ws = *(const f32x4*)(s_ws + wn * TN + c4 * 4);
      float val[4];
      if (simple) {
#pragma unroll
        for (int e = 0; e < 4; ++e) val[e] = ((float)a[e] * ws[e]) * xs;
      } else {
        const float xsum_f = s_xsum[row_off + row];
        const f32x4 zp4 = *(const f32x4*)(s_zp + wn * TN + c4 * 4);
        for (int e = 0; e < 4; ++e) {
          float v = qmm_round_dt((float)a[e], g.cvt_dt);
          v = qmm_round_dt(v * ws[e], g.mid_dt);
          if (has_zp) v = qmm_round_dt(v - qmm_round_dt(xsum_f * zp4[e], g.zpo_dt), g.mid_dt);
          val[e] = v * xs;
        }
      }
      if (g.out_dt == XLA_AMD_DT_F32) {
        if (n_vec) *(f32x4*)((float*)g.out + idx0) = f32x4{val[0], val[1], val[2], val[3]};
        else for (int e = 0; e < nvalid; ++e) ((float*)g.out)[idx0 + e] = val[e];
      } else {
        uint16_t h[4];
#pragma unroll
        for (int e = 0; e < 4; ++e)
          h[e] = g.out_dt == XLA_AMD_DT_BF16 ? qmm_f32_to_bf16(val[e]) : qmm_f32_to_f16(val[e]);
        if (n_vec) {
          i32x2 pk = {(int)(h[0] | ((uint32_t)h[1] << 16)), (int)(h[2] | ((uint32_t)h[3] << 16))};
          *(i32x2*)((uint16_t*)g.out + idx0) = pk;
        } else {
          for (int e = 0; e < nvalid; ++e) ((uint16_t*)g.out)[idx0 + e] = h[e];
        }
      }
    }
  };

  qmm_static_for<MI>([&](auto ic) {
    constexpr int i = ic;
    qmm_static_for<NI>([&](auto jc) {
      constexpr int j = jc;
      qmm_static_for<16>([&](auto vc) {
        constexpr int v = vc;
        s_ep[(8 * (v >> 2) + 4 * lchunk + (v & 3)) * kEpStride + j * 32 + lrow] = acc[i][j][v];
      });
    });
    // LDS operations of one wave complete in order: the reads below see the writes above.
    finish_block(m0 + wm * TM + i * 32, wm * TM + i * 32);
  });
}

template <int BM, int BN, int WM, int WN, int EPI, int NS, int KG>
int launch_tile_epi(GemmArgs g, hipStream_t stream) {
  g.tiles_m = (g.M + BM - 1) / BM;
  g.tiles_n = (g.N + BN - 1) / BN;
  const int ntiles = g.tiles_m * g.tiles_n;
  const int per = (ntiles + 7) / 8;
  const unsigned grid = (unsigned)(per * 8);
  constexpr size_t lds = KG * NS * (size_t)(BM + BN) * kBK;
  static_assert(lds <= 160 * 1024 && KG * WM * WN * 64 <= 1024, "workgroup must fit a CU");
  auto kern = qmm_w8a8_gemm_kernel<BM, BN, WM, WN, EPI, NS, KG>;
  static std::atomic<uint64_t> lds_set{0};
  const int rc = qmm_set_max_lds((const void*)kern, (int)lds, lds_set, "w8a8_gemm hipFuncSetAttribute");
  if (rc != XLA_AMD_QMM_OK) return rc;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(KG * WM * WN * 64), lds, stream, g);
  return QMM_CHECK_LAUNCH("w8a8_gemm launch");
}

// The short epilogue applies when the scale chain is all f32, there is no zero
// point, no raw-accumulator output and rows of out are vector-aligned.
template <int BM, int BN, int WM, int WN, int NS = 2, int KG = 1>
int launch_tile(const GemmArgs& g, hipStream_t stream) {
  const bool fast = g.out && !g.acc_out && !g.zp && g.cvt_dt == XLA_AMD_DT_F32 &&
                    g.mid_dt == XLA_AMD_DT_F32 && (g.N % 4) == 0 && (g.ldo % 4) == 0 && (((uintptr_t)g.out) & 15) == 0;
  if (fast && g.out_dt == XLA_AMD_DT_BF16) return launch_tile_epi<BM, BN, WM, WN, 1, NS, KG>(g, stream);
  if (fast && g.out_dt == XLA_AMD_DT_F16) return launch_tile_epi<BM, BN, WM, WN, 2, NS, KG>(g, stream);
  if (fast && g.out_dt == XLA_AMD_DT_F32) return launch_tile_epi<BM, BN, WM, WN, 3, NS, KG>(g, stream);
  return launch_tile_epi<BM, BN, WM, WN, 0, NS, KG>(g, stream);
}

}  // namespace

// Estimated time in us of the launches that cover an output, fitted to measurements at
// K = 128 ... 14336: a launch costs kLaunchUs, and each round of tiles over the 256 CUs
// costs a part per tile (prologue, epilogue) plus a part proportional to K.  A round
// that is only partly full costs a whole one.
struct TileCost { double per_round_us, per_k4096_us; };
static constexpr double kLaunchUs = 4.0;
static constexpr TileCost kCost256 = {11.0, 52.0}, kCost192 = {8.0, 39.0}, kCost128x256 = {9.0, 27.0},
                          kCost128 = {8.0, 14.0};
static double rounds_us(const TileCost& c, int64_t tiles, int64_t K) {
  return (double)((tiles + 255) / 256) * (c.per_round_us + c.per_k4096_us * (double)K / 4096.0);
}

// Columns covered by n1 tiles of 256 followed by n2 tiles of 192 (two launches when
// both are present): the split with the least estimated time.  2048 x 14336:
// 8 x 56 = 448 tiles = 2 rounds becomes 8 x 32 + 8 x 32 = 1 + 0.75 rounds.
static double best_column_split(int64_t M, int64_t N, int64_t K, int64_t* n1_out) {
  const int64_t mt = (M + 255) / 256;
  int64_t best_n1 = (N + 255) / 256;
  double best = kLaunchUs + rounds_us(kCost256, mt * best_n1, K);
  for (int64_t n1 = N / 256; n1 >= 0; --n1) {
    const int64_t n2 = (N - n1 * 256 + 191) / 192;
    if (n2 <= 0) continue;
    const double cost = (n1 > 0 ? 2 : 1) * kLaunchUs + rounds_us(kCost256, mt * n1, K) +
                        rounds_us(kCost192, mt * n2, K);
    if (cost < best - 1e-9) { best = cost; best_n1 = n1; }
  }
  *n1_out = best_n1;
  return best;
}

// Tile choice by shape: 64 x 64 tiles (several workgroups resident per CU, which hides
// the latency of their short K steps) while there are at most three per CU: measured
// faster than one round of 128 x 128 tiles up to there, for K = 2048 ... 14336 (at 208 to 256
// tiles of 128 x 128, three stages, the larger tile is 8 % faster).  Larger
// problems take the tile class with the least estimated time.
static void choose_tile(int64_t M, int64_t N, int64_t K, int* bm, int* bn) {
  auto tiles = [&](int a, int b) { return ((M + a - 1) / a) * ((N + b - 1) / b); };
  // Few output tiles: 64 x 64 tiles would leave half of the CUs or more without work.  Such
  // a launch is bound by what one CU can copy from global memory, so spread it over twice
  // the tiles, each with four K groups: 32 x 32 for decode-sized M (half the activation rows
  // fetched per tile as well) and while that is at most one tile per CU (64 rows against 4096
  // channels: 8.1 against 8.7 us; 128 rows against 1280 x 8192: 10.6 against 12.7 us), else 64 x 32.
  if (tiles(64, 64) <= 128) { *bm = (M <= 32 || tiles(32, 32) <= 256) ? 32 : 64; *bn = 32; return; }
  if (M <= 64 || tiles(64, 64) <= 768) { *bm = 64; *bn = 64; return; }
  int64_t n1;
  const double c256 = M > 128 && N > 128 ? best_column_split(M, N, K, &n1) : 1e30;
  const double c128x256 = N > 128 ? kLaunchUs + rounds_us(kCost128x256, tiles(128, 256), K) : 1e30;
  const double c128 = kLaunchUs + rounds_us(kCost128, tiles(128, 128), K);
  if (c256 <= c128x256 && c256 <= c128) { *bm = 256; *bn = 256; return; }
  if (c128x256 <= c128) { *bm = 128; *bn = 256; return; }
  *bm = 128; *bn = 128;
}

extern "C" int xla_amd_qmm_w8a8_tile(int64_t M, int64_t N, int64_t K, int32_t* tile_mnk) {
  if (!tile_mnk || M <= 0 || N <= 0 || K <= 0) return qmm_fail(XLA_AMD_QMM_EINVAL, "w8a8_tile: bad arguments");
  int bm, bn;
  choose_tile(M, N, K, &bm, &bn);
  tile_mnk[0] = bm; tile_mnk[1] = bn; tile_mnk[2] = kBK;
  return XLA_AMD_QMM_OK;
}

extern "C" int xla_amd_qmm_w8a8_gemm(const int8_t* x_q, const int8_t* w, const void* x_scale,
                                     const void* w_scale, const void* zp, const int32_t* x_sum,
                                     void* out, int32_t* acc_out, int64_t M, int64_t N, int64_t K,
                                     int x_scale_dt, int w_scale_dt, int zp_dt, int cvt_dt,
                                     int mid_dt, int zpo_dt, int out_dt, int block_m, int block_n,
                                     void* stream) {
  if (!x_q || !w) return qmm_fail(XLA_AMD_QMM_EINVAL, "w8a8_gemm: null operand");
  if (!out && !acc_out) return qmm_fail(XLA_AMD_QMM_EINVAL, "w8a8_gemm: neither out nor acc_out given");
  if (out && (!x_scale || !w_scale)) return qmm_fail(XLA_AMD_QMM_EINVAL, "w8a8_gemm: null scale");
  if ((zp != nullptr) != (x_sum != nullptr) && out)
    return qmm_fail(XLA_AMD_QMM_EINVAL, "w8a8_gemm: zp and x_sum must be given together");
  if (M < 0 || N <= 0 || K <= 0) return qmm_fail(XLA_AMD_QMM_EINVAL, "w8a8_gemm: bad sizes");
  if (M > (1 << 30) || N > (1 << 30) || K > (1 << 30))
    return qmm_fail(XLA_AMD_QMM_EUNSUPPORTED, "w8a8_gemm: dimension too large");
  if (out && (!qmm_valid_dt(x_scale_dt) || !qmm_valid_dt(w_scale_dt) || !qmm_valid_dt(cvt_dt) ||
              !qmm_valid_dt(mid_dt) || !qmm_valid_dt(out_dt) ||
              (zp && (!qmm_valid_dt(zp_dt) || !qmm_valid_dt(zpo_dt)))))
    return qmm_fail(XLA_AMD_QMM_EINVAL, "w8a8_gemm: bad dtype enum");
  if (M == 0) return XLA_AMD_QMM_OK;
  hipStream_t s = (hipStream_t)stream;
  const bool fast = (K % 16 == 0) && ((((uintptr_t)x_q | (uintptr_t)w) & 15) == 0);
  if (!fast)
    return qmm_w8a8_generic_launch(x_q, w, x_scale, w_scale, zp, x_sum, out, acc_out, M, N, K,
                                   x_scale_dt, w_scale_dt, zp_dt, cvt_dt, mid_dt, zpo_dt, out_dt, s);
  GemmArgs g;
  g.a = x_q; g.b = w; g.x_scale = x_scale; g.w_scale = w_scale; g.zp = out ? zp : nullptr;
  g.x_sum = x_sum; g.out = out; g.acc_out = acc_out;
  g.M = (int)M; g.N = (int)N; g.K = (int)K; g.ldo = (int)N;
  g.x_scale_dt = x_scale_dt; g.w_scale_dt = w_scale_dt; g.zp_dt = zp_dt; g.cvt_dt = cvt_dt;
  g.mid_dt = mid_dt; g.zpo_dt = zpo_dt; g.out_dt = out_dt;
  g.tiles_m = g.tiles_n = 0;
  int bm = block_m, bn = block_n;
  if (bm == 0 && bn == 0) choose_tile(M, N, K, &bm, &bn);
  // 256x256: 8 waves (2 x 4, wave tile 128 x 64): two waves per SIMD, so that one wave's LDS and
  // barrier waits are the other's MFMA slots (measured 128 us against 154 us with 4 waves of 128 x 128)
  if (bm == 256 && bn == 256) {
    int64_t best_n1;
    best_column_split(M, N, K, &best_n1);
    const int64_t N1 = best_n1 * 256 < N ? best_n1 * 256 : N;
    int rc = XLA_AMD_QMM_OK;
    if (N1 > 0) {
      GemmArgs g1 = g;
      g1.N = (int)N1;
      rc = launch_tile<256, 256, 2, 4>(g1, s);
      if (rc != XLA_AMD_QMM_OK) return rc;
    }
    if (N1 < N) {
      GemmArgs g2 = g;
      g2.N = (int)(N - N1);
      g2.b = w + (size_t)N1 * K;
      if (g.w_scale) g2.w_scale = (const char*)g.w_scale + (size_t)N1 * qmm_dt_size(w_scale_dt);
      if (g.zp) g2.zp = (const char*)g.zp + (size_t)N1 * qmm_dt_size(zp_dt);
      if (g.out) g2.out = (char*)g.out + (size_t)N1 * qmm_dt_size(out_dt);
      if (g.acc_out) g2.acc_out = g.acc_out + N1;
      rc = launch_tile<256, 192, 4, 2>(g2, s);
    }
    return rc;
  }
  if (bm == 128 && bn == 256) return launch_tile<128, 256, 2, 4>(g, s);  // 8 waves, wave tile 64 x 64
  if (bm == 128 && bn == 128) {
    // one workgroup per CU at most: LDS is free for a third stage (two fit a CU with two stages)
    const int64_t tiles = ((M + 127) / 128) * ((N + 127) / 128);
    return tiles <= 256 ? launch_tile<128, 128, 2, 2, 3>(g, s) : launch_tile<128, 128, 2, 2, 2>(g, s);
  }
  if (bm == 64 && bn == 64) {
    // Up to two workgroups per CU there is little else on a CU to cover the latency of a
    // K step's copies with, and a 64 x 64 tile has little MFMA work per step: a third LDS
    // stage keeps two steps' copies in flight (4096 x 14336 at M <= 256: 55 -> 34 us).
    // With more workgroups per CU the LDS is better spent on residency.
    // At most one workgroup per CU and a long K: two K groups halve the K loop.
    const int64_t tiles = ((M + 63) / 64) * ((N + 63) / 64);
    if (tiles <= 256 && K >= 1024) return launch_tile<64, 64, 2, 2, 3, 2>(g, s);
    return tiles <= 512 ? launch_tile<64, 64, 2, 2, 3>(g, s) : launch_tile<64, 64, 2, 2, 2>(g, s);
  }
  if (bm == 64 && bn == 32) {  // two waves per K group
    return K >= 1024 ? launch_tile<64, 32, 2, 1, 3, 4>(g, s) : launch_tile<64, 32, 2, 1, 3, 1>(g, s);
  }
  if (bm == 32 && bn == 32) {
    // one wave per K group; with a short K the groups are not worth their reduction
    return K >= 1024 ? launch_tile<32, 32, 1, 1, 3, 4>(g, s) : launch_tile<32, 32, 1, 1, 3, 1>(g, s);
  }
  return qmm_fail(XLA_AMD_QMM_EUNSUPPORTED, "w8a8_gemm: no kernel for tile %dx%d", bm, bn);
}
