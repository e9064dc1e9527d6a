// Weight-streaming GEMV / skinny GEMM for weight-only quantized linear layers
// on gfx950.  HBM-bound: every weight byte is read from memory exactly once.
//
// Memory access.  The weights are read from a tiled copy made once per weight
// (xla_amd_qmm_tile_weight): for every 16 channels x 128 columns one block
// whose bytes are already in MFMA operand order (lane = channel, 32 consecutive
// k per lane), blocks of a channel group consecutive along K.  A wave therefore
// streams one contiguous region with 1 KB loads that land directly in operand
// registers: no transposition, no LDS traffic for weights.  The activations are
// copied global -> LDS without passing registers, a chunk of up to 160 KB of x
// columns at a time (all of x for 16 rows x 4096 bf16 columns), XOR-swizzled so
// that the operand reads are free of bank conflicts, and stay there while the
// weights stream by.
//
// Work split.  A workgroup has 4 waves arranged as RW row groups x KW k-splits
// (RW * KW == 4).  It owns 16*RW consecutive output channels.  K is walked in
// steps of KS columns (512 B of weight row: 512 columns of int8, 1024 of int4);
// wave (rw, kw) handles steps kw, kw + KW, ...  Large N uses RW = 4 (no
// cross-wave reduction at all); small N trades row groups for k-splits so that
// the grid still covers the chip.
//
// Synchronisation.  The workgroup meets only when the resident x columns are
// replaced.  In between nothing is shared but read-only x, so every wave runs
// at its own pace: wait for its weight loads (one step in flight, each
// fragment re-loaded as soon as it has been used), multiply.  The waves
// of a compute unit drift apart, and the memory waits of one overlap the LDS
// traffic and arithmetic of the others; a barrier per step would instead make
// each step as slow as its slowest wave.
//
// MFMA mapping.  Lane l is (r = l%16, g = l/16).  For a sub-step of 128
// columns the lane supplies, for weight row r and for x row r of each 16-row
// tile, the 32 columns k0+32g..k0+32g+31, as four 16x16x32 MFMAs of 8 columns
// per lane (A = weights, B = x^T).  Both operands use the same columns per
// lane, so the k-order inside the instruction does not matter.  D[i][j] lands
// in lane (j + 16*(i/4)), register i%4: channel 4g + v, x row r.
#include "qmm_common.h"

// This file is compiled once per activation dtype (-DQMM_SKINNY_XT=0|1|2, the
// XLA_AMD_DT_* value) so that the three sets of kernels build in parallel; the
// bf16 unit also holds the C entry point, which calls into the other two.
#ifndef QMM_SKINNY_XT
#error "compile with -DQMM_SKINNY_XT=<XLA_AMD_DT_* value>"
#endif

#include "qmm_frag.h"
#include "qmm_skinny.h"

// Diagnostic build (-DQMM_SKINNY_TIMELINE, a library of its own; see xla_amd/build.py): every wave
// notes the time (the chip-wide 100 MHz counter) at fixed points of the kernel - entry, first
// weights requested / landed, first x chunk there, each step, end - in LDS and writes its notes
// to qmm_tl_buf when it leaves; xla_amd_qmm_timeline_read copies them to the host.  The regular
// build compiles none of it.
#ifdef QMM_SKINNY_TIMELINE
constexpr int kTlSlots = 32;        // notes per wave
constexpr int kTlWaves = 12;        // waves per workgroup at most
constexpr int kTlBlocks = 2048;     // workgroups per launch at most (larger launches are not recorded)
constexpr int kTlLdsBytes = kTlWaves * kTlSlots * 8;
__device__ uint64_t qmm_tl_buf[kTlBlocks * kTlWaves * kTlSlots];
// (no branch around a note: every lane stores the same value to the same LDS address; a branch
// inside the main loop would make the compiler's wait counts for the weight ring conservative)
// (explicit LDS pointers: a generic pointer would make these flat stores, which count as global
// memory operations too and turn every wait of the ring into a wait for all loads)
typedef volatile __attribute__((address_space(3))) uint64_t* qmm_tl_ptr_t;
#define QMM_TL_AREA ((qmm_tl_ptr_t)(__attribute__((address_space(3))) char*)smem + a.tl_off / 8)
#define QMM_TL(i) \
  do { QMM_TL_AREA[wave * kTlSlots + (i)] = __builtin_amdgcn_s_memrealtime(); } while (0)
#define QMM_TL_CLK(i) do { QMM_TL_AREA[wave * kTlSlots + (i)] = __builtin_readcyclecounter(); } while (0)
#define QMM_TL_DUMP()                                                                                    \
  do {                                                                                                   \
    QMM_TL_CLK(27);                                                                                      \
    if (lane < kTlSlots)                                                                                 \
      qmm_tl_buf[((size_t)(blockIdx.y * gridDim.x + blockIdx.x) * kTlWaves + wave) * kTlSlots + lane] =  \
          QMM_TL_AREA[wave * kTlSlots + lane];                                                           \
  } while (0)
#else
#define QMM_TL(i) do {} while (0)
#define QMM_TL_CLK(i) do {} while (0)
#define QMM_TL_DUMP() do {} while (0)
#endif

namespace {

using namespace qmm_frag;

constexpr int kWaves = 4;         // waves per workgroup of the standard shape
constexpr int kWSeg = 512;        // weight bytes per row per step of the standard shape
constexpr int kLdsLimit = 144 * 1024;  // of x in LDS; the 16 KB above it hold the blockwise scales of the resident chunks

// Reduction over the k-splits of a workgroup.
constexpr int kRedNone = 0;    // blockwise, KW == 1: nothing to reduce
constexpr int kRedRaw = 1;     // per-channel (C == K, any KW): raw dot products and x sums are summed, then scaled
constexpr int kRedScaled = 2;  // blockwise, KW > 1, whole blocks per step (KS % C == 0): scaled block results are summed

// NW computing waves per workgroup; WSEG weight bytes per row per step.  Launches use 4 waves and
// 512 bytes, or 8 waves for outputs of more than 16384 channels (see launch_split); an 8-wave
// shape with 256-byte steps measured slower and is not dispatched.
template <int XT, int BITS, int MT, int KW, int NW = kWaves, int WSEG = kWSeg>
struct SkinnyCfg {
  static constexpr int RW = NW / KW;
  static constexpr int XB = XT == XLA_AMD_DT_F32 ? 4 : 2;
  static constexpr int KS = BITS == 8 ? WSEG : 2 * WSEG;    // columns per step
  static constexpr int SUB = KS / 128;                       // 128-column sub-steps per step
  static constexpr int XROW = KS * XB;                       // bytes of one x row per step
  static constexpr int XROWS = 16 * MT;
  static constexpr int NLD = 16 * WSEG / 1024;               // 1 KB weight loads per wave per step
  static constexpr int BLK = BITS == 8 ? 2048 : 1024;        // bytes of one (16 channels x 128 columns) weight block
  static constexpr int X_TILE = XROWS * XROW;                // the x columns of one step, all rows
  // Steps of weight loads in flight per wave (register ring).  One step is
  // 8 KB per wave, 7 MB over the chip: enough to cover the memory latency; with
  // two or more the measured time goes *up* (the extra requests only queue).
  static constexpr int P = 1;
  // x is resident in LDS a chunk of steps at a time.  A chunk holds whole trips around the
  // ring for every wave (a multiple of P * KW steps).  With two chunk slots the next chunk is
  // copied while the current one is used (CS2 steps per chunk); with one slot the workgroup
  // stops while a chunk is replaced (CS1 steps per chunk).
  static constexpr int CS1 = kLdsLimit / X_TILE / (P * KW) * (P * KW);
  // (at most 4 steps per chunk with two slots: the first chunk is all that step 0 waits for)
  static constexpr int CS2 = (kLdsLimit / (2 * X_TILE) < 4 ? kLdsLimit / (2 * X_TILE) : 4) / (P * KW) * (P * KW);
  static constexpr bool kFits = CS1 >= P * KW;
  static constexpr int kRedBytes = NW * 16 * MT * 256;       // cross-wave reduction scratch (reuses the x tiles)
  static constexpr int lds_bytes(int steps, int slots) {
    const int cs = slots == 2 ? CS2 : CS1;
    const int tiles = steps <= cs ? steps : slots * cs;
    const int x = tiles * X_TILE;
    return x > kRedBytes ? x : kRedBytes;
  }
  static_assert(WSEG == 512 || WSEG == 256, "weight segment");
};

// Extra waves per workgroup that do nothing but copy x (and the blockwise scales) into LDS (see the
// kernel).  Two waves then share a SIMD and each may use half of its registers, which every
// configuration fits (at most 190 registers).  With 0 the computing waves copy for themselves, one
// chunk slot, the workgroup stopping for every copy: two x tiles of blockwise int4 weights at
// 14336 x 4096 take 28.2 us that way and 19.5 us with the copying waves.
template <int MT, int RED> constexpr int skinny_copier_waves() { return 4; }
// Chunk slots of x in LDS: two (the copying waves fill one while the other is used) when there
// are copying waves and two chunks fit, else one.
template <typename Cfg, int MT, int RED, int KW> constexpr int skinny_slots() {
  return (skinny_copier_waves<MT, RED>() > 0 && Cfg::CS2 >= Cfg::P * KW) ? 2 : 1;
}

// Blockwise launches keep, next to every resident x tile, the scale and zero point of each of its
// 128-column sub-steps (those of the quantization block the sub-step lies in) for the workgroup's
// channels: "entries" of 16 * RW values, indexed like the x tiles.  The waves that copy a chunk of x
// copy its entries too; the computing waves then read 4 channels' values with one LDS read instead of
// fetching them from global memory between the weight loads.
template <typename Cfg, int XT, int MT, int RED, int KW> constexpr int skinny_scale_bytes() {
  if (RED == 1 /*kRedRaw*/) return 0;
  constexpr int slots = skinny_slots<Cfg, MT, RED, KW>();
  constexpr int cs = slots == 2 ? Cfg::CS2 : Cfg::CS1;
  constexpr int entry = 16 * Cfg::RW * (XT == XLA_AMD_DT_F32 ? 4 : 2);
  return 2 * slots * cs * Cfg::SUB * entry;  // scale and zero point
}

// UNI: scale, zero point, dot product, result and stored tensor all have x's dtype (the common
// case, and the only one for blockwise weights): the dtypes are compile-time constants then, and
// the code that runs once per wave (epilogue, scale conversion) has no dtype branches.
template <int XT, int BITS, int MT, int KW, int RED, bool HASZP, bool UNI, int NW = kWaves, int WSEG = kWSeg>
__global__ void __launch_bounds__((NW + skinny_copier_waves<MT, RED>()) * 64)
qmm_skinny_kernel(SkinnyArgs a) {
  using Cfg = SkinnyCfg<XT, BITS, MT, KW, NW, WSEG>;
  constexpr int NLD = Cfg::NLD;
  constexpr int RW = Cfg::RW, XB = Cfg::XB, KS = Cfg::KS, SUB = Cfg::SUB, XROW = Cfg::XROW;
  constexpr int X_TILE = Cfg::X_TILE, P = Cfg::P, BLK = Cfg::BLK;
  constexpr bool kMfma = XT != XLA_AMD_DT_F32;
  constexpr bool NEEDXS = HASZP || (BITS == 4 && kMfma);  // x sums: zero point, int4 affine map
  constexpr int XQ = kMfma ? 4 : 8;                       // 16-byte x chunks per lane per sub-step
  extern __shared__ __attribute__((aligned(16))) char smem[];

  const int lane = threadIdx.x & 63;
  // wave-uniform values live in scalar registers: branches on them are scalar branches
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int rw = wave % RW, kw = wave / RW;
  const int r = lane & 15, g = lane >> 4;
#ifdef QMM_SKINNY_TIMELINE
  if (lane < kTlSlots) QMM_TL_AREA[wave * kTlSlots + lane] = 0;
#endif
  QMM_TL(0);  // entry
  QMM_TL_CLK(26);
  // this workgroup's K slice: columns k_begin .. k_begin + K of rows that hold ldk columns
  const int ldk = a.K;
  const int k_begin = (int)blockIdx.y * a.k_per_slice;
  const int K = min(a.k_per_slice, ldk - k_begin);
  const int N = a.N, M = a.M, C = a.C == a.K ? K : a.C;  // per-channel: the slice is the one block
  // This wave's channels: group grp_u of G channels (G = 16, or the narrower group of some per-channel int8
  // weights, see xla_amd_qmm_tile_group), ch_lo .. ch_hi - 1.  MFMA row 0 is channel n_wave, the four-aligned
  // channel at or below ch_lo, so that a lane's four results stay four-aligned for its stores; the rows below
  // ch_lo (two at most) and from ch_hi on are fed some other row's weights and their results are dropped.
  constexpr bool kGrouped = RED == kRedRaw && BITS == 8;
  const int G = kGrouped ? a.G : 16;
  const int grp_u = blockIdx.x * RW + rw;
  const int ch_lo = grp_u * G, ch_hi = min(ch_lo + G, N);
  const int n_wave = ch_lo & ~3;
  const int row_off = ch_lo - n_wave;
  const int x_dt = XT;
  const int scale_dt = UNI ? XT : a.scale_dt, zp_dt = UNI ? XT : a.zp_dt, out_dt = UNI ? XT : a.out_dt;
  const int dot_dt = UNI ? XT : a.dot_dt, store_dt = UNI ? XT : a.store_dt;
  static_assert(UNI || RED == kRedRaw, "blockwise launches have a single dtype");

  // ---- weights: global -> registers, already in MFMA operand order ------------------
  // The tiled weight holds, for every group of 16 channels and every sub-step of
  // 128 columns, one block of BLK bytes; the blocks of a group follow each other
  // along K, so a wave streams one contiguous region.  Lane l of a 1 KB load
  // takes bytes [16 l, 16 l + 16): its own operand fragment.
  const int n_blk = K / 128;                                    // blocks of this slice per channel group
  const int groups = (N + G - 1) / G;
  const int my_group = min(grp_u, groups - 1);  // tail groups re-read the last one
  const int blk_bytes = kGrouped ? G * 128 : BLK;                // bytes of one (G channels x 128 columns) weight block
  const int half_bytes = G * 64;                                 // (bits 8) second half of a block: columns 16 .. 31 of every quarter
  const int srow = min(max(r - row_off, 0), G - 1);              // row of the block that this lane's MFMA row reads
  const uint8_t* const w_base = a.w + ((size_t)my_group * (ldk / 128) + k_begin / 128) * blk_bytes + (g * G + srow) * 16;
  const char* const x_base = (const char*)a.x + (size_t)k_begin * XB;
  // x: copied global -> LDS without passing registers (global_load_lds_dwordx4:
  // lane l of an instruction lands at base + 16 l), 1 KB of one row per
  // instruction.  The XOR swizzle of the tile is applied on the source side: LDS
  // slot c' of a row receives global chunk c' ^ (row % 16).
  constexpr int kPiecesPerRow = XROW / 1024;
  static_assert(XROW % 1024 == 0, "a step of one x row is a whole number of 1 KB pieces");

  const int steps_total = (K + KS - 1) / KS;
  const int my_steps = steps_total > kw ? (steps_total - kw + KW - 1) / KW : 0;

  // ring slot p holds the fragments of one step: register 2t + h is half h of
  // sub-step t (bits 8), register t is sub-step t (bits 4)
  i32x4 wreg[P][NLD];
  constexpr int kLoadsPerSub = NLD / SUB;
  // The fragments of sub-step t of this wave's s-th step into ring slot p.  Steps
  // and sub-steps past the end (loaded only to keep the number of outstanding
  // loads the same on every path) re-read the last block of the group.
  auto load_sub = [&](auto pc, int s, auto tc) __attribute__((always_inline)) {
    constexpr int p = pc, t = tc;
    const int blk = min((s * KW + kw) * SUB + t, n_blk - 1);
    const uint8_t* const wp = w_base + (size_t)blk * blk_bytes;
    qmm_static_for<kLoadsPerSub>([&](auto hc) {
      constexpr int h = hc;
      wreg[p][kLoadsPerSub * t + h] = __builtin_nontemporal_load((const i32x4*)(wp + h * half_bytes));
    });
  };
  auto load_regs = [&](auto pc, int s) __attribute__((always_inline)) {
    qmm_static_for<SUB>([&](auto tc) { load_sub(pc, s, tc); });
  };
  // x is used a chunk of CS steps at a time; chunk c lives in LDS slot c % kSlots (CS tiles
  // per slot).  x_chunk_load copies chunk c: the copying waves (the extra ones, or all waves
  // when there are none) share the rows below M of every tile, a row per instruction (rows
  // from M on are never stored, so their x is not copied: a decode step of one row copies
  // 1/16 of a tile).
  typedef __attribute__((address_space(3))) void* lds_ptr_t;
  const int x_rows = min(M, Cfg::XROWS);
  constexpr int kCopiers = skinny_copier_waves<MT, RED>();
  constexpr int kSlots = skinny_slots<Cfg, MT, RED, KW>();
  constexpr int CS = kSlots == 2 ? Cfg::CS2 : Cfg::CS1;
  constexpr int kCopyWaves = kCopiers > 0 ? kCopiers : NW;
  const int copy_wave = kCopiers > 0 ? wave - NW : wave;
  const int n_chunks = (steps_total + CS - 1) / CS;
  // LDS: [blockwise scale entries][x tiles]
  constexpr int kSclBytes = skinny_scale_bytes<Cfg, XT, MT, RED, KW>();
  static_assert(kSclBytes <= 16 * 1024, "scale entries must fit above the x tiles");
  constexpr int SE = XT == XLA_AMD_DT_F32 ? 4 : 2;   // bytes of a blockwise scale (x's dtype)
  constexpr int kEntryBytes = 16 * RW * SE;          // one entry: the workgroup's channels
  constexpr int kSclTensor = kSclBytes / 2;          // the scales' entries, then the zero points'
  char* const xsm = smem + kSclBytes;
  const int n_sblk = ldk / a.C;       // quantization blocks of the whole K (blockwise)
  const int sblk0 = k_begin / a.C;    // first block of this slice
  const int c_shift = (C & (C - 1)) == 0 ? __builtin_ctz(C) : -1;  // block size a power of two: shift instead of divide
  auto x_chunk_load = [&](int c) __attribute__((always_inline)) {
    const int c0 = c * CS;
    const int nst = min(CS, steps_total - c0);
    if constexpr (RED != kRedRaw) {
      // entries of this chunk's tiles, 4 bytes per lane and instruction (256 bytes of consecutive entries):
      // entry e of the slot is sub-step e of the chunk, columns (c0 * SUB + e) * 128 ...
      constexpr int kPieces = kEntryBytes / 4;   // 4-byte pieces per entry (<= 64)
      constexpr int kEpi = 64 / kPieces;         // entries per instruction
      static_assert(kPieces <= 64 && (CS * SUB) % kEpi == 0, "whole instructions per chunk");
      constexpr int kInstr = CS * SUB / kEpi;
      const int n_wg0 = n_wave - 16 * rw;        // the workgroup's first channel
      char* const ent0 = smem + (kSlots == 2 ? (c & 1) * CS : 0) * SUB * kEntryBytes;
      for (int i = copy_wave; i < kInstr * (HASZP ? 2 : 1); i += kCopyWaves) {
        const bool is_zp = i >= kInstr;
        const int ii = is_zp ? i - kInstr : i;
        const int e = ii * kEpi + lane / kPieces, piece = lane % kPieces;
        const int k_at = (c0 * SUB + e) * 128;
        const int sblk = min(sblk0 + (c_shift >= 0 ? (k_at >> c_shift) : k_at / C), n_sblk - 1);
        int ch = n_wg0 + piece * (4 / SE);
        if (ch + 4 / SE > N) ch = N - 4 / SE;    // channels past N: any valid address (never used)
        const char* src = (const char*)(is_zp ? a.zp : a.scale) + ((size_t)sblk * N + ch) * SE;
        char* dst = ent0 + (is_zp ? kSclTensor : 0) + ii * (kEpi * kEntryBytes);
        __builtin_amdgcn_global_load_lds((const void*)src, (lds_ptr_t)dst, 4, 0, 0);
      }
    }
    char* const slot = xsm + (kSlots == 2 ? (c & 1) * (CS * X_TILE) : 0);
    for (int row = copy_wave; row < x_rows; row += kCopyWaves) {
      const char* xrow = x_base + (size_t)row * ((size_t)ldk * XB) + (size_t)c0 * XROW;  // row `row`, first column of the chunk
      char* lrow = slot + row * XROW;
      const int sw = row & 15;
      for (int t = 0; t < nst; ++t) {
        const char* xp = xrow + (size_t)t * XROW;
        char* dst = lrow + t * X_TILE;
        if ((c0 + t + 1) * KS <= K) {
          qmm_static_for<kPiecesPerRow>([&](auto pc) {
            constexpr int piece = pc;
            const uint32_t col = (uint32_t)(((piece * 64 + lane) ^ sw) * 16);
            __builtin_amdgcn_global_load_lds((const void*)(xp + col), (lds_ptr_t)(dst + piece * 1024), 16, 0, 0);
          });
        } else {
          // last, partial step: chunks past K re-read the last valid 16 bytes of the row
          const int x_left = K * XB - (c0 + t) * XROW;  // >= 256
          qmm_static_for<kPiecesPerRow>([&](auto pc) {
            constexpr int piece = pc;
            const int col = ((piece * 64 + lane) ^ sw) * 16;
            const int back = max(col + 16 - x_left, 0);  // 0 <= back <= col
            __builtin_amdgcn_global_load_lds((const void*)(xp + (col - back)), (lds_ptr_t)(dst + piece * 1024), 16, 0, 0);
          });
        }
      }
    }
  };
  // Copying all of x into every compute unit (the same 128 KB for each of them, out of a few L2
  // slices) takes longer than the first weights take to arrive from memory, so step 0 waits for
  // the first chunk only; the next chunk lands while the current one is used, and the workgroup
  // meets once per chunk.
  //
  // The computing waves cannot do the copying themselves: with global -> LDS copies in flight
  // when they enter the main loop, the compiler can no longer count their loads in flight and
  // turns every wait of the loop into a wait for all of them.  So kCopiers extra waves do all
  // the copying and nothing else: they wait for their copies, meet the workgroup at each of
  // its meeting points, and leave.  The computing waves only request weights.
  if constexpr (kCopiers > 0) {
    // (marked unlikely so that this block is laid out behind the computing waves' code: they
    // then run straight on from the kernel's entry to their first loads; a taken branch over
    // this block would cost them an instruction fetch from memory, the weights of the
    // previous launch having pushed the code out of L2)
    if (__builtin_expect(wave >= NW, 0)) {
      x_chunk_load(0);
      QMM_TL(1);  // first copies requested
      __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's copies have landed
      QMM_TL(2);  // ... landed
      for (int c = 0; c < n_chunks; ++c) {
        if (kSlots == 1 && c > 0) {
          qmm_bare_barrier();  // every wave has finished reading the old columns
          x_chunk_load(c);
          __builtin_amdgcn_s_waitcnt(0x0F70);
        }
        qmm_bare_barrier();    // chunk c is there (and, with two slots, chunk c - 1 has been read)
        if (c == 0) QMM_TL(3);
        if (kSlots == 2 && c + 1 < n_chunks) {
          x_chunk_load(c + 1);
          __builtin_amdgcn_s_waitcnt(0x0F70);
          QMM_TL(4 + min(c, 21));  // chunk c + 1 landed
        }
      }
      if constexpr (KW > 1) { qmm_bare_barrier(); qmm_bare_barrier(); }  // the two of the k-split reduction
      QMM_TL(30);
      QMM_TL_DUMP();
      return;
    }
  }

  // The first step's weights (the longest latency of the kernel: a cold HBM access) go out
  // before anything else is computed.
  qmm_static_for<P>([&](auto pc) { load_regs(pc, pc); });
  __builtin_amdgcn_sched_barrier(0);
  QMM_TL(1);  // first weights requested
  if constexpr (kCopiers == 0) {
    // Loads complete in order, so waiting for the copies also waits for those weights, which
    // step 0 needs anyway.
    x_chunk_load(0);
    __builtin_amdgcn_sched_barrier(0);
  }

  // ---- accumulators ----------------------------------------------------------------
  // (register arrays are only ever indexed by compile-time constants: every
  // loop over them is a qmm_static_for)
  // acc/accb: two interleaved accumulation chains per tile (dependent MFMAs
  // would otherwise wait for each other); their sum is the dot product.
  f32x4 acc[MT], accb[MT], xs[MT], sacc[MT], zacc[MT];
  qmm_static_for<MT>([&](auto mc) {
    constexpr int mt = mc;
    acc[mt] = f32x4{0, 0, 0, 0};
    accb[mt] = f32x4{0, 0, 0, 0};
    xs[mt] = f32x4{0, 0, 0, 0};
    sacc[mt] = f32x4{0, 0, 0, 0};
    zacc[mt] = f32x4{0, 0, 0, 0};
  });

  // Undo the int4 affine map (MFMA path only): dot = 16 * (acc - 1.5 * xsum).
  auto true_dot = [&](float accv, float xsv) __attribute__((always_inline)) -> float {
    if constexpr (BITS == 4 && kMfma) return 16.0f * (accv - 1.5f * xsv);
    return accv;
  };

  // End of quantization block sblk: p = round_x(dot); sacc += scale[s,n] * p;
  // zacc += round_x(xsum) * zp[s,n]; the block accumulators restart.
  // Per-channel: the only scales a lane ever needs are fetched now, so that
  // their latency is hidden behind the main loop instead of trailing it.
  uint32_t pre_sc[4] = {0u, 0u, 0u, 0u}, pre_zp[4] = {0u, 0u, 0u, 0u};  // raw bits: converted where they are used
  auto fetch_channel_scales = [&]() __attribute__((always_inline)) {
    if constexpr (RED == kRedRaw) {
      qmm_static_for<4>([&](auto vc) {
        constexpr int v = vc;
        const int n = min(n_wave + 4 * g + v, N - 1);
        pre_sc[v] = qmm_load_raw(a.scale, n, scale_dt);
        if constexpr (HASZP) pre_zp[v] = qmm_load_raw(a.zp, n, zp_dt);
      });
    }
  };
  // Blockwise: scale / zero point of this lane's 4 channels come from the entry of the sub-step
  // that ends the block (x tile `ep_tile`, sub-step t), one LDS read each.
  int ep_tile = 0;
  auto bw_read = [&](int tensor, auto tc, float (&val)[4]) __attribute__((always_inline)) {
    constexpr int t = tc;
    const char* ent = smem + tensor * kSclTensor + (ep_tile * SUB + t) * kEntryBytes + (16 * rw + 4 * g) * SE;
    if constexpr (SE == 4) {
      const f32x4 r4 = *(const f32x4*)ent;
      val[0] = r4[0]; val[1] = r4[1]; val[2] = r4[2]; val[3] = r4[3];
    } else {
      const i32x2 r2 = *(const i32x2*)ent;
      val[0] = qmm_from_raw((uint32_t)r2[0] & 0xffffu, XT); val[1] = qmm_from_raw((uint32_t)r2[0] >> 16, XT);
      val[2] = qmm_from_raw((uint32_t)r2[1] & 0xffffu, XT); val[3] = qmm_from_raw((uint32_t)r2[1] >> 16, XT);
    }
  };
  auto block_epilogue = [&](int sblk, auto tc) __attribute__((always_inline)) {
    constexpr int t = tc;
    float sc4[4], zp4[4] = {0.f, 0.f, 0.f, 0.f};
    if constexpr (RED != kRedRaw) {
      bw_read(0, tc, sc4);
      if constexpr (HASZP) bw_read(1, tc, zp4);
    }
    // (every register of xs holds the row's sum: the lane's x row is the same for its 4 channels)
    float xs_rounded[MT];
    qmm_static_for<MT>([&](auto mc) { xs_rounded[(int)mc] = NEEDXS ? qmm_round_dt(xs[(int)mc][0], x_dt) : 0.f; });
    qmm_static_for<4>([&](auto vc) {
      constexpr int v = vc;
      float sc, zv = 0.f;
      if constexpr (RED == kRedRaw) {
        sc = qmm_from_raw(pre_sc[v], scale_dt);
        if constexpr (HASZP) zv = qmm_from_raw(pre_zp[v], zp_dt);
      } else {
        sc = sc4[v];
        zv = zp4[v];
      }
      qmm_static_for<MT>([&](auto mc) {
        constexpr int mt = mc;
        const float xsv = NEEDXS ? xs[mt][0] : 0.f;
        float p;
        if constexpr (RED != kRedRaw && BITS == 4 && kMfma) {
          // the int4 map's factor 16 is applied once, to the sum over the blocks (a power of two commutes with the rounding)
          p = qmm_round_dt(fmaf(-1.5f, xsv, acc[mt][v] + accb[mt][v]), dot_dt);
        } else {
          p = qmm_round_dt(true_dot(acc[mt][v] + accb[mt][v], xsv), dot_dt);
        }
        sacc[mt][v] = fmaf(sc, p, sacc[mt][v]);
        if constexpr (HASZP) zacc[mt][v] = fmaf(xs_rounded[mt], zv, zacc[mt][v]);
      });
    });
    qmm_static_for<MT>([&](auto mc) {
      constexpr int mt = mc;
      acc[mt] = f32x4{0, 0, 0, 0};
      accb[mt] = f32x4{0, 0, 0, 0};
      xs[mt] = f32x4{0, 0, 0, 0};
    });
  };

  // ---- one step out of LDS -----------------------------------------------------------
  // Sub-steps (128 columns) left in the current quantization block; uniform.
  const int sub_per_block = C / 128;
  int block_left = sub_per_block;
  // One step: the weights of ring slot p against the x columns in LDS tile
  // `tile`.  As soon as a sub-step's fragments have been used, the same
  // registers are re-loaded with that sub-step of step s + P: the loads trickle
  // out between the multiplies instead of as one burst.  Sub-steps at or beyond K
  // are skipped (a uniform branch around arithmetic only: the loads stay in
  // straight-line code, so the compiler's wait counts for the ring stay exact).
  // refill = 0 is the wave's last step: nothing is fetched for later steps, so
  // that the epilogue does not have to wait for loads nobody reads before it may
  // reuse their registers.
  auto compute = [&](auto pc, int tile, int s, auto refillc) __attribute__((always_inline)) {
    constexpr int p = pc;
    constexpr bool kRefill = refillc != 0;
    const char* xb = xsm + tile * X_TILE;
    ep_tile = tile;
    const int k_step = (s * KW + kw) * KS;
    if constexpr (RED == kRedScaled) block_left = sub_per_block;  // steps start on block boundaries
    // x fragments of sub-step t: per tile of 16 x rows, this lane's XQ 16-byte chunks
    auto read_frags = [&](auto tc, i32x4 (&xq)[MT][XQ]) __attribute__((always_inline)) {
      constexpr int t = tc;
      qmm_static_for<MT>([&](auto mc) {
        constexpr int mt = mc;
        qmm_static_for<XQ>([&](auto qc) {
          constexpr int q = qc;
          xq[mt][q] = *(const i32x4*)(xb + (16 * mt + r) * XROW + (((XQ * 4 * t + XQ * g + q) ^ r) * 16));
        });
      });
    };
    auto math = [&](auto tc, const i32x4& wq0, const i32x4& wq1, const i32x4 (&xq)[MT][XQ]) __attribute__((always_inline)) {
      constexpr int t = tc;
      const int k_sub = k_step + t * 128;
      if constexpr (kMfma) {
        qmm_static_for<4>([&](auto jc) {
          constexpr int j = jc;
          i32x4 af;
          if constexpr (BITS == 8) {
            const i32x4 src = (j >> 1) ? wq1 : wq0;
            af = cvt_w8<XT>((uint32_t)src[(j & 1) * 2], (uint32_t)src[(j & 1) * 2 + 1]);
          } else {
            af = cvt_w4<XT>((uint32_t)wq0[j]);
          }
          qmm_static_for<MT>([&](auto mc) {
            constexpr int mt = mc;
            if constexpr (j & 1) accb[mt] = mfma16<XT>(af, xq[mt][j], accb[mt]);
            else acc[mt] = mfma16<XT>(af, xq[mt][j], acc[mt]);
            if constexpr (NEEDXS) xs[mt] = mfma16<XT>(ones_frag<XT>(), xq[mt][j], xs[mt]);
          });
        });
      } else {
        // f32 x: 16x16x4 f32 MFMA, one column per lane per instruction.
        qmm_static_for<32>([&](auto kc) {
          constexpr int kk = kc;  // 0..31 within the lane's columns
          float wf;
          if constexpr (BITS == 8) {
            const i32x4 src = (kk >> 4) ? wq1 : wq0;
            const uint32_t dw = (uint32_t)src[(kk >> 2) & 3];
            wf = (float)(int8_t)(dw >> (8 * (kk & 3)));
          } else {
            // column kk = 8*word + P[nibble]: nibble = (c&1)*4 + (c>>1), c = kk % 8
            const uint32_t dw = (uint32_t)wq0[kk >> 3];
            constexpr int c = kk & 7, nib = (c & 1) * 4 + (c >> 1);
            wf = (float)(int)((dw >> (4 * nib)) & 15u) - 8.0f;
          }
          qmm_static_for<MT>([&](auto mc) {
            constexpr int mt = mc;
            constexpr int xq_i = kk >> 2, xe_i = kk & 3;
            const f32x4 xv4 = __builtin_bit_cast(f32x4, xq[mt][xq_i]);
            const float xv = xv4[xe_i];
            if constexpr (kk & 1) accb[mt] = __builtin_amdgcn_mfma_f32_16x16x4f32(wf, xv, accb[mt], 0, 0, 0);
            else acc[mt] = __builtin_amdgcn_mfma_f32_16x16x4f32(wf, xv, acc[mt], 0, 0, 0);
            if constexpr (NEEDXS) xs[mt] = __builtin_amdgcn_mfma_f32_16x16x4f32(1.0f, xv, xs[mt], 0, 0, 0);
          });
        });
      }
      if constexpr (RED != kRedRaw) {
        if (--block_left == 0) {
          block_epilogue(k_sub / C, tc);
          block_left = sub_per_block;
        }
      }
    };
    // (two x tiles with per-block scale accumulators leave no registers for the second fragment set)
    constexpr bool kPipe = kMfma && !(MT == 2 && RED == kRedScaled);
    constexpr int kW1 = kLoadsPerSub - 1;  // second half of a sub-step's fragment (bits 8), else the same register
    if constexpr (kPipe) {
      // The LDS reads of sub-step t+1 are issued before the math of sub-step t
      // (a wave has few neighbours on its SIMD to hide LDS latency).
      i32x4 xq[2][MT][XQ];
      read_frags(qmm_const<0>{}, xq[0]);
      qmm_static_for<SUB>([&](auto tc) {
        constexpr int t = tc;
        constexpr int cur = t & 1, nxt = cur ^ 1;
        if constexpr (t + 1 < SUB) read_frags(qmm_const<t + 1>{}, xq[nxt]);
        __builtin_amdgcn_sched_barrier(0);
        if (k_step + t * 128 < K) math(tc, wreg[p][kLoadsPerSub * t], wreg[p][kLoadsPerSub * t + kW1], xq[cur]);
        if constexpr (kRefill) {
          load_sub(pc, s + P, tc);
        }
        __builtin_amdgcn_sched_barrier(0);
      });
    } else {
      qmm_static_for<SUB>([&](auto tc) {
        constexpr int t = tc;
        if (k_step + t * 128 < K) {
          i32x4 xq[MT][XQ];
          read_frags(tc, xq);
          math(tc, wreg[p][kLoadsPerSub * t], wreg[p][kLoadsPerSub * t + kW1], xq);
        }
        if constexpr (kRefill) {
          load_sub(pc, s + P, tc);
        }
      });
    }
  };

  // ---- main loop ---------------------------------------------------------------------
  // The x columns of a chunk of CS steps are resident in LDS; the workgroup meets once per
  // chunk, and between those points every wave runs its steps at its own pace (wait for its
  // weights, multiply), so that the waves of a compute unit drift apart and their memory
  // waits, LDS traffic and arithmetic overlap.
  // Every wave runs the chunk loop the same number of times, whether it has steps in a chunk
  // or not: the barriers always match.  A chunk holds whole trips around the ring for every
  // wave, so each chunk starts on ring slot 0.
  //
  // Weight loads are issued unconditionally, also for steps past the end (those
  // re-read the last block): a load that is issued on some paths only would force
  // the compiler to wait for *all* outstanding loads wherever it needs one of
  // them.
  // First chunk: weights of step 0 are under way (issued at the top of the kernel) and so
  // are the x copies (with the blockwise scales of their sub-steps).
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the first weights (and this wave's copies, if it copies) have landed
  QMM_TL(2);  // first weights landed
  qmm_bare_barrier();
  QMM_TL(3);  // first x chunk there
  fetch_channel_scales();  // (per-channel) needed at the very end: their latency hides behind the main loop
  int s0 = 0;  // this wave's next step
  for (int c = 0; c < n_chunks; ++c) {
    const int c0 = c * CS;
    const int nst = min(CS, steps_total - c0);
    const int tile0 = kSlots == 2 ? (c & 1) * CS : 0;
    if (c > 0) {
      if constexpr (kSlots == 1) {
        qmm_bare_barrier();                    // every wave has finished reading the old columns
        if constexpr (kCopiers == 0) {
          x_chunk_load(c);
          __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's copies have landed
        }
      }
      qmm_bare_barrier();                      // chunk c is there
    }
    int s_end = min(my_steps, (c0 + CS) / KW);
    // Without k-splits the wave's last step lies in the last chunk: it is run
    // after the loop, in a form that fetches nothing more.
    if constexpr (KW == 1 && P == 1) {
      if (c + 1 == n_chunks) --s_end;
    }
    for (; s0 < s_end; s0 += P) {
      qmm_static_for<P>([&](auto hc) {
        const int s = s0 + hc;
        const int gs = s * KW + kw;
        // (a step past the end, which only occurs to complete a trip around the
        // ring, has every sub-step beyond K: it issues its loads and computes nothing)
        compute(hc, tile0 + min(gs - c0, nst - 1), s, qmm_const<1>{});
        QMM_TL(4 + min(s, 21));  // this wave's step s done
      });
    }
    if constexpr (KW == 1 && P == 1) {
      if (c + 1 == n_chunks) compute(qmm_const<0>{}, tile0 + s0 - c0, s0, qmm_const<0>{});
    }
  }
  QMM_TL(28);  // all steps done

  // ---- reduction over k-splits, final rounding, store ------------------------------------
  const int zpo_dt = qmm_promote(x_dt, zp_dt);
  if constexpr (KW > 1) {
    __syncthreads();  // every wave is done with the x tiles: reuse LDS
    float* red = (float*)smem;  // [KW][RW][slot][64]
    constexpr int kSlots = RED == kRedRaw ? 4 * MT + (NEEDXS ? MT : 0) : (HASZP ? 8 * MT : 4 * MT);
    float* mine = red + ((kw * RW + rw) * kSlots) * 64 + lane;
    qmm_static_for<MT>([&](auto mc) {
      constexpr int mt = mc;
      qmm_static_for<4>([&](auto vc) {
        constexpr int v = vc;
        if constexpr (RED == kRedRaw) {
          mine[(4 * mt + v) * 64] = acc[mt][v] + accb[mt][v];
        } else {
          mine[(4 * mt + v) * 64] = sacc[mt][v];
          if constexpr (HASZP) mine[(4 * MT + 4 * mt + v) * 64] = zacc[mt][v];
        }
      });
      if constexpr (RED == kRedRaw && NEEDXS) mine[(4 * MT + mt) * 64] = xs[mt][0];
    });
    __syncthreads();
    if (kw != 0) {
      QMM_TL(30);
      QMM_TL_DUMP();
      return;
    }
    QMM_TL(29);  // partial sums of the k-splits are in LDS
    qmm_static_for<MT>([&](auto mc) {
      constexpr int mt = mc;
      qmm_static_for<4>([&](auto vc) {
        constexpr int v = vc;
        float t = 0.f, z = 0.f;
#pragma unroll
        for (int k2 = 0; k2 < KW; ++k2) {
          const float* other = red + ((k2 * RW + rw) * kSlots) * 64 + lane;
          t += other[(4 * mt + v) * 64];
          if constexpr (RED == kRedScaled && HASZP) z += other[(4 * MT + 4 * mt + v) * 64];
        }
        if constexpr (RED == kRedRaw) { acc[mt][v] = t; accb[mt][v] = 0.f; }
        else { sacc[mt][v] = t; zacc[mt][v] = z; }
      });
      if constexpr (RED == kRedRaw && NEEDXS) {
        float t = 0.f;
#pragma unroll
        for (int k2 = 0; k2 < KW; ++k2) t += (red + ((k2 * RW + rw) * kSlots) * 64 + lane)[(4 * MT + mt) * 64];
        xs[mt] = f32x4{t, t, t, t};
      }
    });
  }
  if constexpr (RED == kRedRaw) {
    if (a.slices > 1) {
      // one K slice of several: the raw sums go to the workspace, a second kernel adds the slices and finishes them
      const int slice = blockIdx.y;
      qmm_static_for<MT>([&](auto mc) {
        constexpr int mt = mc;
        const int m = 16 * mt + r;
        const int n = n_wave + 4 * g;
        if (m < M && n + 3 >= ch_lo && n < ch_hi) {
          float* p = a.part + ((size_t)slice * M + m) * N + n;
          // (the slice's dot product: with int4 weights the affine map is undone with the slice's own row sum)
          const float xsv = NEEDXS ? xs[mt][0] : 0.f;
          const f32x4 t = {true_dot(acc[mt][0] + accb[mt][0], xsv), true_dot(acc[mt][1] + accb[mt][1], xsv),
                           true_dot(acc[mt][2] + accb[mt][2], xsv), true_dot(acc[mt][3] + accb[mt][3], xsv)};
          if ((N & 3) == 0 && n >= ch_lo && n + 3 < ch_hi) *(f32x4*)p = t;
          else for (int v = 0; v < 4; ++v) if (n + v >= ch_lo && n + v < ch_hi) p[v] = t[v];
          if constexpr (NEEDXS) {
            if (n_wave == 0 && g == 0) a.part_xs[(size_t)slice * M + m] = xs[mt][0];
          }
        }
      });
      QMM_TL(30);
      QMM_TL_DUMP();
      return;
    }
    block_epilogue(0, qmm_const<0>{});  // the single block ends here
  }

  qmm_static_for<MT>([&](auto mc) {
    constexpr int mt = mc;
    const int m = 16 * mt + r;
    const int n = n_wave + 4 * g;
    if (m < M && n + 3 >= ch_lo && n < ch_hi) {
      constexpr float kBlockFactor = (RED != kRedRaw && BITS == 4 && kMfma) ? 16.0f : 1.0f;  // see block_epilogue
      if constexpr (RED != kRedRaw) {
        if (a.slices > 1) {
          // one K slice of several (whole quantization blocks): the sums over this slice's blocks go to the workspace,
          // a second kernel adds the slices and does the final roundings
          const size_t at = ((size_t)blockIdx.y * M + m) * N + n;  // N % 4 == 0 for blockwise weights
          *(f32x4*)(a.part + at) = f32x4{kBlockFactor * sacc[mt][0], kBlockFactor * sacc[mt][1], kBlockFactor * sacc[mt][2],
                                         kBlockFactor * sacc[mt][3]};
          if constexpr (HASZP) *(f32x4*)(a.part_z + at) = zacc[mt];
          return;  // (this row tile is done)
        }
      }
      float o0 = qmm_round_dt(kBlockFactor * sacc[mt][0], out_dt), o1 = qmm_round_dt(kBlockFactor * sacc[mt][1], out_dt);
      float o2 = qmm_round_dt(kBlockFactor * sacc[mt][2], out_dt), o3 = qmm_round_dt(kBlockFactor * sacc[mt][3], out_dt);
      if constexpr (HASZP) {
        o0 = qmm_round_dt(o0 - qmm_round_dt(zacc[mt][0], zpo_dt), out_dt);
        o1 = qmm_round_dt(o1 - qmm_round_dt(zacc[mt][1], zpo_dt), out_dt);
        o2 = qmm_round_dt(o2 - qmm_round_dt(zacc[mt][2], zpo_dt), out_dt);
        o3 = qmm_round_dt(o3 - qmm_round_dt(zacc[mt][3], zpo_dt), out_dt);
      }
      // (a store dtype narrower than out_dt is the caller's final cast: one more rounding, done by the conversion)
      const int st = store_dt;
      const size_t idx = (size_t)m * N + n;
      if ((N & 3) == 0 && n >= ch_lo && n + 3 < ch_hi) {  // 4 consecutive channels of this wave: one aligned 8- or 16-byte store
        if (st == XLA_AMD_DT_F32) {
          *(f32x4*)((float*)a.out + idx) = f32x4{o0, o1, o2, o3};
        } else {
          const bool bf = st == XLA_AMD_DT_BF16;
          const uint32_t h0 = bf ? qmm_f32_to_bf16(o0) : qmm_f32_to_f16(o0);
          const uint32_t h1 = bf ? qmm_f32_to_bf16(o1) : qmm_f32_to_f16(o1);
          const uint32_t h2 = bf ? qmm_f32_to_bf16(o2) : qmm_f32_to_f16(o2);
          const uint32_t h3 = bf ? qmm_f32_to_bf16(o3) : qmm_f32_to_f16(o3);
          *(i32x2*)((uint16_t*)a.out + idx) = i32x2{(int)(h0 | (h1 << 16)), (int)(h2 | (h3 << 16))};
        }
      } else {
        if (n >= ch_lo) qmm_store(a.out, idx, o0, st);
        if (n + 1 >= ch_lo && n + 1 < ch_hi) qmm_store(a.out, idx + 1, o1, st);
        if (n + 2 >= ch_lo && n + 2 < ch_hi) qmm_store(a.out, idx + 2, o2, st);
        if (n + 3 < ch_hi) qmm_store(a.out, idx + 3, o3, st);
      }
    }
  });
  QMM_TL(30);  // results stored (requested)
  QMM_TL_DUMP();
}

template <int XT, int BITS, int MT, int KW, int RED, bool HASZP, bool UNI, int NW = kWaves, int WSEG = kWSeg>
int launch_kernel(const SkinnyArgs& a, hipStream_t stream) {
  using Cfg = SkinnyCfg<XT, BITS, MT, KW, NW, WSEG>;
  if constexpr (!Cfg::kFits) {
    return qmm_fail(XLA_AMD_QMM_EUNSUPPORTED, "weight_only_skinny: tile does not fit in LDS");
  } else {
    auto kern = qmm_skinny_kernel<XT, BITS, MT, KW, RED, HASZP, UNI, NW, WSEG>;
    static std::atomic<uint64_t> lds_set{0};
    constexpr int kSlots = skinny_slots<Cfg, MT, RED, KW>();
#ifdef QMM_SKINNY_TIMELINE
    constexpr int kMaxLds = 160 * 1024;  // (room for the time notes wherever the kernel leaves it)
#else
    constexpr int kMaxLds = Cfg::lds_bytes(1 << 20, kSlots) + skinny_scale_bytes<Cfg, XT, MT, RED, KW>();
#endif
    const int rc = qmm_set_max_lds((const void*)kern, kMaxLds, lds_set, "weight_only_skinny hipFuncSetAttribute");
    if (rc != XLA_AMD_QMM_OK) return rc;
    const int g_ch = (RED == kRedRaw && BITS == 8) ? a.G : 16;
    const int groups = (a.N + g_ch - 1) / g_ch;
    const unsigned blocks = (unsigned)((groups + Cfg::RW - 1) / Cfg::RW);
    const int steps = (a.k_per_slice + Cfg::KS - 1) / Cfg::KS;
    constexpr int kScl = skinny_scale_bytes<Cfg, XT, MT, RED, KW>();
    int lds = Cfg::lds_bytes(steps, kSlots) + kScl;
#ifdef QMM_SKINNY_TIMELINE
    SkinnyArgs at = a;
    if (lds + kTlLdsBytes > 160 * 1024 || (uint64_t)blocks * a.slices > kTlBlocks)
      return qmm_fail(XLA_AMD_QMM_EUNSUPPORTED, "weight_only_skinny (timeline build): no room for the time notes of this launch");
    at.tl_off = lds;
    lds += kTlLdsBytes;
    hipLaunchKernelGGL(kern, dim3(blocks, (unsigned)a.slices), dim3((NW + skinny_copier_waves<MT, RED>()) * 64), lds, stream, at);
#else
    hipLaunchKernelGGL(kern, dim3(blocks, (unsigned)a.slices), dim3((NW + skinny_copier_waves<MT, RED>()) * 64), lds, stream, a);
#endif
    return QMM_CHECK_LAUNCH("weight_only_skinny launch");
  }
}

template <int XT, int BITS, int MT, int KW, int RED>
int launch_zp(const SkinnyArgs& a, bool haszp, hipStream_t stream) {
  const bool uni = a.scale_dt == XT && a.zp_dt == XT && a.out_dt == XT && a.dot_dt == XT && a.store_dt == XT;
  if (uni) {
    return haszp ? launch_kernel<XT, BITS, MT, KW, RED, true, true>(a, stream)
                 : launch_kernel<XT, BITS, MT, KW, RED, false, true>(a, stream);
  }
  if constexpr (RED == kRedRaw) {
    return haszp ? launch_kernel<XT, BITS, MT, KW, RED, true, false>(a, stream)
                 : launch_kernel<XT, BITS, MT, KW, RED, false, false>(a, stream);
  } else {
    return qmm_fail(XLA_AMD_QMM_EUNSUPPORTED, "weight_only_skinny: blockwise weights need scale, zero point and result of x's dtype");
  }
}

// K split over the waves of a workgroup (KW = 1, 2, 4: 64, 32, 16 channels per workgroup): the
// largest that still gives one workgroup per compute unit at most (256 of them), where the
// reduction is defined (per-channel, or whole quantization blocks per step) and the wider x tile
// fits in LDS.  More workgroups than compute units is a second, partly empty round and more
// copies of x: measured at M = 32, K = 4096 with cold weights, N = 6144 takes 16.9 us in 384
// workgroups of 16 channels and 11.5 us in 192 of 32; N = 11008 takes 21.1 us in 344 workgroups of
// 32 channels and 13.4 us in 172 of 64.
template <int XT, int BITS, int MT>
int launch_split(const SkinnyArgs& a, bool haszp, hipStream_t stream) {
  constexpr int KS = BITS == 8 ? kWSeg : 2 * kWSeg;
  constexpr int64_t kComputeUnits = 256;
  const bool perch = a.C == a.K;
  const bool can_split = perch || (KS % a.C == 0);
  const int steps = (a.k_per_slice + KS - 1) / KS;  // of one workgroup
  const int g_ch = (perch && BITS == 8) ? a.G : 16;                    // channels per group of the tiled weight
  const int64_t groups = ((int64_t)a.N + g_ch - 1) / g_ch;
  auto workgroups = [&](int kw_) { return (groups + 4 / kw_ - 1) / (4 / kw_) * a.slices; };  // K slices multiply them too
  int kw = 1;
  if (can_split) {
    if (workgroups(2) <= kComputeUnits && steps >= 2 && SkinnyCfg<XT, BITS, MT, 2>::kFits) kw = 2;
    if (workgroups(4) <= kComputeUnits && steps >= 4 && SkinnyCfg<XT, BITS, MT, 4>::kFits) kw = 4;
  }
  // More than one round of 64-channel workgroups (N > 16384: the fused gate / up projection, a
  // vocabulary projection): eight computing waves, 128 channels per workgroup.  Half as many
  // copies of x out of L2 and no part-full second round; three waves per SIMD still fit the
  // registers of the int8 per-channel kernels with one dtype throughout.  Measured with cold
  // weights: 28672 x 4096 at M = 32 29.0 -> 25.9 us, at M = 16 24.8 -> 23.5; 18432 x 8192 at
  // M = 1 37.4 -> 28.6 us (288 workgroups had been a round and an eighth).
  // More channel groups than wave slots, up to 16 rows of x that fit in LDS whole: persistent waves that each
  // stream a run of groups without a break (qmm_skinny_resident.hip).  Measured with cold weights at M = 16 / M = 1:
  // see the numbers at that kernel's dispatch in the design notes.
  if constexpr (BITS == 8 && XT != XLA_AMD_DT_F32 && MT == 1) {
    if (const int wgs = qmm_skinny_resident_workgroups(a, XT, BITS)) {
      if constexpr (XT == XLA_AMD_DT_BF16) return qmm_skinny_resident_launch_bf16(a, haszp, wgs, stream);
      else return qmm_skinny_resident_launch_f16(a, haszp, wgs, stream);
    }
  }
  if constexpr (BITS == 8 && XT != XLA_AMD_DT_F32) {
    const bool uni = a.scale_dt == XT && a.zp_dt == XT && a.out_dt == XT && a.dot_dt == XT && a.store_dt == XT;
    if (kw == 1 && perch && uni && workgroups(1) > kComputeUnits)
      return haszp ? launch_kernel<XT, BITS, MT, 1, kRedRaw, true, true, 8, kWSeg>(a, stream)
                   : launch_kernel<XT, BITS, MT, 1, kRedRaw, false, true, 8, kWSeg>(a, stream);
  }
  // Blockwise int4 against few channels (one channel group per compute unit at most) with all of x in one chunk:
  // a wave's step is issue-bound arithmetic (every block has its own rounding sequence), so eight computing waves
  // with half-length steps (256 weight bytes per row) split K eight ways.
  if constexpr (BITS == 4 && XT != XLA_AMD_DT_F32 && MT == 1) {
    using Cfg8 = SkinnyCfg<XT, BITS, MT, 8, 8, 256>;
    const int steps8 = (a.k_per_slice + Cfg8::KS - 1) / Cfg8::KS;
    if (!perch && Cfg8::KS % a.C == 0 && a.k_per_slice % Cfg8::KS == 0 && groups * a.slices <= kComputeUnits &&
        steps8 == 8 && Cfg8::kFits)
      return haszp ? launch_kernel<XT, BITS, MT, 8, kRedScaled, true, true, 8, 256>(a, stream)
                   : launch_kernel<XT, BITS, MT, 8, kRedScaled, false, true, 8, 256>(a, stream);
  }
  if (kw == 1) {
    return perch ? launch_zp<XT, BITS, MT, 1, kRedRaw>(a, haszp, stream)
                 : launch_zp<XT, BITS, MT, 1, kRedNone>(a, haszp, stream);
  }
  if (kw == 2) return perch ? launch_zp<XT, BITS, MT, 2, kRedRaw>(a, haszp, stream)
                            : launch_zp<XT, BITS, MT, 2, kRedScaled>(a, haszp, stream);
  return perch ? launch_zp<XT, BITS, MT, 4, kRedRaw>(a, haszp, stream)
               : launch_zp<XT, BITS, MT, 4, kRedScaled>(a, haszp, stream);
}

template <int XT, int BITS>
int launch_mt(const SkinnyArgs& a, bool haszp, hipStream_t stream) {
  if constexpr (XT != XLA_AMD_DT_F32) {
    if (a.M > 16) return launch_split<XT, BITS, 2>(a, haszp, stream);
  }
  return launch_split<XT, BITS, 1>(a, haszp, stream);
}

template <int XT>
int launch_bits(const SkinnyArgs& a, int bits, bool haszp, hipStream_t stream) {
  return bits == 8 ? launch_mt<XT, 8>(a, haszp, stream) : launch_mt<XT, 4>(a, haszp, stream);
}

}  // namespace

#if QMM_SKINNY_XT == XLA_AMD_DT_F32
int qmm_skinny_launch_f32(const SkinnyArgs& a, int bits, bool haszp, hipStream_t stream) {
  return launch_bits<XLA_AMD_DT_F32>(a, bits, haszp, stream);
}
#elif QMM_SKINNY_XT == XLA_AMD_DT_F16
int qmm_skinny_launch_f16(const SkinnyArgs& a, int bits, bool haszp, hipStream_t stream) {
  return launch_bits<XLA_AMD_DT_F16>(a, bits, haszp, stream);
}
#else
int qmm_skinny_launch_bf16(const SkinnyArgs& a, int bits, bool haszp, hipStream_t stream) {
  return launch_bits<XLA_AMD_DT_BF16>(a, bits, haszp, stream);
}

#ifdef QMM_SKINNY_TIMELINE
// The notes of the last recorded launch: [workgroup][wave (12)][note (32)] of 100 MHz ticks, 0 = not reached.
extern "C" int xla_amd_qmm_timeline_read(uint64_t* host, size_t count) {
  if (!host || count > sizeof(qmm_tl_buf) / sizeof(uint64_t)) return qmm_fail(XLA_AMD_QMM_EINVAL, "timeline_read: bad arguments");
  return qmm_check_hip(hipMemcpyFromSymbol(host, HIP_SYMBOL(qmm_tl_buf), count * sizeof(uint64_t)), "timeline_read");
}
#endif

extern "C" int xla_amd_qmm_weight_only_skinny(const void* x, const void* w_tiled, const void* scale,
                                              const void* zp, void* out, int64_t M, int64_t N,
                                              int64_t K, int64_t C, int bits, int x_dt, int scale_dt,
                                              int zp_dt, int dot_dt, int out_dt, int store_dt,
                                              void* stream) {
  if (!x || !w_tiled || !scale || !out) return qmm_fail(XLA_AMD_QMM_EINVAL, "weight_only_skinny: null pointer");
  if (M < 0 || N <= 0 || K <= 0 || C <= 0 || K % C != 0)
    return qmm_fail(XLA_AMD_QMM_EINVAL, "weight_only_skinny: bad sizes M=%lld N=%lld K=%lld C=%lld",
                    (long long)M, (long long)N, (long long)K, (long long)C);
  if (bits != 4 && bits != 8) return qmm_fail(XLA_AMD_QMM_EINVAL, "weight_only_skinny: bits must be 4 or 8");
  if (!qmm_valid_dt(x_dt) || !qmm_valid_dt(scale_dt) || !qmm_valid_dt(out_dt) || !qmm_valid_dt(dot_dt) ||
      !qmm_valid_dt(store_dt) || (zp && !qmm_valid_dt(zp_dt)))
    return qmm_fail(XLA_AMD_QMM_EINVAL, "weight_only_skinny: bad dtype enum");
  if (out_dt != qmm_promote(x_dt, scale_dt))
    return qmm_fail(XLA_AMD_QMM_EINVAL, "weight_only_skinny: out dtype must be promote(x, scale)");
  if (dot_dt != x_dt && (dot_dt != XLA_AMD_DT_F32 || C != K))
    return qmm_fail(XLA_AMD_QMM_EINVAL, "weight_only_skinny: dot dtype must be x's, or f32 for per-channel weights");
  if (K % 128 != 0 || C % 128 != 0)
    return qmm_fail(XLA_AMD_QMM_EUNSUPPORTED, "weight_only_skinny: K=%lld and C=%lld must be multiples of 128",
                    (long long)K, (long long)C);
  if (C != K && (N % 4 != 0 || (K / C) * N < 8 || scale_dt != x_dt || (zp && zp_dt != x_dt)))
    return qmm_fail(XLA_AMD_QMM_EUNSUPPORTED,
                    "weight_only_skinny: blockwise needs N %% 4 == 0, >= 8 scales and scale / zero point of x's dtype (N=%lld)",
                    (long long)N);
  if (N > (1 << 30) || K > (1 << 24) || M > (1 << 30))
    return qmm_fail(XLA_AMD_QMM_EUNSUPPORTED, "weight_only_skinny: dimension too large");
  if (((uintptr_t)x | (uintptr_t)w_tiled) & 15)
    return qmm_fail(XLA_AMD_QMM_EUNSUPPORTED, "weight_only_skinny: x and w must be 16-byte aligned");
  if (((uintptr_t)out & 15) && (N & 3) == 0)
    return qmm_fail(XLA_AMD_QMM_EUNSUPPORTED, "weight_only_skinny: out must be 16-byte aligned");
  if (M == 0) return XLA_AMD_QMM_OK;
  const int xsz = qmm_dt_size(x_dt), osz = qmm_dt_size(store_dt);
  const int pass = x_dt == XLA_AMD_DT_F32 ? 16 : 32;  // rows of x per pass over the weight
  for (int64_t m0 = 0; m0 < M; m0 += pass) {
    SkinnyArgs a;
    a.x = (const char*)x + (size_t)m0 * K * xsz;
    a.w = (const uint8_t*)w_tiled;
    a.scale = scale;
    a.zp = zp;
    a.out = (char*)out + (size_t)m0 * N * osz;
    a.M = (int)((M - m0) < pass ? (M - m0) : pass);
    a.N = (int)N; a.K = (int)K; a.C = (int)C;
    a.scale_dt = scale_dt; a.zp_dt = zp ? zp_dt : x_dt; a.out_dt = out_dt;
    a.dot_dt = dot_dt; a.store_dt = store_dt;
    a.k_per_slice = (int)K; a.slices = 1; a.part = nullptr; a.part_xs = nullptr; a.part_z = nullptr;
    a.G = xla_amd_qmm_tile_group(N, K, C, bits);
    int rc;
    if (x_dt == XLA_AMD_DT_BF16) rc = qmm_skinny_launch_bf16(a, bits, zp != nullptr, (hipStream_t)stream);
    else if (x_dt == XLA_AMD_DT_F16) rc = qmm_skinny_launch_f16(a, bits, zp != nullptr, (hipStream_t)stream);
    else rc = qmm_skinny_launch_f32(a, bits, zp != nullptr, (hipStream_t)stream);
    if (rc != XLA_AMD_QMM_OK) return rc;
  }
  return XLA_AMD_QMM_OK;
}
#endif  // QMM_SKINNY_XT
