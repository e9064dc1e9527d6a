// Weight-only quantized matmul for many rows of x with blockwise or int4 weights: a tiled
// bf16/f16 MFMA GEMM with the reference's per-block rounding points.
//
// The weight-streaming kernel (qmm_skinny.hip) re-reads the whole weight for every 32 rows of
// x; a prefill-sized M against blockwise int4 weights would take M / 32 passes.  Here a
// workgroup owns a tile of 64 rows x 128 channels and reads its weights once.
//
// Operands, as in qmm_wo_gemm.hip: weights come from the tiled copy (one block per 16 channels x
// 128 columns, 2 KB int8 / 1 KB int4, in MFMA operand order) straight into registers, one step
// (128 columns) ahead; x goes through LDS in two chunk slots filled by four copying waves, which
// also copy, for every resident step, the scale and zero point of the quantization block that
// step lies in ("entries" of the workgroup's 128 channels, indexed like the x tiles).  The
// kernel is persistent over the output tiles.
//
// Arithmetic (every dtype is x's; the reference's sequence, xla_quantized_matmul.py:115-133, with
// the per-channel case as one block):
//   per block s:  p = round_x(sum_c w x);  out_acc += scale[s,n] * p;  z_acc += round_x(sum_c x) * zp[s,n]
//   out = round_x(out_acc);  with a zero point  out = round_x(out - round_x(z_acc)).
// int4 weights are expanded to 1 + u/16 (u = w + 8) and the affine map is undone with the exact
// block sum of x, sum w x = 16 (sum a x - 1.5 sum x); the factor 16 is applied once per output (a
// power of two commutes with the rounding).
#include "qmm_common.h"
#include "qmm_frag.h"
#include "qmm_wo_bw.h"

#ifndef QMM_WO_BW_XT
#error "compile with -DQMM_WO_BW_XT=<XLA_AMD_DT_BF16|XLA_AMD_DT_F16 value>"
#endif

namespace {

using namespace qmm_frag;

constexpr int kComputeWaves = 4;
constexpr int kCopyWaves = 4;
constexpr int MT = 4;                    // 16-row tiles of x per workgroup
constexpr int NG = 2;                    // channel groups of 16 per computing wave
constexpr int BM = 16 * MT;              // 64 rows
constexpr int BN = 16 * NG * kComputeWaves;  // 128 channels
constexpr int X_TILE = BM * 256;         // bytes of the x columns of one step (128 columns, 2-byte x)
constexpr int CS = 4;                    // steps per chunk slot
constexpr int kEntryBytes = BN * 2;      // one entry: the workgroup's channels, 2-byte values
constexpr int kSclTensor = 2 * CS * kEntryBytes;  // the scales' entries (one per resident step), then the zero points'
constexpr int kSclBytes = 2 * kSclTensor;
constexpr int kLdsBytes = kSclBytes + 2 * CS * X_TILE;  // 4 KB + 128 KB
static_assert(kEntryBytes == 64 * 4, "one 4-byte copy instruction per entry");

struct BwItem {
  int m0, n0, rows;
};

// BLK1: quantization blocks of 128 columns, one per step.  The block's rounding sequence (some 180 of the step's 250
// vector instructions) then runs a step late, between the MFMAs of the next block, which accumulate into a second
// set of registers: a wave issues in order, so the MFMAs of a step only overlap with vector instructions that sit
// between them in the instruction stream.
template <int XT, int BITS, bool HASZP, bool BLK1>
__global__ void __launch_bounds__((kComputeWaves + kCopyWaves) * 64)
qmm_wo_bw_gemm_kernel(WoBwArgs a) {
  constexpr bool NEEDXS = HASZP || BITS == 4;        // block sums of x: zero point, int4 affine map
  constexpr int BLK = BITS == 8 ? 2048 : 1024;       // bytes of one weight block (16 channels x 128 columns)
  constexpr int WL = BITS == 8 ? 2 : 1;              // 16-byte loads per lane and block
  extern __shared__ __attribute__((aligned(16))) char smem[];
  typedef __attribute__((address_space(3))) void* lds_ptr_t;
  char* const xsm = smem + kSclBytes;

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r = lane & 15, g = lane >> 4;
  const int M = a.M, N = a.N, K = a.K, C = a.C;
  const int steps = K / 128;
  const int n_chunks = (steps + CS - 1) / CS;
  const int n_sblk = K / C;
  const int sub_per_block = C / 128;
  const int tiles_n = (N + BN - 1) / BN;
  const int n_items = tiles_n * ((M + BM - 1) / BM);
  // item -> (row tile, column tile), column tiles fastest: workgroups that run together share x rows
  auto item_of = [&](int it) __attribute__((always_inline)) {
    BwItem w;
    w.m0 = (it / tiles_n) * BM;
    w.n0 = (it % tiles_n) * BN;
    w.rows = min(BM, M - w.m0);
    return w;
  };

  if (__builtin_expect(wave >= kComputeWaves, 0)) {
    // ---- copying waves: chunk after chunk of x (and its scale entries) into the two slots in turn ----
    const int cw = wave - kComputeWaves;
    auto chunk_load = [&](const BwItem& w, int c, int slot_i) __attribute__((always_inline)) {
      const int s0 = c * CS;
      const int nst = min(CS, steps - s0);
      // entry e of the slot: step s0 + e.  One instruction copies one entry, 4 bytes (two channels) per lane;
      // wave cw copies entry cw of the scales and of the zero points.
      static_assert(CS == kCopyWaves, "one entry per copying wave");
      {
        const int k_at = min(s0 + cw, steps - 1) * 128;
        const int sblk = min(k_at / C, n_sblk - 1);
        int ch = w.n0 + 2 * lane;
        if (ch + 2 > N) ch = N - 2;  // channels past N: any valid address (never used)
        const size_t off = ((size_t)sblk * N + ch) * 2;
        char* const ent = smem + (slot_i * CS + cw) * kEntryBytes;
        __builtin_amdgcn_global_load_lds((const void*)((const char*)a.scale + off), (lds_ptr_t)ent, 4, 0, 0);
        if constexpr (HASZP)
          __builtin_amdgcn_global_load_lds((const void*)((const char*)a.zp + off), (lds_ptr_t)(ent + kSclTensor), 4, 0, 0);
      }
      char* const slot = xsm + slot_i * (CS * X_TILE);
      const char* const xb = (const char*)a.x + (size_t)w.m0 * K * 2;
      // a row of one step is 256 bytes: an instruction copies four consecutive rows
      // (lane l: row l/16 of the four, chunk l%16), swizzled on the source side
      for (int r4 = cw * 4; r4 < w.rows; r4 += kCopyWaves * 4) {
        const int row = min(r4 + (lane >> 4), w.rows - 1);  // rows past the end repeat the last one
        const int chunk = (lane & 15) ^ (row & 15);
        const char* src = xb + (size_t)row * ((size_t)K * 2) + (size_t)s0 * 256 + chunk * 16;
        char* dst = slot + r4 * 256;
        for (int t = 0; t < nst; ++t)
          __builtin_amdgcn_global_load_lds((const void*)(src + t * 256), (lds_ptr_t)(dst + t * X_TILE), 16, 0, 0);
      }
    };
    int it = blockIdx.x;
    BwItem cur = item_of(it);
    int c = 0, ring = 0;  // ring: chunks since the kernel began; chunk `ring` lives in slot ring % 2
    chunk_load(cur, 0, 0);
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    for (;;) {
      qmm_bare_barrier();  // chunk `ring` is there, chunk ring - 1 has been read
      ++c; ++ring;
      if (c == n_chunks) {
        it += gridDim.x;
        if (it >= n_items) break;
        cur = item_of(it);
        c = 0;
      }
      chunk_load(cur, c, ring & 1);
      __builtin_amdgcn_s_waitcnt(0x0F70);
    }
    return;
  }

  // ---- computing waves ----
  // wave w owns the channel groups (n0/16 + w*NG) .. + NG-1 of the item's column tile
  const int n_blk = K / 128;  // blocks per channel group in the tiled weight
  const int groups = (N + 15) / 16;
  const uint8_t* wp[NG];
  auto set_weights = [&](const BwItem& w) __attribute__((always_inline)) {
    qmm_static_for<NG>([&](auto gc) {
      constexpr int gi = gc;
      const int grp = min(w.n0 / 16 + wave * NG + gi, groups - 1);  // groups past N re-read the last one
      wp[gi] = a.w + (size_t)grp * n_blk * BLK + lane * 16;
    });
  };
  // the weights of a step are requested a whole step ahead into `wnext` and handed over when the step begins
  i32x4 wcur[NG][WL], wnext[NG][WL];
  auto load_next = [&](int blk) __attribute__((always_inline)) {
    qmm_static_for<NG>([&](auto gc) {
      constexpr int gi = gc;
      qmm_static_for<WL>([&](auto hc) {
        constexpr int h = hc;
        // (an ordinary load, not a streaming one: the other row tiles read the same block out of L2)
        wnext[gi][h] = *(const i32x4*)(wp[gi] + (size_t)blk * BLK + h * 1024);
      });
    });
  };

  f32x4 acc[NG][MT], sacc[NG][MT], zacc[NG][MT], xs[MT];
  auto clear_block = [&]() __attribute__((always_inline)) {
    qmm_static_for<MT>([&](auto mc) {
      constexpr int mt = mc;
      xs[mt] = f32x4{0, 0, 0, 0};
      qmm_static_for<NG>([&](auto gc) { acc[(int)gc][mt] = f32x4{0, 0, 0, 0}; });
    });
  };
  // End of a quantization block whose last step is in LDS tile `tile`.
  auto block_epilogue = [&](int tile) __attribute__((always_inline)) {
    float xs_r[MT];
    qmm_static_for<MT>([&](auto mc) { xs_r[(int)mc] = NEEDXS ? qmm_round_dt(xs[(int)mc][0], XT) : 0.f; });
    qmm_static_for<NG>([&](auto gc) {
      constexpr int gi = gc;
      const char* ent = smem + tile * kEntryBytes + ((wave * NG + gi) * 16 + 4 * g) * 2;
      const i32x2 sraw = *(const i32x2*)ent;
      i32x2 zraw = {0, 0};
      if constexpr (HASZP) zraw = *(const i32x2*)(ent + kSclTensor);
      qmm_static_for<4>([&](auto vc) {
        constexpr int v = vc;
        const uint32_t sw = (uint32_t)sraw[v >> 1], zw = (uint32_t)zraw[v >> 1];
        const float sc = qmm_from_raw((v & 1) ? (sw >> 16) : (sw & 0xffffu), XT);
        const float zv = HASZP ? qmm_from_raw((v & 1) ? (zw >> 16) : (zw & 0xffffu), XT) : 0.f;
        qmm_static_for<MT>([&](auto mc) {
          constexpr int mt = mc;
          float d = acc[gi][mt][v];
          if constexpr (BITS == 4) d = fmaf(-1.5f, xs[mt][0], d);  // (times 16, applied at the end)
          const float p = qmm_round_dt(d, XT);
          sacc[gi][mt][v] = fmaf(sc, p, sacc[gi][mt][v]);
          if constexpr (HASZP) zacc[gi][mt][v] = fmaf(xs_r[mt], zv, zacc[gi][mt][v]);
        });
      });
    });
    clear_block();
  };

  int block_left = sub_per_block;  // steps left in the current quantization block; uniform
  // one step (128 columns) out of LDS tile `tile`
  auto compute = [&](int tile) __attribute__((always_inline)) {
    const char* xbase = xsm + tile * X_TILE;
    qmm_static_for<4>([&](auto jc) {
      constexpr int j = jc;
      i32x4 xq[MT];
      qmm_static_for<MT>([&](auto mc) {
        constexpr int mt = mc;
        xq[mt] = *(const i32x4*)(xbase + (16 * mt + r) * 256 + (((4 * g + j) ^ r) * 16));
      });
      qmm_static_for<NG>([&](auto gc) {
        constexpr int gi = gc;
        i32x4 af;
        if constexpr (BITS == 8) {
          const i32x4 src = wcur[gi][j >> 1];
          af = cvt_w8<XT>((uint32_t)src[(j & 1) * 2], (uint32_t)src[(j & 1) * 2 + 1]);
        } else {
          af = cvt_w4<XT>((uint32_t)wcur[gi][0][j]);
        }
        qmm_static_for<MT>([&](auto mc) {
          constexpr int mt = mc;
          acc[gi][mt] = mfma16<XT>(af, xq[mt], acc[gi][mt]);
        });
      });
      if constexpr (NEEDXS) {
        qmm_static_for<MT>([&](auto mc) {
          constexpr int mt = mc;
          xs[mt] = mfma16<XT>(ones_frag<XT>(), xq[mt], xs[mt]);
        });
      }
    });
    if (--block_left == 0) {
      block_epilogue(tile);
      block_left = sub_per_block;
    }
  };

  // ---- results: four consecutive channels of one row per lane ----
  auto store_results = [&](const BwItem& done) __attribute__((always_inline)) {
  constexpr float kFactor = BITS == 4 ? 16.0f : 1.0f;
  qmm_static_for<MT>([&](auto mc) {
    constexpr int mt = mc;
    const int m = done.m0 + 16 * mt + r;
    qmm_static_for<NG>([&](auto gc) {
      constexpr int gi = gc;
      const int n = done.n0 + (wave * NG + gi) * 16 + 4 * g;
      if (m < M && n < N) {  // N % 4 == 0: the four channels exist and the address is 8-byte aligned
        float o[4];
        qmm_static_for<4>([&](auto vc) {
          constexpr int v = vc;
          float t = qmm_round_dt(kFactor * sacc[gi][mt][v], XT);
          if constexpr (HASZP) t = qmm_round_dt(t - qmm_round_dt(zacc[gi][mt][v], XT), XT);
          o[v] = t;
        });
        uint32_t lo, hi;
        if constexpr (XT == XLA_AMD_DT_BF16) {
          lo = qmm_f32x2_to_bf16x2(o[0], o[1]); hi = qmm_f32x2_to_bf16x2(o[2], o[3]);
        } else {
          lo = qmm_f32x2_to_f16x2(o[0], o[1]); hi = qmm_f32x2_to_f16x2(o[2], o[3]);
        }
        *(i32x2*)((uint16_t*)a.out + (size_t)m * N + n) = i32x2{(int)lo, (int)hi};
      }
    });
  });
  };
  int it = blockIdx.x;
  BwItem cur = item_of(it);
  set_weights(cur);
  load_next(0);
  int ring = 0;

  // ---- one block per step: the block's sums in two sets of registers, used in turn ----
  f32x4 acc2[2][NG][MT], xs2[2][MT];
  i32x2 ent_s[2][NG], ent_z[2][NG];  // scales and zero points of this lane's channels for the block in set P
  // The rounding sequence of the block in set Q for the results (gi, v, mt) and (gi, v, mt + 1), in kPhases parts
  // (one after each of kPhases consecutive MFMAs): the dot products rounded and packed; unpacked and added to the
  // scaled sums; the zero-point sums.
  float xs_r[MT];
  uint32_t packed = 0;  // the pair's rounded dot products between the first and the second part
  constexpr int kPairs = NG * 4 * (MT / 2);                 // pairs of results per block and lane
  constexpr int kSlots = 4 * (NG * MT + (NEEDXS ? MT : 0));  // MFMAs per step
  constexpr int kPhases = kSlots / kPairs;                  // MFMAs per pair
  static_assert(MT % 2 == 0 && kSlots % kPairs == 0 && (kPhases == 2 || kPhases == 3), "the pairs spread evenly over the step's MFMAs");
  auto block_pair = [&](auto qc, auto prc, auto phc) __attribute__((always_inline)) {
    constexpr int Q = qc, pr = prc, ph = phc;  // pair (gi, v, mt): mt fastest
    constexpr int gi = pr / (4 * (MT / 2)), v = (pr / (MT / 2)) % 4, mt = 2 * (pr % (MT / 2));
    if constexpr (ph == 0) {
      float d0 = acc2[Q][gi][mt][v], d1 = acc2[Q][gi][mt + 1][v];
      if constexpr (BITS == 4) {  // (times 16, applied at the end)
        d0 = fmaf(-1.5f, xs2[Q][mt][0], d0);
        d1 = fmaf(-1.5f, xs2[Q][mt + 1][0], d1);
      }
      packed = XT == XLA_AMD_DT_BF16 ? qmm_f32x2_to_bf16x2(d0, d1) : qmm_f32x2_to_f16x2(d0, d1);
    }
    if constexpr (ph == 1) {
      const uint32_t sw = (uint32_t)ent_s[Q][gi][v >> 1];
      const float sc = qmm_from_raw((v & 1) ? (sw >> 16) : (sw & 0xffffu), XT);
      const float p0 = qmm_from_raw(packed & 0xffffu, XT), p1 = qmm_from_raw(packed >> 16, XT);
      sacc[gi][mt][v] = fmaf(sc, p0, sacc[gi][mt][v]);
      sacc[gi][mt + 1][v] = fmaf(sc, p1, sacc[gi][mt + 1][v]);
    }
    if constexpr (HASZP && ph == kPhases - 1) {
      const uint32_t zw = (uint32_t)ent_z[Q][gi][v >> 1];
      const float zv = qmm_from_raw((v & 1) ? (zw >> 16) : (zw & 0xffffu), XT);
      zacc[gi][mt][v] = fmaf(xs_r[mt], zv, zacc[gi][mt][v]);
      zacc[gi][mt + 1][v] = fmaf(xs_r[mt + 1], zv, zacc[gi][mt + 1][v]);
    }
  };
  auto block_sums_of_x = [&](auto qc) __attribute__((always_inline)) {
    constexpr int Q = qc;
    qmm_static_for<MT>([&](auto mc) { xs_r[(int)mc] = NEEDXS ? qmm_round_dt(xs2[Q][(int)mc][0], XT) : 0.f; });
  };
  // Constants of the int4 expansion and the fragment of ones kept in registers the compiler cannot see through: it
  // would otherwise build the ones again for every j (two moves per MFMA against them), and with both constants of
  // (x & mask) | one as literals it cannot use the single instruction for it.
  i32x4 ones = ones_frag<XT>();
  uint32_t k_one = XT == XLA_AMD_DT_BF16 ? 0x3F803F80u : 0x3C003C00u;
  uint32_t k_mask = XT == XLA_AMD_DT_BF16 ? 0x00780078u : 0x03C003C0u;
  asm volatile("" : "+v"(ones), "+v"(k_one), "+s"(k_mask));
  // element q (two columns) of the fragment (j, gi) of the step's weights
  auto frag_q = [&](auto jc, auto gic, auto qc) __attribute__((always_inline)) {
    constexpr int j = jc, gi = gic, q = qc;
    if constexpr (BITS == 8) {
      return (int)cvt_w2<XT>((uint32_t)wcur[gi][j >> 1][(j & 1) * 2 + q / 2], qmm_const<(q & 1)>{});
    } else {
      const uint32_t d = (uint32_t)wcur[gi][0][j];
      constexpr int sh = XT == XLA_AMD_DT_BF16 ? 4 * q - 3 : 4 * q - 6;  // right shift (negative: left)
      const uint32_t t = sh < 0 ? d << (sh < 0 ? -sh : 0) : d >> (sh < 0 ? 0 : sh);
      return (int)((t & k_mask) | k_one);
    }
  };
  // One step = one block into set P, out of LDS tile `tile`, with the rounding sequence of the block in set 1 - P
  // and the conversions of the step's own weights spread over its MFMAs.
  auto step_blk1 = [&](int tile, auto pc) __attribute__((always_inline)) {
    constexpr int P = pc, Q = 1 - P;
    const char* xbase = xsm + tile * X_TILE;
    qmm_static_for<NG>([&](auto gc) {
      constexpr int gi = gc;
      const char* ent = smem + tile * kEntryBytes + ((wave * NG + gi) * 16 + 4 * g) * 2;
      ent_s[P][gi] = *(const i32x2*)ent;
      if constexpr (HASZP) ent_z[P][gi] = *(const i32x2*)(ent + kSclTensor);
      else ent_z[P][gi] = i32x2{0, 0};
    });
    i32x4 xq[MT];
    qmm_static_for<MT>([&](auto mc) {
      constexpr int mt = mc;
      xq[mt] = *(const i32x4*)(xbase + (16 * mt + r) * 256 + (((4 * g + 0) ^ r) * 16));
    });
    i32x4 af, af_next;
    qmm_static_for<4>([&](auto qc) { af[(int)qc] = frag_q(qmm_const<0>{}, qmm_const<0>{}, qc); });
    af_next = af;
    block_sums_of_x(qmm_const<Q>{});
    __builtin_amdgcn_sched_barrier(0);
    // after MFMA `slot` of the step: its share of the other block's rounding sequence
    auto after = [&](auto slotc) __attribute__((always_inline)) {
      constexpr int slot = slotc;
      block_pair(qmm_const<Q>{}, qmm_const<slot / kPhases>{}, qmm_const<slot % kPhases>{});
      __builtin_amdgcn_sched_barrier(0);
    };
    constexpr int kPerJ = kSlots / 4;
    static_assert(MT == 4, "a fragment has four elements: one is converted after each of the MT MFMAs of a fragment");
    qmm_static_for<4>([&](auto jc) {
      constexpr int j = jc;
      qmm_static_for<NG>([&](auto gc) {
        constexpr int gi = gc;
        // the next fragment in the order (j, 0), (j, 1), .., (j + 1, 0): converted during this one's MFMAs, the first
        // of the next j during the MFMAs against the ones (or, without them, during the last fragment of this j)
        constexpr bool kConvHere = gi + 1 < NG || (!NEEDXS && j + 1 < 4);
        constexpr int jn = gi + 1 < NG ? j : j + 1, gn = gi + 1 < NG ? gi + 1 : 0;
        qmm_static_for<MT>([&](auto mc) {
          constexpr int mt = mc;
          if constexpr (j == 0) acc2[P][gi][mt] = mfma16<XT>(af, xq[mt], f32x4{0, 0, 0, 0});
          else acc2[P][gi][mt] = mfma16<XT>(af, xq[mt], acc2[P][gi][mt]);
          if constexpr (kConvHere) af_next[mt] = frag_q(qmm_const<jn>{}, qmm_const<gn>{}, mc);
          if constexpr (!NEEDXS && gi == NG - 1 && j + 1 < 4)
            xq[mt] = *(const i32x4*)(xbase + (16 * mt + r) * 256 + (((4 * g + j + 1) ^ r) * 16));
          after(qmm_const<j * kPerJ + gi * MT + mt>{});
        });
        if constexpr (kConvHere) af = af_next;
      });
      if constexpr (NEEDXS) {
        qmm_static_for<MT>([&](auto mc) {
          constexpr int mt = mc;
          if constexpr (j == 0) xs2[P][mt] = mfma16<XT>(ones, xq[mt], f32x4{0, 0, 0, 0});
          else xs2[P][mt] = mfma16<XT>(ones, xq[mt], xs2[P][mt]);
          if constexpr (j + 1 < 4) {
            af_next[mt] = frag_q(qmm_const<j + 1>{}, qmm_const<0>{}, mc);
            xq[mt] = *(const i32x4*)(xbase + (16 * mt + r) * 256 + (((4 * g + j + 1) ^ r) * 16));
          }
          after(qmm_const<j * kPerJ + NG * MT + mt>{});
        });
        if constexpr (j + 1 < 4) af = af_next;
      }
    });
  };
  if constexpr (BLK1) {
    for (;;) {
      qmm_static_for<MT>([&](auto mc) {
        constexpr int mt = mc;
        xs2[1][mt] = f32x4{0, 0, 0, 0};
        qmm_static_for<NG>([&](auto gc) {
          sacc[(int)gc][mt] = f32x4{0, 0, 0, 0};
          zacc[(int)gc][mt] = f32x4{0, 0, 0, 0};
          acc2[1][(int)gc][mt] = f32x4{0, 0, 0, 0};
        });
      });
      // (the first step's rounding sequence runs over zeros: a scale of 0 and sums of 0 add nothing)
      qmm_static_for<NG>([&](auto gc) { ent_s[1][(int)gc] = i32x2{0, 0}; ent_z[1][(int)gc] = i32x2{0, 0}; });
      int s = 0;
      for (int c = 0; c < n_chunks; ++c, ++ring) {
        qmm_bare_barrier();  // chunk `ring` is there (the copying waves waited for it)
        const int tile0 = (ring & 1) * CS - c * CS;
        const int s_end = min(steps, (c + 1) * CS);
        static_assert(CS % 2 == 0, "a chunk begins with set 0");
        qmm_static_for<CS>([&](auto kc) {
          if (s < s_end) {
            qmm_static_for<NG>([&](auto gc) {
              qmm_static_for<WL>([&](auto hc) { wcur[(int)gc][(int)hc] = wnext[(int)gc][(int)hc]; });
            });
            if (s + 1 < steps) load_next(s + 1);
            step_blk1(tile0 + s, qmm_const<(int)kc % 2>{});
            ++s;
          }
        });
      }
      const BwItem done = cur;
      const int it_next = it + (int)gridDim.x;
      const bool more = it_next < n_items;
      if (more) {
        it = it_next;
        cur = item_of(it);
        set_weights(cur);
        load_next(0);
      }
      // the last block's rounding sequence: it is in set 1 after an even number of steps, else in set 0
      auto last_block = [&](auto qc) __attribute__((always_inline)) {
        block_sums_of_x(qc);
        qmm_static_for<kPairs>([&](auto prc) {
          qmm_static_for<kPhases>([&](auto phc) { block_pair(qc, prc, phc); });
        });
      };
      if (steps & 1) last_block(qmm_const<0>{});
      else last_block(qmm_const<1>{});
      store_results(done);
      if (!more) break;
    }
    return;
  }

  for (;;) {
    qmm_static_for<MT>([&](auto mc) {
      constexpr int mt = mc;
      qmm_static_for<NG>([&](auto gc) {
        sacc[(int)gc][mt] = f32x4{0, 0, 0, 0};
        zacc[(int)gc][mt] = f32x4{0, 0, 0, 0};
      });
    });
    clear_block();
    block_left = sub_per_block;
    int s = 0;
    for (int c = 0; c < n_chunks; ++c, ++ring) {
      qmm_bare_barrier();  // chunk `ring` is there (the copying waves waited for it)
      const int tile0 = (ring & 1) * CS - c * CS;
      const int s_end = min(steps, (c + 1) * CS);
      for (; s < s_end; ++s) {
        // hand over the weights of this step (the only loads this wave has in flight), request the next step's
        qmm_static_for<NG>([&](auto gc) {
          qmm_static_for<WL>([&](auto hc) { wcur[(int)gc][(int)hc] = wnext[(int)gc][(int)hc]; });
        });
        if (s + 1 < steps) load_next(s + 1);
        compute(tile0 + s);
      }
    }

    // the next item's first weights are requested before this item's results are stored
    const BwItem done = cur;
    const int it_next = it + (int)gridDim.x;
    const bool more = it_next < n_items;
    if (more) {
      it = it_next;
      cur = item_of(it);
      set_weights(cur);
      load_next(0);
    }

    store_results(done);
    if (!more) break;
  }
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

template <int XT, int BITS>
int launch(const WoBwArgs& a, hipStream_t stream) {
  const int64_t items = (int64_t)((a.M + BM - 1) / BM) * ((a.N + BN - 1) / BN);
  const int cus = cu_count();
  const dim3 grid((unsigned)(items < cus ? items : cus)), block((kComputeWaves + kCopyWaves) * 64);
  auto go = [&](auto kern) -> int {
    static std::atomic<uint64_t> lds_set{0};
    const int rc = qmm_set_max_lds((const void*)kern, kLdsBytes, lds_set, "weight_only_gemm hipFuncSetAttribute");
    if (rc != XLA_AMD_QMM_OK) return rc;
    hipLaunchKernelGGL(kern, grid, block, kLdsBytes, stream, a);
    return QMM_CHECK_LAUNCH("weight_only_gemm (blockwise) launch");
  };
  // blocks of 128 columns: the kernel with two sets of block sums (int8 weights with a zero point keep the other
  // one: their two 16-byte weight loads per row set leave no registers for the second set)
  if (a.C == 128) {
    if (!a.zp) return go(qmm_wo_bw_gemm_kernel<XT, BITS, false, true>);
    if constexpr (BITS == 4) return go(qmm_wo_bw_gemm_kernel<XT, BITS, true, true>);
  }
  return a.zp ? go(qmm_wo_bw_gemm_kernel<XT, BITS, true, false>) : go(qmm_wo_bw_gemm_kernel<XT, BITS, false, false>);
}

}  // namespace

#if QMM_WO_BW_XT == XLA_AMD_DT_BF16
int qmm_wo_bw_launch_bf16(const WoBwArgs& a, int bits, hipStream_t stream) {
  return bits == 8 ? launch<XLA_AMD_DT_BF16, 8>(a, stream) : launch<XLA_AMD_DT_BF16, 4>(a, stream);
}
#else
int qmm_wo_bw_launch_f16(const WoBwArgs& a, int bits, hipStream_t stream) {
  return bits == 8 ? launch<XLA_AMD_DT_F16, 8>(a, stream) : launch<XLA_AMD_DT_F16, 4>(a, stream);
}
#endif
