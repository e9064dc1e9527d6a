/*
 * xla_amd_qmm.h -- C ABI of libxla_amd_qmm.so: gfx950 (MI355X) kernels for the
 * quantized-linear operator torch.ops.xla.quantized_matmul and the int8
 * quantized_matmul_int8 operator of PyTorch/XLA.
 *
 * The reference has no native entry point for this path: the operator schema in
 *   torch_xla/experimental/xla_quantized_matmul.py:7-9
 *   torch_xla/experimental/custom_kernel.py:1742-1744
 * is its plugin boundary and the arithmetic is emitted as XLA ops.  Each entry
 * point below cites the reference statement(s) it replaces.
 *
 * Conventions
 *  - plain pointers and sizes only; every pointer is DEVICE memory unless the
 *    comment says "host"; all tensors are dense and contiguous (row-major).
 *  - `stream` is a hipStream_t passed as void* (NULL = default stream).  No
 *    entry point synchronises the device, allocates or frees device memory, or
 *    keeps a pointer after it returns.
 *  - return value: XLA_AMD_QMM_OK or a negative XLA_AMD_QMM_E* code; the text
 *    of the last error of the calling thread is xla_amd_qmm_last_error().
 *    No C++ exception crosses this boundary.
 *  - M = rows of x (tokens), K = in features, N = out features,
 *    C = block size along K (C == K for per-channel), S = K / C.
 */
#ifndef XLA_AMD_QMM_H_
#define XLA_AMD_QMM_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define XLA_AMD_QMM_ABI_VERSION 5

/* return codes */
#define XLA_AMD_QMM_OK 0
#define XLA_AMD_QMM_EINVAL (-1)       /* null pointer, bad size, bad enum */
#define XLA_AMD_QMM_EUNSUPPORTED (-2) /* shape/dtype the chosen kernel cannot take */
#define XLA_AMD_QMM_EHIP (-3)         /* HIP launch/runtime error */

/* element types of floating tensors */
#define XLA_AMD_DT_F32 0
#define XLA_AMD_DT_BF16 1
#define XLA_AMD_DT_F16 2

/* integer dtypes of quantized tensors (quantize_affine / dequantize_affine) */
#define XLA_AMD_QDT_I8 0
#define XLA_AMD_QDT_U8 1
#define XLA_AMD_QDT_I16 2
#define XLA_AMD_QDT_I32 3

/* float -> int8 conversion of a rounded value outside [-128,127]
 * (reference: `.to(torch.int8)` with no clamp, xla_quantized_matmul.py:72;
 * XLA's ConvertElementType saturates, torch's CPU cast wraps modulo 256). */
#define XLA_AMD_OVERFLOW_SATURATE 0
#define XLA_AMD_OVERFLOW_WRAP 1

/* memory layout of the int8 weight container handed to the operator */
#define XLA_AMD_W_NK 0  /* per-channel: [N, K]                 (xla_quantized_matmul.py:88) */
#define XLA_AMD_W_SCN 1 /* blockwise:   [K/C, C, N]            (xla_quantized_matmul.py:89) */

/* kernels the dispatcher can choose (xla_amd_qmm_dispatch) */
#define XLA_AMD_KERNEL_GENERIC 0    /* one thread per output, any shape          */
#define XLA_AMD_KERNEL_SKINNY_MFMA 1 /* weight-streaming GEMV / skinny GEMM       */
#define XLA_AMD_KERNEL_W8A8_MFMA 2  /* LDS-tiled int8 MFMA GEMM                   */
#define XLA_AMD_KERNEL_W8A8_GENERIC 3
#define XLA_AMD_KERNEL_WEIGHT_ONLY_GEMM 4 /* tiled bf16/f16 MFMA GEMM on int8 weights */

int xla_amd_qmm_abi_version(void);

/* Text of the last error raised on the calling thread ("" if none). Host. */
const char* xla_amd_qmm_last_error(void);

/*
 * Bytes of the K-major ("packed") copy of a weight: N*K for bits == 8,
 * N*K/2 for bits == 4.  Returns 0 for arguments the pack kernel rejects.
 */
size_t xla_amd_qmm_packed_bytes(int64_t N, int64_t K, int bits);

/*
 * One-time re-layout of a weight into plain K-major form (rows of K values;
 * for bits == 4 two values per byte).  Replaces the reference's `_xla_cast_int4(w, w.cpu()...tolist())`
 * (xla_quantized_matmul.py:101-103 -> csrc/ops/cast_int4.cpp:30-39), which
 * rebuilds the weight as an s4 literal: values are unchanged, only storage.
 *   src_layout XLA_AMD_W_NK : w is [N, K]       (C ignored, S*C == K)
 *   src_layout XLA_AMD_W_SCN: w is [S, C, N]
 *   bits 8: packed[n*K + k] = w(n,k)
 *   bits 4: values must lie in [-8,7]; packed is [N, K/2] bytes, K % 8 == 0.
 *           Each aligned group of 8 consecutive k of a row is one 32-bit
 *           little-endian word; nibble j of the word (bits 4j..4j+3) holds
 *           (w(n, k0 + P[j]) + 8) with P = {0,2,4,6,1,3,5,7}.
 */
int xla_amd_qmm_pack_weight(const int8_t* w, void* packed, int64_t S, int64_t C, int64_t N,
                            int src_layout, int bits, void* stream);

/*
 * Channels per group of the tiled copy of a weight [N, K] with quantization
 * blocks of C columns (C == K or C <= 0: per-channel): 16, except that
 * per-channel int8 weights of 4096 channels or more are tiled in groups of
 * 14, 12 or 10 channels when that fills the chip's 1024 wave slots better
 * (14336 channels: groups of 14, 1024 waves instead of 896).  Host.
 */
int xla_amd_qmm_tile_group(int64_t N, int64_t K, int64_t C, int bits);

/*
 * Bytes of the tiled copy of a weight that the streaming kernel reads:
 * ceil(N/G)*G * K for bits == 8 (G = xla_amd_qmm_tile_group), half of that
 * for bits == 4.  Needs K % 128 == 0; returns 0 for arguments the tile kernel
 * rejects.
 */
size_t xla_amd_qmm_tiled_bytes(int64_t N, int64_t K, int64_t C, int bits);

/*
 * One-time re-layout of a weight into the tiled form the streaming kernel
 * reads (same arguments and the same reference statement as
 * xla_amd_qmm_pack_weight: values are unchanged, only storage).  Needs
 * K % 128 == 0.  With G = xla_amd_qmm_tile_group(N, K, C, bits) there is, for
 * every group p of G consecutive channels and every sub-step t of 128
 * consecutive columns, one block of BLK bytes at byte offset
 * (p * (K/128) + t) * BLK; channels past N are stored as zero.
 *   bits 8 (BLK 128 G): byte ((h*4 + q)*G + r)*16 + j (h in 0..1, q in 0..3, r in 0..G-1,
 *           j in 0..15) holds w(G p + r, 128t + 32q + 16h + j).
 *   bits 4 (BLK 1024, G = 16): the 32-bit word at byte (q*16 + r)*16 + 4i (i in 0..3) holds the
 *           8 columns 128t + 32q + 8i .. +7 of channel 16p + r in the
 *           nibble order of xla_amd_qmm_pack_weight.
 * With G = 16 a 64-lane load of 16 bytes per lane from consecutive addresses
 * puts into lane l = 16q + r exactly the MFMA operand fragment of channel r;
 * with a narrower group lane 16q + r' reads row r' - (G p % 4) of quarter q
 * (clamped to 0..G-1), so that the lane's four results are the channels
 * 4 floor(G p / 4) + 4q .. +3: four-aligned, as with groups of 16.
 */
int xla_amd_qmm_tile_weight(const int8_t* w, void* tiled, int64_t S, int64_t C, int64_t N,
                            int src_layout, int bits, void* stream);

/*
 * Inverse of xla_amd_qmm_tile_weight: rebuilds the operator's int8 container
 * ([N, K] for XLA_AMD_W_NK, [S, C, N] for XLA_AMD_W_SCN) from a tiled copy, so
 * that a module which keeps only the tiled form on the device can still save
 * the reference's `weight` buffer (xla_quantized_matmul.py:202, :231) unchanged.
 */
int xla_amd_qmm_untile_weight(const void* tiled, int8_t* w, int64_t S, int64_t C, int64_t N,
                              int dst_layout, int bits, void* stream);

/*
 * Weight-only quantized matmul, fast path: streams a tiled weight once and
 * keeps up to 32 rows of x per pass in MFMA fragments (passes over w repeat
 * for larger M).  Replaces, with the reference's rounding points,
 *   per-channel (C == K):  out = F.linear(x, w) * scaler      (:113-114)
 *   blockwise   (C <  K):  einsum('scn,...sc->...sn'), einsum('sn,...sn->...n') (:122-124)
 *   zero point:            out -= rowsum/blocksum(x) (x) zp    (:125-133)
 * x [M,K] (bf16/f16/f32), w_tiled from xla_amd_qmm_tile_weight, scale [S,N],
 * zp [S,N] or NULL, out [M,N].
 * Needs K % 128 == 0 and C % 128 == 0; blockwise (C < K) also needs N % 4 == 0
 * and scale / zp of x's dtype (the reference's einsum raises on mixed dtypes);
 * else XLA_AMD_QMM_EUNSUPPORTED.
 * out_dt must be the torch promotion of (x_dt, scale_dt).
 * dot_dt is the dtype the dot product is rounded to before it is scaled: x_dt
 * for quantized_matmul (the XLA dot's result has x's type, csrc/ops/ops.cpp:252-259),
 * or XLA_AMD_DT_F32 (per-channel only) for the float branch of the Pallas kernel,
 * which keeps a float32 accumulator, scales it and casts once
 * (pallas_kernels/quantized_matmul_kernel.py:108-121, :246).
 * store_dt is the dtype out is stored as: out_dt, or the type of a final cast
 * of the result (`.to(x.dtype)`, custom_kernel.py:1105-1106; `.astype`,
 * quantized_matmul_kernel.py:121).
 */
int xla_amd_qmm_weight_only_skinny(const void* x, const void* w_tiled, const void* scale,
                                   const void* zp, void* out, int64_t M, int64_t N, int64_t K,
                                   int64_t C, int bits, int x_dt, int scale_dt, int zp_dt,
                                   int dot_dt, int out_dt, int store_dt, void* stream);

/*
 * Bytes of workspace xla_amd_qmm_weight_only_gemm needs for a shape (0 when it
 * needs none, or for arguments it rejects).
 */
size_t xla_amd_qmm_weight_only_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K, int64_t C, int bits);

/*
 * Weight-only quantized matmul for many rows of x (prefill-sized M), and for
 * few output channels with a long K: a tiled MFMA GEMM that reads the weight
 * once per tile of up to 128 rows, where xla_amd_qmm_weight_only_skinny reads
 * it once per 32 rows.  Replaces the same reference statements with the same
 * rounding points,
 *   out = F.linear(x, w) * scaler;  out -= rowsum(x) (x) zp   (xla_quantized_matmul.py:113-114, :125-133)
 * and, with dot_dt = f32, the float branch of the Pallas kernel
 * (pallas_kernels/quantized_matmul_kernel.py:108-121).
 * x [M,K] bf16 or f16, w_tiled from xla_amd_qmm_tile_weight, K % 128 == 0; other
 * cases return XLA_AMD_QMM_EUNSUPPORTED (the streaming kernel takes them).
 * Per-channel int8 weights (C == K, bits == 8): dtype arguments as for
 * xla_amd_qmm_weight_only_skinny.  Blockwise (C < K, C % 128 == 0) and int4
 * weights (bits == 4): a tile of 64 rows x 128 channels with the rounding points
 * of the blockwise statements (xla_quantized_matmul.py:115-133: every block's dot
 * product rounded to x's dtype before it is scaled); scale / zp [K/C, N]; they
 * need N % 4 == 0 and every dtype argument equal to x_dt, and use no workspace.
 * With at most 32 rows, few output channels and a long K (where
 * xla_amd_qmm_dispatch returns this kernel for such an M) the call runs the
 * streaming kernel over K slices instead, one slice of 64 channels per
 * workgroup, and a second kernel adds the slices in slice order; slices of
 * blockwise weights are whole quantization blocks, and what is added are the
 * blocks' scaled, rounded dot products (and zero-point terms), so the rounding
 * points stay the reference's.
 * When K is split over workgroups the partial sums live in `workspace`
 * (device memory of at least
 * xla_amd_qmm_weight_only_gemm_workspace_bytes(M, N, K, C, bits) bytes,
 * 16-byte aligned, free again when the call's work has completed); it may be
 * NULL when that size is 0.
 */
int xla_amd_qmm_weight_only_gemm(const void* x, const void* w_tiled, const void* scale, const void* zp,
                                 void* out, void* workspace, size_t workspace_bytes, int64_t M, int64_t N,
                                 int64_t K, int64_t C, int bits, int x_dt, int scale_dt, int zp_dt, int dot_dt,
                                 int out_dt, int store_dt, void* stream);

/*
 * The same for f32 activations (xla_amd_qmm_dispatch sends 128 rows or more
 * here; fewer take the streaming kernel, 16 rows per pass): out f32 [M,N] = F.linear(x, w) * scaler
 * (- rowsum(x) (x) zp), xla_quantized_matmul.py:113-114 with x of any floating
 * dtype, here f32.  x is split into three bf16 parts whose sum is x to the last
 * bit (hi = bf16(x), mid = bf16(x - hi), lo = bf16(x - hi - mid)) and the bf16
 * GEMM runs over the 3 K columns of the parts against the weight three times
 * over, accumulating in f32: every product is exact, so the result differs from
 * an f32 dot product by the order of the additions only.  Per-channel int8
 * weights, K % 128 == 0, 3 K <= 2^23; scale / zp of any floating dtype.
 * `workspace`: xla_amd_qmm_weight_only_gemm_f32_workspace_bytes(M, N, K) bytes
 * of device memory (the three parts: 6 M K), 16-byte aligned, free again when
 * the call's work has completed.
 */
size_t xla_amd_qmm_weight_only_gemm_f32_workspace_bytes(int64_t M, int64_t N, int64_t K);
int xla_amd_qmm_weight_only_gemm_f32(const float* x, const void* w_tiled, const void* scale, const void* zp,
                                     float* out, void* workspace, size_t workspace_bytes, int64_t M, int64_t N,
                                     int64_t K, int scale_dt, int zp_dt, void* stream);

/*
 * Weight-only quantized matmul for any shape, reading the operator's own
 * weight layout (one thread per output element; the slow, always-correct path
 * for shapes the streaming kernel rejects).  Same reference statements and
 * rounding points as xla_amd_qmm_weight_only_skinny.
 */
int xla_amd_qmm_weight_only_generic(const void* x, const int8_t* w, const void* scale,
                                    const void* zp, void* out, int64_t M, int64_t N, int64_t K,
                                    int64_t C, int w_layout, int x_dt, int scale_dt, int zp_dt,
                                    int dot_dt, int out_dt, int store_dt, void* stream);

/*
 * Per-token dynamic activation quantization (`_quantize_tensor`,
 * xla_quantized_matmul.py:56-73; Pallas `_quantize_array`,
 * pallas_kernels/quantized_matmul_kernel.py:10-18):
 *   max = amax(|x|, -1); scale = max / 127; x_q = int8(round_half_even(x / scale))
 * with every intermediate rounded to x_dt as the reference does op by op.
 * x [M,K], x_q int8 [M,K], x_scale [M] stored as scale_out_dt (x_dt for the
 * torch op, f32 for the Pallas variant).  A row of zeros yields x_q = 0,
 * scale = 0; a row that holds a NaN yields scale = NaN (as torch.amax does)
 * and x_q = 0 (the reference leaves both cases undefined).
 * x_sum (nullable) receives sum_k x_q[m,k] as int32 [M]: the factor of the
 * zero-point term once x has been replaced by its quantized form (:109,:128).
 */
int xla_amd_qmm_quantize_per_token(const void* x, int8_t* x_q, void* x_scale, int32_t* x_sum,
                                   int64_t M, int64_t K, int x_dt, int scale_out_dt,
                                   int overflow_policy, void* stream);

/*
 * int8 x int8 -> int32 GEMM with fused scale epilogue.  Replaces
 *   `_xla_dot_general(x_int, w, (([-1],[-1]),()), preferred_element_type=int32)`
 *   (xla_quantized_matmul.py:110-111 -> csrc/ops/dot_general.cpp:16-37),
 *   `out * scaler` (:114), the zero-point term (:125-133), `out * x_scale` (:135)
 *   and the Pallas matmul_kernel body (pallas_kernels/quantized_matmul_kernel.py:88-124).
 * x_q int8 [M,K], w int8 [N,K], x_scale [M], w_scale [N]; zp [N] and
 * x_sum int32 [M] (from xla_amd_qmm_quantize_per_token) both given or both NULL.
 * Epilogue per element, with round_d = round-to-nearest-even to dtype d:
 *   v = round_{cvt_dt}(float(acc))
 *   v = round_{mid_dt}(v * w_scale[n])
 *   if zp: v = round_{mid_dt}(v - round_{zpo_dt}(round_{zpo_dt}(float(x_sum[m])) * zp[n]))
 *   v = round_{out_dt}(v * x_scale[m])               -> out[m,n]
 * (torch converts an integer tensor to the float operand's dtype before it
 * multiplies, hence cvt_dt and the inner round of x_sum.)
 * If acc_out != NULL the raw int32 accumulators are also stored to
 * acc_out [M,N] (parity/debug).  If out == NULL only acc_out is written.
 * The MFMA kernel needs K % 16 == 0 and 16-byte aligned x_q and w; other
 * shapes run a one-thread-per-output kernel.
 * block_m/block_n select the workgroup tile (the role of batch_block_size /
 * out_block_size, custom_kernel.py:1088-1100): 0,0 = choose by shape;
 * otherwise one of the pairs xla_amd_qmm_w8a8_tile can return, else
 * XLA_AMD_QMM_EUNSUPPORTED.
 */
int xla_amd_qmm_w8a8_gemm(const int8_t* x_q, const int8_t* w, const void* x_scale,
                          const void* w_scale, const void* zp, const int32_t* x_sum, void* out,
                          int32_t* acc_out, int64_t M, int64_t N, int64_t K, int x_scale_dt,
                          int w_scale_dt, int zp_dt, int cvt_dt, int mid_dt, int zpo_dt,
                          int out_dt, int block_m, int block_n, void* stream);

/*
 * Bytes of workspace xla_amd_qmm_w8a8_linear needs for an [M, K] activation
 * against an [N, K] weight (0 for arguments it rejects).
 */
size_t xla_amd_qmm_w8a8_linear_workspace_bytes(int64_t M, int64_t N, int64_t K);

/*
 * The whole `quantize_activation=True` operator in one call: the statements of
 * xla_amd_qmm_quantize_per_token followed by those of xla_amd_qmm_w8a8_gemm
 * (xla_quantized_matmul.py:108-114, :125-135; Pallas wrapper
 * pallas_kernels/quantized_matmul_kernel.py:199-221 with its matmul_kernel).
 * x [M,K] of x_dt, w int8 [N,K], w_scale [N], zp [N] or NULL, out [M,N].
 * The quantized activations (int8 [M,K]), their scales (stored as x_scale_dt:
 * x_dt for the torch operator, f32 for the Pallas variant) and, with a zero
 * point, their row sums live in `workspace`: device memory of at least
 * xla_amd_qmm_w8a8_linear_workspace_bytes(M, N, K) bytes, 256-byte aligned,
 * which the call may overwrite entirely and does not need afterwards.
 * cvt_dt / mid_dt / out_dt, block_m / block_n as for xla_amd_qmm_w8a8_gemm
 * (the zero-point term is rounded to zp_dt).
 */
int xla_amd_qmm_w8a8_linear(const void* x, const int8_t* w, const void* w_scale, const void* zp,
                            void* out, void* workspace, size_t workspace_bytes, int64_t M, int64_t N,
                            int64_t K, int x_dt, int w_scale_dt, int zp_dt, int x_scale_dt, int cvt_dt,
                            int mid_dt, int out_dt, int overflow_policy, int block_m, int block_n,
                            void* stream);

/*
 * xla_amd_qmm_w8a8_linear without a workspace argument and without any
 * allocation.  It has no counterpart in the reference; it is for callers that
 * cannot allocate device memory around the call: code under HIP-graph capture,
 * tight serving loops, harnesses that forbid hipMalloc.  The quantized
 * activations live in a fixed array inside the library's device image (16 MiB
 * + 64 KiB, held by every GPU the library is loaded on until the process
 * ends): at most 8192 rows and M * K <= 16 Mi elements
 * (xla_amd_qmm_w8a8_linear_noalloc_limits), else XLA_AMD_QMM_EUNSUPPORTED.
 * Apart from the one-time set-up of a device (xla_amd_qmm_init, or the first
 * call on that device), the call performs no hipMalloc / hipFree and calls no
 * allocating library routine; outputs are identical to xla_amd_qmm_w8a8_linear.  Every
 * call on a GPU shares that GPU's array and nothing in it needs clearing
 * between calls (each call overwrites what it reads); calls that overlap in
 * time on one GPU (different streams or threads) race on it and must be
 * serialised by the caller.
 */
int xla_amd_qmm_w8a8_linear_noalloc(const void* x, const int8_t* w, const void* w_scale, const void* zp,
                                    void* out, int64_t M, int64_t N, int64_t K, int x_dt, int w_scale_dt,
                                    int zp_dt, int x_scale_dt, int cvt_dt, int mid_dt, int out_dt,
                                    int overflow_policy, int block_m, int block_n, void* stream);

/*
 * Per-device set-up of the library for the current device: resolves the address
 * of this GPU's copy of the fixed scratch array (the HIP runtime backs the array
 * with device memory when it is first looked up).  Optional:
 * xla_amd_qmm_w8a8_linear_noalloc does the same on its first call on a device.
 * Call it outside HIP-graph capture.  Safe to call repeatedly and from several
 * threads.
 */
int xla_amd_qmm_init(void);

/* Limits of xla_amd_qmm_w8a8_linear_noalloc: rows of x, and elements M * K of x.  Host pointers, nullable. */
void xla_amd_qmm_w8a8_linear_noalloc_limits(int64_t* max_rows, int64_t* max_elements);

/*
 * Shape-based choice between the kernels (the role of the tuned-table lookup
 * with fallback in torch_xla/experimental/custom_kernel.py:1088-1106).
 * Pure host function; returns an XLA_AMD_KERNEL_* id.
 */
int xla_amd_qmm_dispatch(int64_t M, int64_t N, int64_t K, int64_t C, int bits, int x_dt,
                         int quantize_activation);

/*
 * Tile configuration the W8A8 GEMM would use for a shape: fills
 * tile_mnk[3] = {block_M, block_N, block_K}; the analogue of
 * get_tuned_block_sizes (pallas_kernels/quantized_matmul_kernel.py:537-555).
 */
int xla_amd_qmm_w8a8_tile(int64_t M, int64_t N, int64_t K, int32_t* tile_mnk /* host */);

/*
 * Affine quantization of a whole tensor, per tensor (channels == 1) or per
 * channel; the contiguous tensor is read as [outer, channels, inner].
 *   q[o,c,i] = cast(clamp(rint(f32(x[o,c,i]) * inv_scale[c]) + zp[c], qmin, qmax))
 * (all in f32, rint = half to even, NaN -> 0): the decomposition that
 * quantized_decomposed::quantize_per_tensor / quantize_per_channel denote
 * (bound to XLA in torch_xla/experimental/quantized.py:7-22, where they lower
 * to stablehlo.uniform_quantize through _xla_quantize_tensor,
 * csrc/init_python_bindings.cpp:1964).  inv_scale and zp are device arrays of
 * `channels` entries.
 */
int xla_amd_qmm_quantize_affine(const void* x, void* q, const float* inv_scale, const int32_t* zp,
                                int64_t outer, int64_t channels, int64_t inner, int x_dt, int q_dt,
                                int32_t qmin, int32_t qmax, void* stream);

/*
 * Affine dequantization (quantized_decomposed::dequantize_per_tensor /
 * dequantize_per_channel, torch_xla/experimental/quantized.py:25-41).
 *   int_subtract != 0: out = cast(f32(q - zp[c]) * scale[c])            (per-channel form)
 *   int_subtract == 0: out = round(round(cast(q) - zp[c]) * scale[c]),  each result rounded to out's dtype,
 *                      zp and scale entering as f32 scalars            (per-tensor form)
 * zp may be NULL (zero).
 */
int xla_amd_qmm_dequantize_affine(const void* q, void* out, const float* scale, const int32_t* zp,
                                  int64_t outer, int64_t channels, int64_t inner, int q_dt, int out_dt,
                                  int int_subtract, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* XLA_AMD_QMM_H_ */
