// Operator-level entry points of the W8A8 path: per-token activation quantization
// followed by the int8 GEMM, in one call.  The quantized activations (x_q, their
// scales and row sums) are intermediate device memory: the first entry point takes
// it from a caller-provided workspace, the second from a fixed array that lives in
// the library's own device image, for callers that cannot allocate.
#include <mutex>

#include "qmm_common.h"

namespace {

constexpr size_t kAlign = 256;
constexpr size_t round_up(size_t v) { return (v + kAlign - 1) / kAlign * kAlign; }

// Layout of the intermediate memory for an [M, K] activation:
//   x_q     int8  [M, K]   at 0
//   x_scale 4-byte slots [M] (f32, or bf16/f16 in the low half) after it
//   x_sum   int32 [M]      after that
struct Carve {
  size_t xq, scale, sum, total;
};
Carve carve(int64_t M, int64_t K) {
  Carve c;
  c.xq = 0;
  c.scale = round_up((size_t)M * (size_t)K);
  c.sum = c.scale + round_up((size_t)M * 4);
  c.total = c.sum + round_up((size_t)M * 4);
  return c;
}

// Fixed scratch of the no-allocation entry point: 16 MiB of quantized activations
// (M * K <= 16 Mi elements, e.g. 2048 x 8192 or 1024 x 14336) plus the scales and row
// sums of up to 8192 rows.  Every GPU the library runs on holds its own copy of this
// array from the moment the code object is loaded until the process ends.
constexpr size_t kScratchXq = 16u << 20;
constexpr int64_t kScratchRows = 8192;
constexpr size_t kScratchBytes = kScratchXq + 2 * round_up((size_t)kScratchRows * 4);

}  // namespace

// (No device code names the array - kernels get its address as an argument.  What keeps it in the code object
// is the host's reference through HIP_SYMBOL below: the compiler emits a static device variable that host code
// names under a symbol the runtime can look up.  Marking it `used` instead breaks that: the library then aborts
// inside hipGetSymbolAddress.)
static __device__ __align__(256) unsigned char qmm_noalloc_scratch[kScratchBytes];

namespace {

// Device address of this GPU's copy of the scratch array.  The array's name is only a
// host-side handle: the address comes from hipGetSymbolAddress, once per device, with that
// device current, and is what kernels, memsets and copies must be given.
std::mutex g_scratch_mu;
std::atomic<void*> g_scratch_ptr[64] = {};

int scratch_of_current_device(void** out) {
  int dev = -1;
  int rc = qmm_check_hip(hipGetDevice(&dev), "w8a8_linear_noalloc hipGetDevice");
  if (rc != XLA_AMD_QMM_OK) return rc;
  if (dev < 0 || dev >= 64) return qmm_fail(XLA_AMD_QMM_EUNSUPPORTED, "w8a8_linear_noalloc: device ordinal %d out of range", dev);
  // (the steady state is one atomic load; the lock is only taken while a device's address is still unknown)
  void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!p) {
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    p = g_scratch_ptr[dev].load(std::memory_order_relaxed);
    if (!p) {
      rc = qmm_check_hip(hipGetSymbolAddress(&p, HIP_SYMBOL(qmm_noalloc_scratch)), "w8a8_linear_noalloc hipGetSymbolAddress");
      if (rc != XLA_AMD_QMM_OK) return rc;
      if (!p) return qmm_fail(XLA_AMD_QMM_EHIP, "w8a8_linear_noalloc: hipGetSymbolAddress returned a null address");
      g_scratch_ptr[dev].store(p, std::memory_order_release);
    }
  }
  *out = p;
  return XLA_AMD_QMM_OK;
}

int run_linear(const void* x, const int8_t* w, const void* w_scale, const void* zp, void* out,
               unsigned char* mem, const Carve& c, int64_t M, int64_t N, int64_t K, int x_dt,
               int w_scale_dt, int zp_dt, int x_scale_dt, int cvt_dt, int mid_dt, int out_dt,
               int overflow_policy, int block_m, int block_n, void* stream) {
  int8_t* xq = (int8_t*)(mem + c.xq);
  void* xs = mem + c.scale;
  int32_t* xsum = zp ? (int32_t*)(mem + c.sum) : nullptr;
  int rc = xla_amd_qmm_quantize_per_token(x, xq, xs, xsum, M, K, x_dt, x_scale_dt, overflow_policy, stream);
  if (rc != XLA_AMD_QMM_OK) return rc;
  return xla_amd_qmm_w8a8_gemm(xq, w, xs, w_scale, zp, xsum, out, nullptr, M, N, K, x_scale_dt, w_scale_dt,
                               zp_dt, cvt_dt, mid_dt, zp_dt, out_dt, block_m, block_n, stream);
}

int check_common(const char* who, const void* x, const int8_t* w, const void* w_scale, void* out, int64_t M,
                 int64_t N, int64_t K) {
  if (!x || !w || !w_scale || !out) return qmm_fail(XLA_AMD_QMM_EINVAL, "%s: null pointer", who);
  if (M < 0 || N <= 0 || K <= 0) return qmm_fail(XLA_AMD_QMM_EINVAL, "%s: bad sizes M=%lld N=%lld K=%lld", who,
                                                 (long long)M, (long long)N, (long long)K);
  if (M > (1 << 30) || N > (1 << 30) || K > (1 << 30)) return qmm_fail(XLA_AMD_QMM_EUNSUPPORTED, "%s: dimension too large", who);
  return XLA_AMD_QMM_OK;
}

}  // namespace

extern "C" size_t xla_amd_qmm_w8a8_linear_workspace_bytes(int64_t M, int64_t N, int64_t K) {
  (void)N;
  if (M < 0 || K <= 0) return 0;
  return carve(M, K).total;
}

extern "C" int xla_amd_qmm_w8a8_linear(const void* x, const int8_t* w, const void* w_scale, const void* zp,
                                       void* out, void* workspace, size_t workspace_bytes, int64_t M, int64_t N,
                                       int64_t K, int x_dt, int w_scale_dt, int zp_dt, int x_scale_dt,
                                       int cvt_dt, int mid_dt, int out_dt, int overflow_policy, int block_m,
                                       int block_n, void* stream) {
  int rc = check_common("w8a8_linear", x, w, w_scale, out, M, N, K);
  if (rc != XLA_AMD_QMM_OK) return rc;
  if (M == 0) return XLA_AMD_QMM_OK;
  const Carve c = carve(M, K);
  if (!workspace || workspace_bytes < c.total)
    return qmm_fail(XLA_AMD_QMM_EINVAL, "w8a8_linear: workspace of %zu bytes, need %zu", workspace ? workspace_bytes : (size_t)0, c.total);
  if ((uintptr_t)workspace & (kAlign - 1)) return qmm_fail(XLA_AMD_QMM_EINVAL, "w8a8_linear: workspace must be 256-byte aligned");
  return run_linear(x, w, w_scale, zp, out, (unsigned char*)workspace, c, M, N, K, x_dt, w_scale_dt, zp_dt,
                    x_scale_dt, cvt_dt, mid_dt, out_dt, overflow_policy, block_m, block_n, stream);
}

extern "C" int xla_amd_qmm_init(void) {
  void* base = nullptr;
  return scratch_of_current_device(&base);
}

extern "C" void xla_amd_qmm_w8a8_linear_noalloc_limits(int64_t* max_rows, int64_t* max_elements) {
  if (max_rows) *max_rows = kScratchRows;
  if (max_elements) *max_elements = (int64_t)kScratchXq;
}

extern "C" int xla_amd_qmm_w8a8_linear_noalloc(const void* x, const int8_t* w, const void* w_scale, const void* zp,
                                               void* out, int64_t M, int64_t N, int64_t K, int x_dt,
                                               int w_scale_dt, int zp_dt, int x_scale_dt, int cvt_dt, int mid_dt,
                                               int out_dt, int overflow_policy, int block_m, int block_n,
                                               void* stream) {
  int rc = check_common("w8a8_linear_noalloc", x, w, w_scale, out, M, N, K);
  if (rc != XLA_AMD_QMM_OK) return rc;
  if (M > kScratchRows || (size_t)M * (size_t)K > kScratchXq)
    return qmm_fail(XLA_AMD_QMM_EUNSUPPORTED,
                    "w8a8_linear_noalloc: activation of %lld x %lld exceeds the fixed scratch (at most %lld rows and %zu elements); "
                    "use xla_amd_qmm_w8a8_linear with a workspace",
                    (long long)M, (long long)K, (long long)kScratchRows, kScratchXq);
  if (M == 0) return XLA_AMD_QMM_OK;
  void* base = nullptr;
  rc = scratch_of_current_device(&base);
  if (rc != XLA_AMD_QMM_OK) return rc;
  // Same carving as the workspace variant, but with the fixed offsets of the largest case, so that
  // the three regions never depend on the call's shape.
  Carve c;
  c.xq = 0;
  c.scale = kScratchXq;
  c.sum = kScratchXq + round_up((size_t)kScratchRows * 4);
  c.total = kScratchBytes;
  return run_linear(x, w, w_scale, zp, out, (unsigned char*)base, c, M, N, K, x_dt, w_scale_dt, zp_dt, x_scale_dt,
                    cvt_dt, mid_dt, out_dt, overflow_policy, block_m, block_n, stream);
}
