// The C ABI of libaxn_gfx950.so (declared in axn.h): argument validation and
// dispatch only.  Validation runs before any HIP call so that bad arguments are
// reported the same way on a host without a GPU.
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>

#include "axn_internal.h"

namespace axn {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

int hip_fail(hipError_t e, const char* what) {
  set_error("HIP error %d (%s) in %s", (int)e, hipGetErrorString(e), what);
  return AXN_EHIP;
}

namespace {

bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

#define REQUIRE(cond, code, ...)   \
  do {                             \
    if (!(cond)) {                 \
      set_error(__VA_ARGS__);      \
      return (code);               \
    }                              \
  } while (0)

int check_gemm(const char* name, const void* a, const void* b, const void* c,
               int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb,
               int64_t ldc, int64_t min_lda, int64_t min_ldb, int64_t min_ldc) {
  REQUIRE(a && b && c, AXN_EINVAL, "%s: null operand pointer", name);
  REQUIRE(M >= 1 && N >= 1 && K >= 1, AXN_EINVAL,
          "%s: M, N, K must be >= 1 (got %lld, %lld, %lld)", name, (long long)M,
          (long long)N, (long long)K);
  REQUIRE(M <= 0x7fffffff && N <= 0x7fffffff && K <= 0x7fffffff, AXN_ELIMIT,
          "%s: dimension exceeds 2^31-1", name);
  REQUIRE(N % 8 == 0 && K % 8 == 0, AXN_ESHAPE,
          "%s: N and K must be multiples of 8 (got N=%lld, K=%lld)", name,
          (long long)N, (long long)K);
  REQUIRE(lda >= min_lda && ldb >= min_ldb && ldc >= min_ldc, AXN_EINVAL,
          "%s: leading dimension smaller than the row length", name);
  REQUIRE(lda % 8 == 0 && ldb % 8 == 0 && ldc % 8 == 0, AXN_EALIGN,
          "%s: leading dimensions must be multiples of 8", name);
  REQUIRE(aligned16(a) && aligned16(b) && aligned16(c), AXN_EALIGN,
          "%s: operand pointers must be 16-byte aligned", name);
  return AXN_OK;
}

int check_epilogue(const char* name, int epilogue, const float* bias) {
  REQUIRE(epilogue >= AXN_EPI_NONE && epilogue <= AXN_EPI_GELU, AXN_EINVAL,
          "%s: unknown epilogue %d", name, epilogue);
  const bool needs_bias = epilogue == AXN_EPI_BIAS || epilogue == AXN_EPI_BIAS_GELU;
  REQUIRE(!needs_bias || bias != nullptr, AXN_EINVAL,
          "%s: epilogue %d needs a bias vector", name, epilogue);
  REQUIRE(!needs_bias || aligned16(bias), AXN_EALIGN,
          "%s: bias must be 16-byte aligned", name);
  return AXN_OK;
}

int check_f32(const char* name, const void* a, const void* b, const void* c,
              int64_t M, int64_t N, int64_t K) {
  REQUIRE(a && b && c, AXN_EINVAL, "%s: null operand pointer", name);
  REQUIRE(M >= 1 && N >= 1 && K >= 1, AXN_EINVAL,
          "%s: M, N, K must be >= 1 (got %lld, %lld, %lld)", name, (long long)M,
          (long long)N, (long long)K);
  REQUIRE(M <= 0x7fffffff && N <= 0x7fffffff && K <= 0x7fffffff, AXN_ELIMIT,
          "%s: dimension exceeds 2^31-1", name);
  REQUIRE((((uintptr_t)a | (uintptr_t)b | (uintptr_t)c) & 3u) == 0, AXN_EALIGN,
          "%s: operand pointers must be 4-byte aligned", name);
  return AXN_OK;
}

bool known_dtype(int dt) { return dt == AXN_BF16 || dt == AXN_F16 || dt == AXN_F32; }

int check_list(const char* name, const void* const* h_ptrs, const char* what,
               const int64_t* h_sizes, int64_t n, int elem_size) {
  for (int64_t i = 0; i < n; ++i) {
    if (h_sizes[i] == 0) continue;
    REQUIRE(h_ptrs[i] != nullptr, AXN_EINVAL, "%s: %s[%lld] is null", name, what,
            (long long)i);
    REQUIRE(((uintptr_t)h_ptrs[i] % (uintptr_t)elem_size) == 0, AXN_EALIGN,
            "%s: %s[%lld] is not aligned to its element size", name, what,
            (long long)i);
  }
  return AXN_OK;
}

int check_sizes(const char* name, const int64_t* h_sizes, int64_t n) {
  REQUIRE(n >= 0, AXN_EINVAL, "%s: negative tensor count", name);
  REQUIRE(n == 0 || h_sizes != nullptr, AXN_EINVAL, "%s: null size array", name);
  for (int64_t i = 0; i < n; ++i)
    REQUIRE(h_sizes[i] >= 0, AXN_EINVAL, "%s: sizes[%lld] is negative", name,
            (long long)i);
  return AXN_OK;
}

}  // namespace
}  // namespace axn

using namespace axn;

extern "C" {

int axn_abi_version(void) { return AXN_ABI_VERSION; }

const char* axn_last_error(void) { return g_err; }

// The 16-bit GEMM entry points: `half` selects IEEE half instead of bfloat16.
static int gemm_fwd_16(const char* name, bool half, const void* X, const void* W,
                       const float* bias, void* Y, void* Zsave, int64_t M, int64_t N, int64_t K,
                       int64_t ldx, int64_t ldw, int64_t ldy, int epilogue, void* stream,
                       bool y_f32 = false) {
  int rc = check_gemm(name, X, W, Y, M, N, K, ldx, ldw, ldy, K, K, N);
  if (rc) return rc;
  rc = check_epilogue(name, epilogue, bias);
  if (rc) return rc;
  REQUIRE(!y_f32 || epilogue == AXN_EPI_BIAS || epilogue == AXN_EPI_BIAS_GELU, AXN_EINVAL,
          "%s: an fp32 result is the promotion of an fp32 bias: epilogue must be BIAS or BIAS_GELU",
          name);
  REQUIRE(Zsave == nullptr || aligned16(Zsave), AXN_EALIGN, "%s: Zsave must be 16-byte aligned",
          name);
  GemmArgs g = {};
  g.A = (const uint16_t*)X;
  g.B = (const uint16_t*)W;
  g.C = Y;
  g.bias = bias;
  g.Z = (uint16_t*)Zsave;
  g.M = (int)M;
  g.N = (int)N;
  g.Kc = (int)K;
  g.lda = ldx;
  g.ldb = ldw;
  g.ldc = ldy;
  g.beta = 0;
  return half ? launch_gemm_f16(GEMM_NT, g, epilogue, y_f32, (hipStream_t)stream)
              : launch_gemm_bf16(GEMM_NT, g, epilogue, y_f32, (hipStream_t)stream);
}

static int gemm_dgrad_16(const char* name, bool half, const void* dY, const void* W, void* dX,
                         int64_t M, int64_t N, int64_t K, int64_t lddy, int64_t ldw,
                         int64_t lddx, void* stream) {
  int rc = check_gemm(name, dY, W, dX, M, N, K, lddy, ldw, lddx, N, K, K);
  if (rc) return rc;
  GemmArgs g = {};
  g.A = (const uint16_t*)dY;  // [M][N]: rows of the output, contraction contiguous
  g.B = (const uint16_t*)W;   // [N][K]: contraction-major
  g.C = dX;
  g.M = (int)M;
  g.N = (int)K;
  g.Kc = (int)N;
  g.lda = lddy;
  g.ldb = ldw;
  g.ldc = lddx;
  g.beta = 0;
  return half ? launch_gemm_f16(GEMM_NN, g, AXN_EPI_NONE, false, (hipStream_t)stream)
              : launch_gemm_bf16(GEMM_NN, g, AXN_EPI_NONE, false, (hipStream_t)stream);
}

static int gemm_wgrad_16(const char* name, bool half, const void* dY, const void* X, void* dW,
                         int64_t M, int64_t N, int64_t K, int64_t lddy, int64_t ldx,
                         int64_t lddw, int beta, int dw_dtype, void* stream) {
  int rc = check_gemm(name, dY, X, dW, M, N, K, lddy, ldx, lddw, N, K, K);
  if (rc) return rc;
  REQUIRE(beta == 0 || beta == 1, AXN_EINVAL, "%s: beta must be 0 or 1", name);
  REQUIRE(dw_dtype == (half ? AXN_F16 : AXN_BF16) || dw_dtype == AXN_F32, AXN_EINVAL,
          "%s: dW must be %s or fp32", name, half ? "fp16" : "bf16");
  GemmArgs g = {};
  g.A = (const uint16_t*)dY;  // [M][N]: contraction-major, output rows = N
  g.B = (const uint16_t*)X;   // [M][K]: contraction-major, output cols = K
  g.C = dW;
  g.M = (int)N;
  g.N = (int)K;
  g.Kc = (int)M;
  g.lda = lddy;
  g.ldb = ldx;
  g.ldc = lddw;
  g.beta = beta;
  return half ? launch_gemm_f16(GEMM_TN, g, AXN_EPI_NONE, dw_dtype == AXN_F32,
                                (hipStream_t)stream)
              : launch_gemm_bf16(GEMM_TN, g, AXN_EPI_NONE, dw_dtype == AXN_F32,
                                 (hipStream_t)stream);
}

int axn_gemm_fwd(const void* X, const void* W, const float* bias, void* Y,
                 void* Zsave, int64_t M, int64_t N, int64_t K, int64_t ldx,
                 int64_t ldw, int64_t ldy, int epilogue, void* stream) {
  return gemm_fwd_16("axn_gemm_fwd", false, X, W, bias, Y, Zsave, M, N, K, ldx, ldw, ldy,
                     epilogue, stream);
}

int axn_gemm_fwd_f32out(const void* X, const void* W, const float* bias, float* Y, void* Zsave,
                        int dtype, int64_t M, int64_t N, int64_t K, int64_t ldx, int64_t ldw,
                        int64_t ldy, int epilogue, void* stream) {
  const char* name = "axn_gemm_fwd_f32out";
  REQUIRE(dtype == AXN_BF16 || dtype == AXN_F16, AXN_EINVAL, "%s: dtype must be bf16 or fp16", name);
  return gemm_fwd_16(name, dtype == AXN_F16, X, W, bias, Y, Zsave, M, N, K, ldx, ldw, ldy, epilogue,
                     stream, true);
}

int axn_gemm_dgrad(const void* dY, const void* W, void* dX, int64_t M, int64_t N,
                   int64_t K, int64_t lddy, int64_t ldw, int64_t lddx,
                   void* stream) {
  return gemm_dgrad_16("axn_gemm_dgrad", false, dY, W, dX, M, N, K, lddy, ldw, lddx, stream);
}

int axn_gemm_wgrad(const void* dY, const void* X, void* dW, int64_t M, int64_t N,
                   int64_t K, int64_t lddy, int64_t ldx, int64_t lddw, int beta,
                   int dw_dtype, void* stream) {
  return gemm_wgrad_16("axn_gemm_wgrad", false, dY, X, dW, M, N, K, lddy, ldx, lddw, beta,
                       dw_dtype, stream);
}

int axn_gemm_fwd_f16(const void* X, const void* W, const float* bias, void* Y,
                     void* Zsave, int64_t M, int64_t N, int64_t K, int64_t ldx,
                     int64_t ldw, int64_t ldy, int epilogue, void* stream) {
  return gemm_fwd_16("axn_gemm_fwd_f16", true, X, W, bias, Y, Zsave, M, N, K, ldx, ldw, ldy,
                     epilogue, stream);
}

int axn_gemm_dgrad_f16(const void* dY, const void* W, void* dX, int64_t M, int64_t N,
                       int64_t K, int64_t lddy, int64_t ldw, int64_t lddx, void* stream) {
  return gemm_dgrad_16("axn_gemm_dgrad_f16", true, dY, W, dX, M, N, K, lddy, ldw, lddx, stream);
}

int axn_gemm_wgrad_f16(const void* dY, const void* X, void* dW, int64_t M, int64_t N,
                       int64_t K, int64_t lddy, int64_t ldx, int64_t lddw, int beta,
                       int dw_dtype, void* stream) {
  return gemm_wgrad_16("axn_gemm_wgrad_f16", true, dY, X, dW, M, N, K, lddy, ldx, lddw, beta,
                       dw_dtype, stream);
}

int axn_gemm_bwd(const void* dY, const void* W, const void* X, void* dX, void* dW, int dtype,
                 int64_t M, int64_t N, int64_t K, int64_t lddy, int64_t ldw, int64_t ldx,
                 int64_t lddx, int64_t lddw, int beta, int dw_dtype, void* stream) {
  const char* name = "axn_gemm_bwd";
  REQUIRE(dtype == AXN_BF16 || dtype == AXN_F16, AXN_EINVAL, "%s: dtype must be bf16 or fp16", name);
  const bool half = dtype == AXN_F16;
  int rc = check_gemm(name, dY, W, dX, M, N, K, lddy, ldw, lddx, N, K, K);
  if (rc) return rc;
  rc = check_gemm(name, dY, X, dW, M, N, K, lddy, ldx, lddw, N, K, K);
  if (rc) return rc;
  REQUIRE(beta == 0 || beta == 1, AXN_EINVAL, "%s: beta must be 0 or 1", name);
  REQUIRE(dw_dtype == dtype || dw_dtype == AXN_F32, AXN_EINVAL, "%s: dW must be %s or fp32", name,
          half ? "fp16" : "bf16");
  GemmArgs gd = {}, gw = {};
  gd.A = (const uint16_t*)dY;
  gd.B = (const uint16_t*)W;
  gd.C = dX;
  gd.M = (int)M, gd.N = (int)K, gd.Kc = (int)N;
  gd.lda = lddy, gd.ldb = ldw, gd.ldc = lddx;
  gw.A = (const uint16_t*)dY;
  gw.B = (const uint16_t*)X;
  gw.C = dW;
  gw.M = (int)N, gw.N = (int)K, gw.Kc = (int)M;
  gw.lda = lddy, gw.ldb = ldx, gw.ldc = lddw;
  gw.beta = beta;
  return launch_gemm_backward(gd, gw, half, dw_dtype == AXN_F32, (hipStream_t)stream);
}

// ---- split-contraction variants --------------------------------------------------
static void fill_gemm_args(GemmArgs& g, int op, const void* a, const void* b, void* c, int64_t M,
                           int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc) {
  g.A = (const uint16_t*)a;
  g.B = (const uint16_t*)b;
  g.C = c;
  g.lda = lda;
  g.ldb = ldb;
  g.ldc = ldc;
  if (op == AXN_GEMM_FWD) {  // Y[M,N] = X[M,K] W[N,K]^T
    g.M = (int)M, g.N = (int)N, g.Kc = (int)K;
  } else if (op == AXN_GEMM_DGRAD) {  // dX[M,K] = dY[M,N] W[N,K]
    g.M = (int)M, g.N = (int)K, g.Kc = (int)N;
  } else {  // dW[N,K] = dY[M,N]^T X[M,K]
    g.M = (int)N, g.N = (int)K, g.Kc = (int)M;
  }
}

static const GemmLayout kLayoutOfOp[3] = {GEMM_NT, GEMM_NN, GEMM_TN};

size_t axn_gemm_workspace_bytes(int op, int64_t M, int64_t N, int64_t K) {
  if (op < AXN_GEMM_FWD || op > AXN_GEMM_WGRAD || M < 1 || N < 1 || K < 1 || M > 0x7fffffff ||
      N > 0x7fffffff || K > 0x7fffffff)
    return 0;
  GemmArgs g = {};
  // dense operands: the leading dimensions are the row lengths
  fill_gemm_args(g, op, nullptr, nullptr, nullptr, M, N, K, op == AXN_GEMM_FWD ? K : N, K,
                 op == AXN_GEMM_FWD ? N : K);
  const int s = gemm_splits(kLayoutOfOp[op], g);
  return s > 1 ? (size_t)s * (size_t)g.M * (size_t)g.N * sizeof(float) : 0;
}

static int gemm_ws(const char* name, int op, const void* a, const void* b, void* c, int dtype,
                   int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc, int beta,
                   int out_dtype, void* workspace, size_t workspace_bytes, void* stream,
                   const float* bias = nullptr, void* zsave = nullptr, int epilogue = AXN_EPI_NONE) {
  REQUIRE(dtype == AXN_BF16 || dtype == AXN_F16, AXN_EINVAL, "%s: dtype must be bf16 or fp16", name);
  const bool half = dtype == AXN_F16;
  int rc;
  if (op == AXN_GEMM_FWD)
    rc = check_gemm(name, a, b, c, M, N, K, lda, ldb, ldc, K, K, N);
  else
    rc = check_gemm(name, a, b, c, M, N, K, lda, ldb, ldc, N, K, K);
  if (rc) return rc;
  REQUIRE(beta == 0 || beta == 1, AXN_EINVAL, "%s: beta must be 0 or 1", name);
  REQUIRE(out_dtype == dtype || (op == AXN_GEMM_WGRAD && out_dtype == AXN_F32), AXN_EINVAL,
          "%s: unsupported output type", name);
  GemmArgs g = {};
  fill_gemm_args(g, op, a, b, c, M, N, K, lda, ldb, ldc);
  g.beta = beta;
  g.bias = bias;
  g.Z = (uint16_t*)zsave;
  const GemmLayout layout = kLayoutOfOp[op];
  bool wide_tiles = false;
  const int splits =
      (workspace != nullptr && epilogue == AXN_EPI_NONE) ? gemm_splits(layout, g, &wide_tiles) : 1;
  if (splits > 1) {
    const size_t need = (size_t)splits * (size_t)g.M * (size_t)g.N * sizeof(float);
    REQUIRE(workspace_bytes >= need, AXN_EINVAL,
            "%s: workspace too small (%zu bytes given, %zu needed)", name, workspace_bytes, need);
    REQUIRE(aligned16(workspace), AXN_EALIGN, "%s: workspace must be 16-byte aligned", name);
    return launch_gemm_splitk(layout, g, half, out_dtype, splits, wide_tiles, (float*)workspace,
                              (hipStream_t)stream);
  }
  return half ? launch_gemm_f16(layout, g, epilogue, out_dtype == AXN_F32, (hipStream_t)stream)
              : launch_gemm_bf16(layout, g, epilogue, out_dtype == AXN_F32, (hipStream_t)stream);
}

int axn_gemm_fwd_ws(const void* X, const void* W, const float* bias, void* Y, void* Zsave, int dtype,
                    int64_t M, int64_t N, int64_t K, int64_t ldx, int64_t ldw, int64_t ldy,
                    int epilogue, void* workspace, size_t workspace_bytes, void* stream) {
  const char* name = "axn_gemm_fwd_ws";
  int rc = check_epilogue(name, epilogue, bias);
  if (rc) return rc;
  REQUIRE(Zsave == nullptr || aligned16(Zsave), AXN_EALIGN, "%s: Zsave must be 16-byte aligned",
          name);
  return gemm_ws(name, AXN_GEMM_FWD, X, W, Y, dtype, M, N, K, ldx, ldw, ldy, 0, dtype, workspace,
                 workspace_bytes, stream, bias, Zsave, epilogue);
}

int axn_gemm_dgrad_ws(const void* dY, const void* W, void* dX, int dtype, int64_t M, int64_t N,
                      int64_t K, int64_t lddy, int64_t ldw, int64_t lddx, void* workspace,
                      size_t workspace_bytes, void* stream) {
  return gemm_ws("axn_gemm_dgrad_ws", AXN_GEMM_DGRAD, dY, W, dX, dtype, M, N, K, lddy, ldw, lddx, 0,
                 dtype, workspace, workspace_bytes, stream);
}

int axn_gemm_wgrad_ws(const void* dY, const void* X, void* dW, int dtype, int64_t M, int64_t N,
                      int64_t K, int64_t lddy, int64_t ldx, int64_t lddw, int beta, int dw_dtype,
                      void* workspace, size_t workspace_bytes, void* stream) {
  return gemm_ws("axn_gemm_wgrad_ws", AXN_GEMM_WGRAD, dY, X, dW, dtype, M, N, K, lddy, ldx, lddw,
                 beta, dw_dtype, workspace, workspace_bytes, stream);
}

int axn_gemm_swiglu_fwd(const void* X, const void* Wg, const void* Wu, void* H, void* gate_save,
                        void* up_save, int dtype, int64_t M, int64_t N, int64_t K, int64_t ldx,
                        int64_t ldw, int64_t ldh, void* stream) {
  const char* name = "axn_gemm_swiglu_fwd";
  REQUIRE(dtype == AXN_BF16 || dtype == AXN_F16, AXN_EINVAL, "%s: dtype must be bf16 or fp16", name);
  int rc = check_gemm(name, X, Wg, H, M, N, K, ldx, ldw, ldh, K, K, N);
  if (rc) return rc;
  REQUIRE(Wu != nullptr, AXN_EINVAL, "%s: null operand pointer", name);
  REQUIRE(aligned16(Wu) && aligned16(gate_save) && aligned16(up_save), AXN_EALIGN,
          "%s: operand pointers must be 16-byte aligned", name);
  GemmArgs g = {};
  g.A = (const uint16_t*)X;
  g.B = (const uint16_t*)Wg;
  g.B2 = (const uint16_t*)Wu;
  g.C = H;
  g.G = (uint16_t*)gate_save;
  g.U = (uint16_t*)up_save;
  g.M = (int)M;
  g.N = (int)N;
  g.Kc = (int)K;
  g.lda = ldx;
  g.ldb = ldw;
  g.ldc = ldh;
  return launch_gemm_swiglu(g, dtype == AXN_F16, (hipStream_t)stream);
}

int axn_gemm_dgrad_pair(const void* dY1, const void* W1, const void* dY2, const void* W2, void* dX,
                        int dtype, int64_t M, int64_t N1, int64_t N2, int64_t K, int64_t lddy,
                        int64_t ldw, int64_t lddx, void* stream) {
  const char* name = "axn_gemm_dgrad_pair";
  REQUIRE(dtype == AXN_BF16 || dtype == AXN_F16, AXN_EINVAL, "%s: dtype must be bf16 or fp16", name);
  REQUIRE(N1 >= 1 && N2 >= 1 && N1 <= 0x7fffffff - N2, AXN_EINVAL, "%s: N1 and N2 must be >= 1", name);
  int rc = check_gemm(name, dY1, W1, dX, M, N1, K, lddy, ldw, lddx, N1 > N2 ? N1 : N2, K, K);
  if (rc) return rc;
  REQUIRE(N2 % 8 == 0, AXN_ESHAPE, "%s: N and K must be multiples of 8 (got N=%lld)", name,
          (long long)N2);
  REQUIRE(dY2 != nullptr && W2 != nullptr, AXN_EINVAL, "%s: null operand pointer", name);
  REQUIRE(aligned16(dY2) && aligned16(W2), AXN_EALIGN, "%s: operand pointers must be 16-byte aligned",
          name);
  GemmArgs g = {};
  g.A = (const uint16_t*)dY1;
  g.B = (const uint16_t*)W1;
  g.A2 = (const uint16_t*)dY2;
  g.B2 = (const uint16_t*)W2;
  g.C = dX;
  g.M = (int)M;
  g.N = (int)K;
  g.Kc = (int)(N1 + N2);
  g.k_first = (int)N1;
  g.lda = lddy;
  g.ldb = ldw;
  g.ldc = lddx;
  return launch_gemm_pair(g, dtype == AXN_F16, (hipStream_t)stream);
}

size_t axn_dgelu_dbias_workspace_bytes(int64_t M, int64_t N) {
  return dgelu_dbias_workspace_bytes(M, N);
}

int axn_dgelu_dbias(const void* dY, const void* Z, void* dZ, int dtype,
                    float* dbias, int64_t M, int64_t N, int64_t ld, int beta,
                    void* workspace, size_t workspace_bytes, void* stream) {
  const char* name = "axn_dgelu_dbias";
  REQUIRE(dY != nullptr, AXN_EINVAL, "%s: dY is null", name);
  REQUIRE(dtype == AXN_BF16 || dtype == AXN_F16 || dtype == AXN_F32, AXN_EINVAL,
          "%s: unknown dtype %d", name, dtype);
  REQUIRE(M >= 1 && N >= 1, AXN_EINVAL, "%s: M and N must be >= 1", name);
  REQUIRE(N % 8 == 0, AXN_ESHAPE, "%s: N must be a multiple of 8", name);
  REQUIRE(ld >= N && ld % 8 == 0, AXN_EALIGN,
          "%s: ld must be >= N and a multiple of 8", name);
  REQUIRE((Z == nullptr) == (dZ == nullptr), AXN_EINVAL,
          "%s: Z and dZ must be given together", name);
  REQUIRE(Z != nullptr || dbias != nullptr, AXN_EINVAL, "%s: nothing to compute", name);
  REQUIRE(aligned16(dY) && aligned16(Z) && aligned16(dZ), AXN_EALIGN,
          "%s: pointers must be 16-byte aligned", name);
  REQUIRE(beta == 0 || beta == 1, AXN_EINVAL, "%s: beta must be 0 or 1", name);
  return launch_dgelu_dbias(dY, Z, dZ, dtype, dbias, M, N, ld, beta, workspace,
                            workspace_bytes, (hipStream_t)stream);
}

static int check_swiglu(const char* name, int dtype, int64_t M, int64_t N, int64_t ld) {
  REQUIRE(dtype == AXN_BF16 || dtype == AXN_F16 || dtype == AXN_F32, AXN_EINVAL,
          "%s: unknown dtype %d", name, dtype);
  REQUIRE(M >= 1 && N >= 1, AXN_EINVAL, "%s: M and N must be >= 1", name);
  REQUIRE(N % 8 == 0, AXN_ESHAPE, "%s: N must be a multiple of 8", name);
  REQUIRE(ld >= N && ld % 8 == 0, AXN_EALIGN, "%s: ld must be >= N and a multiple of 8", name);
  return AXN_OK;
}

int axn_swiglu_fwd(const void* gate, const void* up, void* out, int dtype, int64_t M,
                   int64_t N, int64_t ld, void* stream) {
  const char* name = "axn_swiglu_fwd";
  REQUIRE(gate && up && out, AXN_EINVAL, "%s: null pointer", name);
  int rc = check_swiglu(name, dtype, M, N, ld);
  if (rc) return rc;
  REQUIRE(aligned16(gate) && aligned16(up) && aligned16(out), AXN_EALIGN,
          "%s: pointers must be 16-byte aligned", name);
  return launch_swiglu_fwd(gate, up, out, dtype, M, N, ld, (hipStream_t)stream);
}

int axn_swiglu_bwd(const void* dout, const void* gate, const void* up, void* dgate,
                   void* dup, int dtype, int64_t M, int64_t N, int64_t ld, void* stream) {
  const char* name = "axn_swiglu_bwd";
  REQUIRE(dout && gate && up && dgate && dup, AXN_EINVAL, "%s: null pointer", name);
  int rc = check_swiglu(name, dtype, M, N, ld);
  if (rc) return rc;
  REQUIRE(aligned16(dout) && aligned16(gate) && aligned16(up) && aligned16(dgate) && aligned16(dup),
          AXN_EALIGN, "%s: pointers must be 16-byte aligned", name);
  return launch_swiglu_bwd(dout, gate, up, dgate, dup, dtype, M, N, ld, ld, (hipStream_t)stream);
}

static int elem_bytes_of(int dtype) { return dtype == AXN_F32 ? 4 : 2; }

static int check_embedding(const char* name, int64_t T, int64_t V, int64_t H) {
  REQUIRE(T >= 0 && V >= 1 && H >= 1, AXN_EINVAL, "%s: T must be >= 0, V and H >= 1", name);
  REQUIRE(T < (1LL << 31) && V < (1LL << 31) - 1, AXN_ELIMIT,
          "%s: T and V must be below 2^31", name);
  return AXN_OK;
}

static int check_rows16(const char* name, const char* what, int dtype, int64_t H, int64_t ld) {
  const int per = 16 / elem_bytes_of(dtype);
  REQUIRE(H % per == 0, AXN_ESHAPE, "%s: H must be a multiple of %d for %s", name, per, what);
  REQUIRE(ld >= H && ld % per == 0, AXN_EALIGN, "%s: ld of %s must be >= H and a multiple of %d",
          name, what, per);
  return AXN_OK;
}

int axn_embedding_fwd(const int64_t* ids, const void* W, void* out, int dtype, int64_t T,
                      int64_t V, int64_t H, int64_t ldw, int64_t ldo, int32_t* status,
                      void* stream) {
  const char* name = "axn_embedding_fwd";
  REQUIRE(W && ((ids && out) || T == 0), AXN_EINVAL, "%s: null pointer", name);
  REQUIRE(dtype == AXN_BF16 || dtype == AXN_F16 || dtype == AXN_F32, AXN_EINVAL,
          "%s: unknown dtype %d", name, dtype);
  int rc = check_embedding(name, T, V, H);
  if (rc) return rc;
  if ((rc = check_rows16(name, "W", dtype, H, ldw))) return rc;
  if ((rc = check_rows16(name, "out", dtype, H, ldo))) return rc;
  REQUIRE(aligned16(W) && aligned16(out), AXN_EALIGN, "%s: pointers must be 16-byte aligned", name);
  if (T == 0) return AXN_OK;
  return launch_embedding_fwd(ids, W, out, elem_bytes_of(dtype), T, V, H, ldw, ldo, (int*)status,
                              (hipStream_t)stream);
}

size_t axn_embedding_workspace_bytes(int64_t T, int64_t V) {
  return embedding_workspace_bytes(T, V);
}

int axn_embedding_bwd(const int64_t* ids, const void* dY, void* dW, int dy_dtype, int dw_dtype,
                      int64_t T, int64_t V, int64_t H, int64_t lddy, int64_t lddw,
                      int64_t padding_idx, int scale_grad_by_freq, int beta, void* workspace,
                      size_t workspace_bytes, void* stream) {
  const char* name = "axn_embedding_bwd";
  REQUIRE(dW && ((ids && dY) || T == 0), AXN_EINVAL, "%s: null pointer", name);
  REQUIRE((dy_dtype == AXN_BF16 || dy_dtype == AXN_F32) &&
              (dw_dtype == AXN_BF16 || dw_dtype == AXN_F32),
          AXN_EINVAL, "%s: dtypes must be bf16 or fp32", name);
  int rc = check_embedding(name, T, V, H);
  if (rc) return rc;
  if ((rc = check_rows16(name, "dY", dy_dtype, H, lddy))) return rc;
  if ((rc = check_rows16(name, "dW", dw_dtype, H, lddw))) return rc;
  REQUIRE(padding_idx >= -1 && padding_idx < V, AXN_EINVAL,
          "%s: padding_idx must be -1 or a row of the table", name);
  REQUIRE(beta == 0 || beta == 1, AXN_EINVAL, "%s: beta must be 0 or 1", name);
  REQUIRE((T == 0 || aligned16(dY)) && aligned16(dW), AXN_EALIGN,
          "%s: pointers must be 16-byte aligned", name);
  REQUIRE(workspace != nullptr && workspace_bytes >= embedding_workspace_bytes(T, V), AXN_EINVAL,
          "%s: workspace too small (%zu bytes given, %zu needed)", name, workspace_bytes,
          embedding_workspace_bytes(T, V));
  REQUIRE(aligned16(workspace), AXN_EALIGN, "%s: workspace must be 16-byte aligned", name);
  return launch_embedding_bwd(ids, dY, dW, dy_dtype, dw_dtype, T, V, H, lddy, lddw, padding_idx,
                              scale_grad_by_freq != 0, beta, workspace, workspace_bytes,
                              (hipStream_t)stream);
}

int axn_embedding_renorm(const int64_t* ids, void* W, int dtype, int64_t T, int64_t V, int64_t H,
                         int64_t ldw, float max_norm, float norm_type, void* workspace,
                         size_t workspace_bytes, void* stream) {
  const char* name = "axn_embedding_renorm";
  REQUIRE(W && (ids || T == 0), AXN_EINVAL, "%s: null pointer", name);
  REQUIRE(known_dtype(dtype), AXN_EINVAL, "%s: dtype must be bf16, fp16 or fp32",
          name);
  int rc = check_embedding(name, T, V, H);
  if (rc) return rc;
  if ((rc = check_rows16(name, "W", dtype, H, ldw))) return rc;
  REQUIRE(max_norm > 0.0f && norm_type > 0.0f, AXN_EINVAL,
          "%s: max_norm and norm_type must be positive", name);
  REQUIRE(aligned16(W), AXN_EALIGN, "%s: pointers must be 16-byte aligned", name);
  REQUIRE(workspace != nullptr && workspace_bytes >= embedding_workspace_bytes(T, V), AXN_EINVAL,
          "%s: workspace too small (%zu bytes given, %zu needed)", name, workspace_bytes,
          embedding_workspace_bytes(T, V));
  REQUIRE(aligned16(workspace), AXN_EALIGN, "%s: workspace must be 16-byte aligned", name);
  if (T == 0) return AXN_OK;
  return launch_embedding_renorm(ids, W, dtype, T, V, H, ldw, max_norm, norm_type, workspace,
                                 workspace_bytes, (hipStream_t)stream);
}

int axn_gemm_fwd_f32(const float* X, const float* W, const float* bias, float* Y,
                     float* Zsave, int64_t M, int64_t N, int64_t K, int epilogue,
                     void* stream) {
  int rc = check_f32("axn_gemm_fwd_f32", X, W, Y, M, N, K);
  if (rc) return rc;
  REQUIRE(epilogue >= AXN_EPI_NONE && epilogue <= AXN_EPI_GELU, AXN_EINVAL,
          "axn_gemm_fwd_f32: unknown epilogue %d", epilogue);
  const bool needs_bias = epilogue == AXN_EPI_BIAS || epilogue == AXN_EPI_BIAS_GELU;
  REQUIRE(!needs_bias || bias != nullptr, AXN_EINVAL,
          "axn_gemm_fwd_f32: epilogue %d needs a bias vector", epilogue);
  return launch_gemm_f32(GEMM_NT, X, W, Y, bias, Zsave, (int)M, (int)N, (int)K,
                         epilogue, 0, (hipStream_t)stream);
}

int axn_gemm_dgrad_f32(const float* dY, const float* W, float* dX, int64_t M,
                       int64_t N, int64_t K, void* stream) {
  int rc = check_f32("axn_gemm_dgrad_f32", dY, W, dX, M, N, K);
  if (rc) return rc;
  return launch_gemm_f32(GEMM_NN, dY, W, dX, nullptr, nullptr, (int)M, (int)K,
                         (int)N, AXN_EPI_NONE, 0, (hipStream_t)stream);
}

int axn_gemm_wgrad_f32(const float* dY, const float* X, float* dW, int64_t M,
                       int64_t N, int64_t K, int beta, void* stream) {
  int rc = check_f32("axn_gemm_wgrad_f32", dY, X, dW, M, N, K);
  if (rc) return rc;
  REQUIRE(beta == 0 || beta == 1, AXN_EINVAL, "axn_gemm_wgrad_f32: beta must be 0 or 1");
  return launch_gemm_f32(GEMM_TN, dY, X, dW, nullptr, nullptr, (int)N, (int)K,
                         (int)M, AXN_EPI_NONE, beta, (hipStream_t)stream);
}

size_t axn_mt_scan_workspace_bytes(int64_t n, int64_t total) {
  return mt_scan_workspace_bytes(n, total);
}

namespace {
int check_scan_args(const char* name, const void* const* h_g, const int64_t* h_sizes, int64_t n,
                    int g_dtype, float norm_type, int accumulate, axn_scan_result* result) {
  int rc = check_sizes(name, h_sizes, n);
  if (rc) return rc;
  REQUIRE(known_dtype(g_dtype), AXN_EINVAL, "%s: unknown gradient dtype %d", name, g_dtype);
  REQUIRE(n == 0 || h_g != nullptr, AXN_EINVAL, "%s: null pointer array", name);
  REQUIRE(result != nullptr, AXN_EINVAL, "%s: result is null", name);
  REQUIRE(((uintptr_t)result & 7u) == 0, AXN_EALIGN, "%s: result must be 8-byte aligned", name);
  REQUIRE(norm_type == norm_type, AXN_EINVAL, "%s: the norm's order is NaN", name);
  rc = check_list(name, h_g, "g", h_sizes, n, g_dtype == AXN_F32 ? 4 : 2);
  if (rc) return rc;
  REQUIRE(accumulate == 0 || accumulate == 1, AXN_EINVAL, "%s: accumulate must be 0 or 1", name);
  return AXN_OK;
}
}  // namespace

int axn_mt_scan_norm(const void* const* h_g, const int64_t* h_sizes, int64_t n,
                     int g_dtype, float inv_scale, float max_norm, float norm_type,
                     int accumulate, axn_scan_result* result, void* workspace,
                     size_t workspace_bytes, void* stream) {
  const char* name = "axn_mt_scan";
  int rc = check_scan_args(name, h_g, h_sizes, n, g_dtype, norm_type, accumulate, result);
  if (rc) return rc;
  REQUIRE(workspace != nullptr || workspace_bytes == 0, AXN_EINVAL, "%s: null workspace", name);
  REQUIRE(((uintptr_t)workspace & 15u) == 0, AXN_EALIGN,
          "%s: workspace must be 16-byte aligned", name);
  return launch_mt_scan(h_g, h_sizes, n, g_dtype, inv_scale, max_norm, norm_type, accumulate,
                        result, workspace, workspace_bytes, (hipStream_t)stream);
}

int axn_mt_scan(const void* const* h_g, const int64_t* h_sizes, int64_t n,
                int g_dtype, float inv_scale, float max_norm, int accumulate,
                axn_scan_result* result, void* workspace, size_t workspace_bytes,
                void* stream) {
  return axn_mt_scan_norm(h_g, h_sizes, n, g_dtype, inv_scale, max_norm, 2.0f, accumulate, result,
                          workspace, workspace_bytes, stream);
}

int axn_mt_scan_noalloc(const void* const* h_g, const int64_t* h_sizes, int64_t n,
                        int g_dtype, float inv_scale, float max_norm, int accumulate,
                        axn_scan_result* result, void* stream) {
  int rc = check_scan_args("axn_mt_scan_noalloc", h_g, h_sizes, n, g_dtype, 2.0f, accumulate,
                           result);
  if (rc) return rc;
  return launch_mt_scan_noalloc(h_g, h_sizes, n, g_dtype, inv_scale, max_norm, 2.0f, accumulate,
                                result, (hipStream_t)stream);
}

int axn_mt_adam(const void* const* h_g, void* const* h_p, void* const* h_m,
                void* const* h_v, void* const* h_plow, const int64_t* h_sizes,
                int64_t n, int g_dtype, int plow_dtype, float inv_scale,
                const axn_scan_result* scan, const axn_adam_hparams* hp,
                void* stream) {
  const char* name = "axn_mt_adam";
  int rc = check_sizes(name, h_sizes, n);
  if (rc) return rc;
  REQUIRE(known_dtype(g_dtype), AXN_EINVAL, "%s: unknown gradient dtype %d", name, g_dtype);
  REQUIRE(h_plow == nullptr || plow_dtype == AXN_BF16 || plow_dtype == AXN_F16,
          AXN_EINVAL, "%s: low-precision copy must be bf16 or fp16", name);
  REQUIRE(hp != nullptr, AXN_EINVAL, "%s: hyper-parameters are null", name);
  REQUIRE(n == 0 || (h_g && h_p && h_m && h_v), AXN_EINVAL, "%s: null pointer array", name);
  rc = check_list(name, h_g, "g", h_sizes, n, g_dtype == AXN_F32 ? 4 : 2);
  if (rc) return rc;
  rc = check_list(name, (const void* const*)h_p, "p", h_sizes, n, 4);
  if (rc) return rc;
  rc = check_list(name, (const void* const*)h_m, "m", h_sizes, n, 4);
  if (rc) return rc;
  rc = check_list(name, (const void* const*)h_v, "v", h_sizes, n, 4);
  if (rc) return rc;
  if (h_plow != nullptr) {
    rc = check_list(name, (const void* const*)h_plow, "p_lowp", h_sizes, n, 2);
    if (rc) return rc;
  }
  return launch_mt_adam(h_g, h_p, h_m, h_v, h_plow, h_sizes, n, g_dtype,
                        h_plow ? plow_dtype : AXN_BF16, inv_scale, scan, *hp,
                        (hipStream_t)stream);
}

int axn_mt_scale(void* const* h_g, const int64_t* h_sizes, int64_t n, int g_dtype,
                 float inv_scale, const axn_scan_result* scan, int use_clip,
                 void* stream) {
  const char* name = "axn_mt_scale";
  int rc = check_sizes(name, h_sizes, n);
  if (rc) return rc;
  REQUIRE(known_dtype(g_dtype), AXN_EINVAL, "%s: unknown gradient dtype %d", name, g_dtype);
  REQUIRE(n == 0 || h_g != nullptr, AXN_EINVAL, "%s: null pointer array", name);
  REQUIRE(!use_clip || scan != nullptr, AXN_EINVAL, "%s: clipping needs a scan result", name);
  rc = check_list(name, (const void* const*)h_g, "g", h_sizes, n, g_dtype == AXN_F32 ? 4 : 2);
  if (rc) return rc;
  return launch_mt_scale(h_g, h_sizes, n, g_dtype, inv_scale, scan, use_clip,
                         (hipStream_t)stream);
}

}  // extern "C"
