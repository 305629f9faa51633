// Internal declarations shared by the kernel translation units and the C ABI.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "axn.h"

namespace axn {

// Thread-local error text behind axn_last_error().
void set_error(const char* fmt, ...);
int hip_fail(hipError_t e, const char* what);

#define AXN_HIP_TRY(expr)                                  \
  do {                                                     \
    hipError_t e__ = (expr);                               \
    if (e__ != hipSuccess) return ::axn::hip_fail(e__, #expr); \
  } while (0)

// ---- exact-erf GELU -----------------------------------------------------------
// gelu(x) = x * Phi(x), Phi(x) = (1 + erf(x / sqrt 2)) / 2, the definition behind
// torch.nn.GELU() (approximate='none').  The library erff costs about 100 VALU
// operations per element with both of its branches taken in a wave, which made
// the fused epilogue as expensive as the GEMM's main loop.  Here
//   erfc(z) = t (a1 + t (a2 + t (a3 + t (a4 + t a5)))) exp(-z^2),  t = 1 / (1 + p z),
// Abramowitz & Stegun 7.1.26, |error| <= 1.5e-7 absolute for z >= 0; the negative
// side uses Phi(-x) = 1 - Phi(x) without cancellation.  The same exponential
// serves the density in the derivative.
struct GeluTerms {
  float cdf;   // Phi(x)
  float expo;  // exp(-x^2 / 2)
};
__device__ __forceinline__ GeluTerms gelu_terms(float x) {
  const float z = fabsf(x) * 0.70710678118654752440f;
  const float t = __builtin_amdgcn_rcpf(fmaf(0.3275911f, z, 1.0f));
  float p = 1.061405429f;
  p = fmaf(p, t, -1.453152027f);
  p = fmaf(p, t, 1.421413741f);
  p = fmaf(p, t, -0.284496736f);
  p = fmaf(p, t, 0.254829592f);
  const float e = __expf(-z * z);
  const float q = 0.5f * p * t * e;  // Phi(-|x|)
  GeluTerms r;
  r.cdf = x < 0.0f ? q : 1.0f - q;
  r.expo = e;
  return r;
}
// gelu(x) = max(x, 0) - |x| Phi(-|x|): no select between the two halves of Phi, and
// Phi(-|x|) = t (a1/2 + t (a2/2 + ...)) exp2(-x^2 log2(e) / 2), t = 1 / (1 + (p / sqrt 2) |x|),
// straight from x (the same approximation as gelu_terms with the constants folded:
// 11 full-rate operations, one reciprocal and one exp2 per element in the GEMM epilogue).
__device__ __forceinline__ float gelu_exact(float x) {
  const float ax = fabsf(x);
  const float t = __builtin_amdgcn_rcpf(fmaf(0.3275911f * 0.70710678118654752440f, ax, 1.0f));
  float p = 0.5f * 1.061405429f;
  p = fmaf(p, t, 0.5f * -1.453152027f);
  p = fmaf(p, t, 0.5f * 1.421413741f);
  p = fmaf(p, t, 0.5f * -0.284496736f);
  p = fmaf(p, t, 0.5f * 0.254829592f);
  const float e = __builtin_amdgcn_exp2f((x * x) * (-0.5f * 1.44269504088896340736f));
  const float q = (p * t) * e;  // Phi(-|x|)
  float pos;  // max(x, 0) as the one instruction (fmaxf adds a pass that quiets NaNs first;
              // a NaN x still gives NaN through the other operand)
  asm("v_max_f32 %0, 0, %1" : "=v"(pos) : "v"(x));
  return fmaf(-ax, q, pos);
}
// d/dx gelu(x) = Phi(x) + x phi(x), phi the standard normal density.
__device__ __forceinline__ float dgelu_exact(float x) {
  const GeluTerms g = gelu_terms(x);
  return fmaf(x * 0.39894228040143267794f, g.expo, g.cdf);
}

// sigmoid(x) = 1 / (1 + exp(-x)); exp overflows to +inf for x < -88 and the
// reciprocal then gives the correct limit 0.
__device__ __forceinline__ float sigmoid_f(float x) {
  return __builtin_amdgcn_rcpf(1.0f + __expf(-x));
}

// ---- bf16 GEMM ------------------------------------------------------------
// C[M x N] (+)= A * B over a contraction of length Kc, bf16 operands, fp32
// accumulate.  Each operand is either "K-major" (stored [rows][Kc], the
// contraction index contiguous) or "MN-major" (stored [Kc][rows]).
struct GemmArgs {
  const uint16_t* A;
  const uint16_t* B;
  void* C;            // bf16 or fp32, row-major [M][N]
  const float* bias;  // [N] or null
  uint16_t* Z;        // optional pre-activation copy, bf16 [M][N], ld = ldc
  int M, N, Kc;
  int64_t lda, ldb, ldc;
  int tiles_m, tiles_n;
  int beta;  // 0: C = AB ; 1: C += AB
  // First workgroup of this problem in a launch that runs two problems (launch_gemm_backward).
  int wg_first;
  // Split of the contraction over workgroups (splits > 1): workgroup id / tiles is the
  // split, which covers k_split contraction elements and writes its fp32 partial
  // product to C + split * M * ldc.  0 or 1: no split.
  int splits, k_split;
  // Gate/up forward with the SwiGLU in the epilogue (launch_gemm_swiglu): B holds the gate
  // weights, B2 the up weights (same shape and ldb); C receives silu(gate) * up, G and U
  // (optional, ld = ldc) the two pre-activations; N counts the columns of C.
  const uint16_t* B2;
  uint16_t* G;
  uint16_t* U;
  // Two-term product C = A B + A2 B2 in one pass (launch_gemm_pair): the first k_first
  // elements of the contraction Kc come from (A, B), the others from (A2, B2), which have
  // the leading dimensions of A and B.
  const uint16_t* A2;
  int k_first;
};

enum GemmLayout { GEMM_NT = 0, GEMM_NN = 1, GEMM_TN = 2 };
// GEMM_NT: A K-major, B K-major   (forward  Y  = X  W^T)
// GEMM_NN: A K-major, B MN-major  (dgrad    dX = dY W  )
// GEMM_TN: A MN-major, B MN-major (wgrad    dW = dY^T X)

int launch_gemm_bf16(GemmLayout layout, const GemmArgs& args, int epilogue,
                     bool out_f32, hipStream_t stream);
// The same kernels on IEEE half operands (v_mfma_f32_16x16x32_f16, half outputs).
int launch_gemm_f16(GemmLayout layout, const GemmArgs& args, int epilogue, bool out_f32,
                    hipStream_t stream);
// Split-contraction variant for problems with few output tiles: the number of splits
// chosen for an [M x N] output over a contraction of Kc (1 = do not split; *wide_tiles:
// the parts run on 256 x 128 tiles instead of 128 x 128), and the
// launch: partial products in fp32 to `ws` (splits * M * N floats), then one pass that
// adds them in split order, adds the old output if args.beta, and stores args.C in
// out_dtype.  No epilogue.
int gemm_splits(GemmLayout layout, const GemmArgs& args, bool* wide_tiles = nullptr);
// dX = dY W and dW (+)= dY^T X of one layer, args as for GEMM_NN and GEMM_TN.  Results are
// those of the two separate launches bit for bit; when the two problems' tile counts leave
// CUs idle one after the other but not together, they run as ONE launch (see gemm_bf16.hip).
int launch_gemm_backward(const GemmArgs& dgrad, const GemmArgs& wgrad, bool half, bool dw_f32,
                         hipStream_t stream);
int launch_gemm_splitk(GemmLayout layout, const GemmArgs& args, bool half, int out_dtype,
                       int splits, bool wide_tiles, float* ws, hipStream_t stream);

// C = silu(A B^T) * (A B2^T) in one launch (both weight matrices [N][Kc], K-major), for
// M % 256 == 0, N % 128 == 0, Kc % 64 == 0 and operands below 2 GiB; AXN_ESHAPE otherwise.
int launch_gemm_swiglu(const GemmArgs& args, bool half, hipStream_t stream);

// C[M x N] = A B + A2 B2, A / A2 K-major [M][k1], [M][k2], B / B2 MN-major [k1][N], [k2][N]
// (two input-gradient products added in the accumulators): args.Kc = k1 + k2,
// args.k_first = k1.  Shapes of whole 128 x 128 tiles, k1 % 64 == 0 and >= 128,
// k2 % 64 == 0 and >= 64, operands below 2 GiB; AXN_ESHAPE otherwise.
int launch_gemm_pair(const GemmArgs& args, bool half, hipStream_t stream);

// ---- fp32 GEMM (full-precision layers) --------------------------------------
int launch_gemm_f32(GemmLayout layout, const float* A, const float* B, float* C,
                    const float* bias, float* Z, int M, int N, int Kc,
                    int epilogue, int beta, hipStream_t stream);

// ---- elementwise backward of the bias/GELU epilogue ----------------------
size_t dgelu_dbias_workspace_bytes(int64_t M, int64_t N);
int launch_dgelu_dbias(const void* dY, const void* Z, void* dZ, int dtype,
                       float* dbias, int64_t M, int64_t N, int64_t ld, int beta,
                       void* ws, size_t ws_bytes, hipStream_t stream);

// ---- SwiGLU activation of the Llama MLP and its backward -----------------------
int launch_swiglu_fwd(const void* gate, const void* up, void* out, int dtype, int64_t M,
                      int64_t N, int64_t ld, hipStream_t stream);
// ld: row stride of dout, gate and up; ld_out: of dgate and dup
int launch_swiglu_bwd(const void* dout, const void* gate, const void* up, void* dgate, void* dup,
                      int dtype, int64_t M, int64_t N, int64_t ld, int64_t ld_out,
                      hipStream_t stream);

// ---- embedding table: row gather, dense weight gradient, max_norm -------------------
size_t embedding_workspace_bytes(int64_t T, int64_t V);
int launch_embedding_fwd(const int64_t* ids, const void* W, void* out, int elem_bytes, int64_t T,
                         int64_t V, int64_t H, int64_t ldw, int64_t ldo, int* status,
                         hipStream_t stream);
int launch_embedding_bwd(const int64_t* ids, const void* dY, void* dW, int dy_dtype, int dw_dtype,
                         int64_t T, int64_t V, int64_t H, int64_t lddy, int64_t lddw,
                         int64_t padding_idx, int scale_by_freq, int beta, void* ws,
                         size_t ws_bytes, hipStream_t stream);
int launch_embedding_renorm(const int64_t* ids, void* W, int dtype, int64_t T, int64_t V,
                            int64_t H, int64_t ldw, float max_norm, float norm_type, void* ws,
                            size_t ws_bytes, hipStream_t stream);

// ---- multi-tensor optimizer ------------------------------------------------
size_t mt_scan_workspace_bytes(int64_t n, int64_t total);
int launch_mt_scan(const void* const* h_g, const int64_t* h_sizes, int64_t n,
                   int g_dtype, float inv_scale, float max_norm, float norm_type,
                   int accumulate, axn_scan_result* result, void* ws, size_t ws_bytes,
                   hipStream_t stream);
// The same with the partial results in the library's own device array (no workspace).
int launch_mt_scan_noalloc(const void* const* h_g, const int64_t* h_sizes, int64_t n,
                           int g_dtype, float inv_scale, float max_norm, float norm_type,
                           int accumulate, axn_scan_result* result, hipStream_t stream);
int launch_mt_adam(const void* const* h_g, void* const* h_p, void* const* h_m,
                   void* const* h_v, void* const* h_plow, const int64_t* h_sizes,
                   int64_t n, int g_dtype, int plow_dtype, float inv_scale,
                   const axn_scan_result* scan, const axn_adam_hparams& hp,
                   hipStream_t stream);
int launch_mt_scale(void* const* h_g, const int64_t* h_sizes, int64_t n,
                    int g_dtype, float inv_scale, const axn_scan_result* scan,
                    int use_clip, hipStream_t stream);


}  // namespace axn
