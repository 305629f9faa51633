// fp32 GEMMs for full-precision Linear layers on gfx950.  The reference's own
// layer tests run in fp32 (axonn/tests/test_intra_layer_fc.py:25); this is the
// same three products as the bf16 path (fully_connected.py:118, :140, :147-151)
// with fp32 operands, for any M, N, K >= 1.  A workgroup owns a 64 x 64 output
// tile, stages 16 contraction steps of both operands in LDS as [k][row] and
// every lane accumulates a 4 x 4 block with fp32 FMAs.
#include "axn_internal.h"

namespace axn {
namespace {

constexpr int FT = 64;   // output tile edge
constexpr int FK = 16;   // contraction steps per stage

// Full-precision layers keep the library erff.
__device__ __forceinline__ float gelu_erff(float z) {
  return 0.5f * z * (1.0f + erff(z * 0.70710678118654752440f));
}

template <bool AK, bool BKM, int EPI>
__global__ void __launch_bounds__(256)
    gemm_f32_kernel(const float* __restrict__ A, const float* __restrict__ B,
                    float* __restrict__ C, const float* __restrict__ bias,
                    float* __restrict__ Z, int M, int N, int Kc, int beta) {
  __shared__ float sA[FK][FT + 4];
  __shared__ float sB[FK][FT + 4];
  const int tid = threadIdx.x;
  const int tx = tid % 16, ty = tid / 16;
  const int m0 = blockIdx.y * FT, n0 = blockIdx.x * FT;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < Kc; k0 += FK) {
#pragma unroll
    for (int i = 0; i < FT * FK / 256; ++i) {
      const int id = i * 256 + tid;
      {
        int r, k;
        if (AK) { r = id / FK; k = id % FK; } else { k = id / FT; r = id % FT; }
        const int gr = m0 + r, gk = k0 + k;
        float x = 0.f;
        if (gr < M && gk < Kc)
          x = AK ? A[(int64_t)gr * Kc + gk] : A[(int64_t)gk * M + gr];
        sA[k][r] = x;
      }
      {
        int r, k;
        if (BKM) { r = id / FK; k = id % FK; } else { k = id / FT; r = id % FT; }
        const int gr = n0 + r, gk = k0 + k;
        float x = 0.f;
        if (gr < N && gk < Kc)
          x = BKM ? B[(int64_t)gr * Kc + gk] : B[(int64_t)gk * N + gr];
        sB[k][r] = x;
      }
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < FK; ++k) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = sA[k][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = sB[k][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = m0 + ty * 4 + i;
    if (row >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int col = n0 + tx * 4 + j;
      if (col >= N) continue;
      const int64_t o = (int64_t)row * N + col;
      float v = acc[i][j];
      if (EPI == AXN_EPI_BIAS || EPI == AXN_EPI_BIAS_GELU) v += bias[col];
      if (EPI == AXN_EPI_BIAS_GELU || EPI == AXN_EPI_GELU) {
        if (Z != nullptr) Z[o] = v;
        v = gelu_erff(v);
      }
      if (beta) v += C[o];
      C[o] = v;
    }
  }
}

template <bool AK, bool BKM>
int launch_epi(const float* A, const float* B, float* C, const float* bias,
               float* Z, int M, int N, int Kc, int epilogue, int beta,
               hipStream_t stream) {
  const dim3 grid((N + FT - 1) / FT, (M + FT - 1) / FT), block(256);
  if (grid.y > 65535) {
    set_error("gemm_f32: too many rows (%d)", M);
    return AXN_ELIMIT;
  }
  switch (epilogue) {
    case AXN_EPI_NONE:
      hipLaunchKernelGGL((gemm_f32_kernel<AK, BKM, AXN_EPI_NONE>), grid, block, 0,
                         stream, A, B, C, bias, Z, M, N, Kc, beta);
      break;
    case AXN_EPI_BIAS:
      hipLaunchKernelGGL((gemm_f32_kernel<AK, BKM, AXN_EPI_BIAS>), grid, block, 0,
                         stream, A, B, C, bias, Z, M, N, Kc, beta);
      break;
    case AXN_EPI_BIAS_GELU:
      hipLaunchKernelGGL((gemm_f32_kernel<AK, BKM, AXN_EPI_BIAS_GELU>), grid, block,
                         0, stream, A, B, C, bias, Z, M, N, Kc, beta);
      break;
    default:
      hipLaunchKernelGGL((gemm_f32_kernel<AK, BKM, AXN_EPI_GELU>), grid, block, 0,
                         stream, A, B, C, bias, Z, M, N, Kc, beta);
      break;
  }
  AXN_HIP_TRY(hipGetLastError());
  return AXN_OK;
}

}  // namespace

int launch_gemm_f32(GemmLayout layout, const float* A, const float* B, float* C,
                    const float* bias, float* Z, int M, int N, int Kc,
                    int epilogue, int beta, hipStream_t stream) {
  switch (layout) {
    case GEMM_NT:
      return launch_epi<true, true>(A, B, C, bias, Z, M, N, Kc, epilogue, beta, stream);
    case GEMM_NN:
      return launch_epi<true, false>(A, B, C, bias, Z, M, N, Kc, epilogue, beta, stream);
    default:
      return launch_epi<false, false>(A, B, C, bias, Z, M, N, Kc, epilogue, beta, stream);
  }
}

}  // namespace axn
