// fp32 GEMMs for full-precision Linear layers on gfx950.  The reference's own
// layer tests run in fp32 (axonn/tests/test_intra_layer_fc.py:25); this is the
// same three products as the bf16 path (fully_connected.py:118, :140, :147-151)
// with fp32 operands, for any M, N, K >= 1.
//
// One wave per workgroup owns a (16 FM) x (16 FN) output tile and feeds
// v_mfma_f32_16x16x4_f32 (true fp32 products, fp32 accumulate) straight from
// global memory: no LDS, no barriers.  A 16 x 4 operand block wants, in lane l,
// the element of one row (r = l % 16) and contraction index q = l / 16; MFMA s of a
// 16-deep block takes contraction index 4 q + s from both operands.  Which row of
// the tile lane r of fragment i stands for is free as long as loads and stores
// agree; it is row FM r + i (column FN r + j), so that
//   * a contraction-contiguous operand is read with one 16-byte load per fragment
//     (indices 4 q .. 4 q + 3 of the lane's row),
//   * an operand stored the other way round is read with one FM- (FN-) float load
//     per contraction index (the lane's FM consecutive rows), and
//   * a lane stores FN consecutive output columns at once.
// Full-precision layers are small or rare here: tiles are chosen for many waves
// (latency hiding by occupancy and by U blocks of loads in flight per wave).
#include "axn_internal.h"

namespace axn {
namespace {

typedef __attribute__((ext_vector_type(4))) float f32x4;

// Full-precision layers keep the library erff.
__device__ __forceinline__ float gelu_erff(float z) {
  return 0.5f * z * (1.0f + erff(z * 0.70710678118654752440f));
}

template <int F>
struct VecOf {
  typedef float type __attribute__((ext_vector_type(F)));
};
template <>
struct VecOf<1> {
  typedef float type;
};
template <int F>
__device__ __forceinline__ float vec_get(const typename VecOf<F>::type& v, int i) {
  if constexpr (F == 1) return v;
  else return v[i];
}

// One 16-deep block of one operand for the F fragments of a lane: x[f][s] is the
// element of row F r + f (clamped to the last row) and contraction index k + s.
//   KMAJOR: element (row, k) at base[row * Kc + k]; else at base[k * rows + row]
//   VEC:    Kc % 4 == 0, a 16-byte aligned base and (unless KMAJOR) rows % F == 0:
//           vector loads
//   GUARD:  indices >= Kc read as zero (the tail of the contraction)
template <bool KMAJOR, int F, bool VEC, bool GUARD>
__device__ __forceinline__ void load_block(float (&x)[F][4], const float* __restrict__ base,
                                           int row0, int rows, int k, int Kc) {
#pragma unroll
  for (int f = 0; f < F; ++f)
#pragma unroll
    for (int s = 0; s < 4; ++s) x[f][s] = 0.f;
  if (KMAJOR) {
#pragma unroll
    for (int f = 0; f < F; ++f) {
      const float* p = base + (int64_t)min(row0 + f, rows - 1) * Kc;
      if (VEC) {  // the four indices are in or out together
        if (!GUARD || k < Kc) {
          const f32x4 v = *(const f32x4*)(p + k);
#pragma unroll
          for (int s = 0; s < 4; ++s) x[f][s] = v[s];
        }
      } else {
#pragma unroll
        for (int s = 0; s < 4; ++s)
          if (!GUARD || k + s < Kc) x[f][s] = p[k + s];
      }
    }
  } else if (VEC) {  // the F rows are in or out together
    const float* p = base + min(row0, rows - F);
#pragma unroll
    for (int s = 0; s < 4; ++s)
      if (!GUARD || k + s < Kc) {
        const typename VecOf<F>::type v = *(const typename VecOf<F>::type*)(p + (int64_t)(k + s) * rows);
#pragma unroll
        for (int f = 0; f < F; ++f) x[f][s] = vec_get<F>(v, f);
      }
  } else {
#pragma unroll
    for (int f = 0; f < F; ++f) {
      const float* p = base + min(row0 + f, rows - 1);
#pragma unroll
      for (int s = 0; s < 4; ++s)
        if (!GUARD || k + s < Kc) x[f][s] = p[(int64_t)(k + s) * rows];
    }
  }
}

// WAVES > 1: the waves of a workgroup share one tile and take the 16 U-deep chunks of
// the contraction in turn; their partial sums meet in LDS and are added in wave order.
template <bool AK, bool BKM, int EPI, int FM, int FN, int U, bool VEC, int WAVES>
__global__ void __launch_bounds__(64 * WAVES)
    gemm_f32_kernel(const float* __restrict__ A, const float* __restrict__ B,
                    float* __restrict__ C, const float* __restrict__ bias,
                    float* __restrict__ Z, int M, int N, int Kc, int tiles_n, int beta) {
  const int lane = threadIdx.x & 63;
  const int wave = WAVES > 1 ? threadIdx.x >> 6 : 0;
  const int r = lane & 15, q = lane >> 4;
  const int tm = blockIdx.x / tiles_n, tn = blockIdx.x - tm * tiles_n;
  const int m0 = tm * 16 * FM, n0 = tn * 16 * FN;
  // Rows and columns past the edge read a valid one: their products land in output
  // elements that are never stored.
  const int arow = m0 + FM * r, bcol = n0 + FN * r;

  f32x4 acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

  auto blocks = [&](auto guard_, int k0, auto nblk_) {
    constexpr bool GUARD = decltype(guard_)::value;
    constexpr int NB = decltype(nblk_)::value;
    float a[NB][FM][4], b[NB][FN][4];
#pragma unroll
    for (int u = 0; u < NB; ++u) {
      const int k = k0 + 16 * u + 4 * q;
      load_block<AK, FM, VEC, GUARD>(a[u], A, arow, M, k, Kc);
      load_block<BKM, FN, VEC, GUARD>(b[u], B, bcol, N, k, Kc);
    }
#pragma unroll
    for (int u = 0; u < NB; ++u)
#pragma unroll
      for (int s = 0; s < 4; ++s)
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
          for (int j = 0; j < FN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[u][i][s], b[u][j][s], acc[i][j], 0, 0, 0);
  };

  const int whole = Kc / (16 * U) * (16 * U);  // the part made of whole chunks
  for (int k0 = wave * 16 * U; k0 < whole; k0 += WAVES * 16 * U)
    blocks(std::false_type{}, k0, std::integral_constant<int, U>{});
  for (int k0 = whole + wave * 16; k0 < Kc; k0 += WAVES * 16)
    blocks(std::true_type{}, k0, std::integral_constant<int, 1>{});

  if constexpr (WAVES > 1) {
    __shared__ f32x4 part[WAVES - 1][FM * FN][64];
    if (wave > 0) {
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) part[wave - 1][i * FN + j][lane] = acc[i][j];
    }
    __syncthreads();
    if (wave > 0) return;
#pragma unroll
    for (int w = 0; w < WAVES - 1; ++w)
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) acc[i][j] += part[w][i * FN + j][lane];
  }

  // Register v of acc[i][j] in lane (r, q) is output row FM (4 q + v) + i, column FN r + j.
  using vec = typename VecOf<FN>::type;
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int row = m0 + FM * (4 * q + v) + i;
      if (row >= M) continue;
      const int64_t o = (int64_t)row * N + bcol;
      float x[FN];
#pragma unroll
      for (int j = 0; j < FN; ++j) x[j] = acc[i][j][v];
      if (VEC) {  // N % FN == 0: the lane's FN columns are in or out together
        if (bcol >= N) continue;
        if (EPI == AXN_EPI_BIAS || EPI == AXN_EPI_BIAS_GELU) {
          const vec bv = *(const vec*)(bias + bcol);
#pragma unroll
          for (int j = 0; j < FN; ++j) x[j] += vec_get<FN>(bv, j);
        }
        vec y;
        if (EPI == AXN_EPI_BIAS_GELU || EPI == AXN_EPI_GELU) {
          if (Z != nullptr) {
#pragma unroll
            for (int j = 0; j < FN; ++j) {
              if constexpr (FN == 1) y = x[j];
              else y[j] = x[j];
            }
            *(vec*)(Z + o) = y;
          }
#pragma unroll
          for (int j = 0; j < FN; ++j) x[j] = gelu_erff(x[j]);
        }
        if (beta) {
          const vec old = *(const vec*)(C + o);
#pragma unroll
          for (int j = 0; j < FN; ++j) x[j] += vec_get<FN>(old, j);
        }
#pragma unroll
        for (int j = 0; j < FN; ++j) {
          if constexpr (FN == 1) y = x[j];
          else y[j] = x[j];
        }
        *(vec*)(C + o) = y;
      } else {
#pragma unroll
        for (int j = 0; j < FN; ++j) {
          if (bcol + j >= N) continue;
          float t = x[j];
          if (EPI == AXN_EPI_BIAS || EPI == AXN_EPI_BIAS_GELU) t += bias[bcol + j];
          if (EPI == AXN_EPI_BIAS_GELU || EPI == AXN_EPI_GELU) {
            if (Z != nullptr) Z[o + j] = t;
            t = gelu_erff(t);
          }
          if (beta) t += C[o + j];
          C[o + j] = t;
        }
      }
    }
}

template <bool AK, bool BKM, int EPI, int FM, int FN, int U, int WAVES>
int launch_tile(const float* A, const float* B, float* C, const float* bias, float* Z, int M,
                int N, int Kc, int beta, hipStream_t stream) {
  const long long tiles_m = (M + 16 * FM - 1) / (16 * FM), tiles_n = (N + 16 * FN - 1) / (16 * FN);
  const long long nwg = tiles_m * tiles_n;
  if (nwg > 0x7fffffffLL) {
    set_error("gemm_f32: too many output tiles (%lld)", nwg);
    return AXN_ELIMIT;
  }
  // Vector accesses need whole groups (four along the contraction, FM rows, FN
  // columns) and 16-byte aligned bases.
  const uintptr_t ptrs = (uintptr_t)A | (uintptr_t)B | (uintptr_t)C | (uintptr_t)bias | (uintptr_t)Z;
  const bool vec = Kc % 4 == 0 && (AK || M % FM == 0) && N % FN == 0 && (ptrs & 15u) == 0;
  if (vec)
    hipLaunchKernelGGL((gemm_f32_kernel<AK, BKM, EPI, FM, FN, U, true, WAVES>), dim3((unsigned)nwg),
                       dim3(64 * WAVES), 0, stream, A, B, C, bias, Z, M, N, Kc, (int)tiles_n, beta);
  else
    hipLaunchKernelGGL((gemm_f32_kernel<AK, BKM, EPI, FM, FN, U, false, WAVES>), dim3((unsigned)nwg),
                       dim3(64 * WAVES), 0, stream, A, B, C, bias, Z, M, N, Kc, (int)tiles_n, beta);
  AXN_HIP_TRY(hipGetLastError());
  return AXN_OK;
}

// The largest of the 64 x 64, 32 x 32 and 16 x 16 tiles (a loaded element is used 4,
// 2, 1 times) that still gives the chip's 1024 SIMDs a wave each; smaller tiles keep
// more loads in flight per wave.  With fewer than 4096 tiles and a contraction of KMIN
// or more (256 for the smallest tile, 2048 for the middle one; measured: the split
// loses on the largest tile and on shorter contractions), four waves share a tile.
template <bool AK, bool BKM, int EPI, int FM, int FN, int U, int KMIN>
int launch_waves(long long tiles, const float* A, const float* B, float* C, const float* bias,
                 float* Z, int M, int N, int Kc, int beta, hipStream_t stream) {
  if (tiles < 4096 && Kc >= KMIN)
    return launch_tile<AK, BKM, EPI, FM, FN, (U > 4 ? 4 : U), 4>(A, B, C, bias, Z, M, N, Kc, beta, stream);
  return launch_tile<AK, BKM, EPI, FM, FN, U, 1>(A, B, C, bias, Z, M, N, Kc, beta, stream);
}

template <bool AK, bool BKM, int EPI>
int launch_epi(const float* A, const float* B, float* C, const float* bias, float* Z, int M, int N,
               int Kc, int beta, hipStream_t stream) {
  const long long tiles64 = (long long)((M + 63) / 64) * ((N + 63) / 64);
  const long long tiles32 = (long long)((M + 31) / 32) * ((N + 31) / 32);
  const long long tiles16 = (long long)((M + 15) / 16) * ((N + 15) / 16);
  if (tiles64 >= 1024)
    return launch_tile<AK, BKM, EPI, 4, 4, 2, 1>(A, B, C, bias, Z, M, N, Kc, beta, stream);
  if (tiles32 >= 1024)
    return launch_waves<AK, BKM, EPI, 2, 2, 4, 2048>(tiles32, A, B, C, bias, Z, M, N, Kc, beta, stream);
  return launch_waves<AK, BKM, EPI, 1, 1, 8, 256>(tiles16, A, B, C, bias, Z, M, N, Kc, beta, stream);
}

}  // namespace

int launch_gemm_f32(GemmLayout layout, const float* A, const float* B, float* C,
                    const float* bias, float* Z, int M, int N, int Kc,
                    int epilogue, int beta, hipStream_t stream) {
  switch (layout) {
    case GEMM_NT:
      switch (epilogue) {
        case AXN_EPI_NONE:
          return launch_epi<true, true, AXN_EPI_NONE>(A, B, C, bias, Z, M, N, Kc, beta, stream);
        case AXN_EPI_BIAS:
          return launch_epi<true, true, AXN_EPI_BIAS>(A, B, C, bias, Z, M, N, Kc, beta, stream);
        case AXN_EPI_BIAS_GELU:
          return launch_epi<true, true, AXN_EPI_BIAS_GELU>(A, B, C, bias, Z, M, N, Kc, beta, stream);
        default:
          return launch_epi<true, true, AXN_EPI_GELU>(A, B, C, bias, Z, M, N, Kc, beta, stream);
      }
    case GEMM_NN:
      return launch_epi<true, false, AXN_EPI_NONE>(A, B, C, bias, Z, M, N, Kc, beta, stream);
    default:
      return launch_epi<false, false, AXN_EPI_NONE>(A, B, C, bias, Z, M, N, Kc, beta, stream);
  }
}

}  // namespace axn
