// Backward of the fused bias/GELU epilogue for gfx950: one HBM pass computing
//   dZ = dY * gelu'(Z)   and   dbias[n] = sum_m dZ[m, n]
// which is what autograd derives from the reference's `x + bias`
// (axonn/intra_layer/fully_connected.py:348) followed by the caller's exact-erf
// nn.GELU.  Lanes move 16 bytes (8 bf16 columns); column sums are kept in
// registers over a band of rows, combined through LDS, written as one fp32
// partial row per band and reduced over bands in a fixed order by a second
// kernel, so the result does not depend on scheduling.
#include "axn_internal.h"

namespace axn {
namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int EW_TX = 64;          // lanes along columns (8 columns each)
constexpr int EW_TY = 4;           // row phases per workgroup
constexpr int EW_COLS = EW_TX * 8; // 512 columns per workgroup
constexpr int EW_BAND = 128;       // rows per workgroup

// 8 consecutive columns as floats, for bf16 (16 bytes) and fp32 (32 bytes) rows.
__device__ __forceinline__ void load8(const uint16_t* p, float (&x)[8]) {
  const bf16x8 v = *(const bf16x8*)p;
#pragma unroll
  for (int e = 0; e < 8; ++e) x[e] = (float)v[e];
}
__device__ __forceinline__ void load8(const float* p, float (&x)[8]) {
  const f32x4 a = *(const f32x4*)p, b = *(const f32x4*)(p + 4);
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    x[e] = a[e];
    x[4 + e] = b[e];
  }
}
// Stores 8 columns rounded to the storage type and returns the stored values.
__device__ __forceinline__ void store8(uint16_t* p, float (&x)[8]) {
  bf16x8 v;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    v[e] = (__bf16)x[e];
    x[e] = (float)v[e];
  }
  *(bf16x8*)p = v;
}
__device__ __forceinline__ void store8(float* p, float (&x)[8]) {
  *(f32x4*)p = f32x4{x[0], x[1], x[2], x[3]};
  *(f32x4*)(p + 4) = f32x4{x[4], x[5], x[6], x[7]};
}

template <typename T, bool HAS_Z>
__global__ void __launch_bounds__(EW_TX* EW_TY)
    dgelu_dbias_kernel(const T* dY, const T* Z, T* dZ, float* partial, int64_t M,
                       int64_t N, int64_t ld) {
  const int tx = threadIdx.x % EW_TX, ty = threadIdx.x / EW_TX;
  const int64_t col = (int64_t)blockIdx.x * EW_COLS + tx * 8;
  const int64_t r0 = (int64_t)blockIdx.y * EW_BAND;
  int64_t r1 = r0 + EW_BAND;
  if (r1 > M) r1 = M;
  float s[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  if (col < N) {
    for (int64_t r = r0 + ty; r < r1; r += EW_TY) {
      const int64_t o = r * ld + col;
      float g[8];
      load8(dY + o, g);
      if (HAS_Z) {
        float z[8];
        load8(Z + o, z);
#pragma unroll
        for (int e = 0; e < 8; ++e) g[e] *= dgelu_exact(z[e]);
        store8(dZ + o, g);  // g becomes what was stored: the sum of what wgrad reads
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) s[e] += g[e];
    }
  }
  if (partial == nullptr) return;
  __shared__ float red[EW_TY][EW_COLS];
#pragma unroll
  for (int e = 0; e < 8; ++e) red[ty][tx * 8 + e] = s[e];
  __syncthreads();
  for (int c = threadIdx.x; c < EW_COLS; c += EW_TX * EW_TY) {
    const int64_t gc = (int64_t)blockIdx.x * EW_COLS + c;
    if (gc < N)
      partial[(int64_t)blockIdx.y * N + gc] =
          (red[0][c] + red[1][c]) + (red[2][c] + red[3][c]);
  }
}

// Column sums over the band partials in a fixed order: 64 columns per workgroup,
// the bands split in 4 consecutive quarters summed by 4 threads each in band
// order, the quarters then combined as (q0 + q1) + (q2 + q3).
__global__ void __launch_bounds__(256)
    dbias_reduce_kernel(const float* partial, float* dbias, int64_t bands,
                        int64_t N, int beta) {
  __shared__ float red[4][64];
  const int tx = threadIdx.x & 63, q = threadIdx.x >> 6;
  const int64_t c = (int64_t)blockIdx.x * 64 + tx;
  const int64_t per = (bands + 3) / 4;
  const int64_t b0 = q * per, b1 = (b0 + per < bands) ? b0 + per : bands;
  float s = 0.f;
  if (c < N)
    for (int64_t b = b0; b < b1; ++b) s += partial[b * N + c];
  red[q][tx] = s;
  __syncthreads();
  if (q == 0 && c < N) {
    const float t = (red[0][tx] + red[1][tx]) + (red[2][tx] + red[3][tx]);
    dbias[c] = beta ? dbias[c] + t : t;
  }
}

}  // namespace

size_t dgelu_dbias_workspace_bytes(int64_t M, int64_t N) {
  if (M <= 0 || N <= 0) return 0;
  return (size_t)((M + EW_BAND - 1) / EW_BAND) * (size_t)N * sizeof(float);
}

int launch_dgelu_dbias(const void* dY, const void* Z, void* dZ, int dtype,
                       float* dbias, int64_t M, int64_t N, int64_t ld, int beta,
                       void* ws, size_t ws_bytes, hipStream_t stream) {
  const int64_t bands = (M + EW_BAND - 1) / EW_BAND;
  float* partial = nullptr;
  if (dbias != nullptr) {
    if (ws == nullptr || ws_bytes < dgelu_dbias_workspace_bytes(M, N)) {
      set_error("dgelu_dbias: workspace too small (%zu bytes given, %zu needed)",
                ws_bytes, dgelu_dbias_workspace_bytes(M, N));
      return AXN_EINVAL;
    }
    partial = (float*)ws;
  }
  const dim3 grid((unsigned)((N + EW_COLS - 1) / EW_COLS), (unsigned)bands);
  if (bands > 65535) {
    set_error("dgelu_dbias: too many rows (%lld)", (long long)M);
    return AXN_ELIMIT;
  }
  const dim3 block(EW_TX * EW_TY);
  if (dtype == AXN_F32) {
    const float *y = (const float*)dY, *z = (const float*)Z;
    if (Z != nullptr)
      hipLaunchKernelGGL((dgelu_dbias_kernel<float, true>), grid, block, 0, stream,
                         y, z, (float*)dZ, partial, M, N, ld);
    else
      hipLaunchKernelGGL((dgelu_dbias_kernel<float, false>), grid, block, 0, stream,
                         y, z, (float*)dZ, partial, M, N, ld);
  } else {
    const uint16_t *y = (const uint16_t*)dY, *z = (const uint16_t*)Z;
    if (Z != nullptr)
      hipLaunchKernelGGL((dgelu_dbias_kernel<uint16_t, true>), grid, block, 0,
                         stream, y, z, (uint16_t*)dZ, partial, M, N, ld);
    else
      hipLaunchKernelGGL((dgelu_dbias_kernel<uint16_t, false>), grid, block, 0,
                         stream, y, z, (uint16_t*)dZ, partial, M, N, ld);
  }
  AXN_HIP_TRY(hipGetLastError());
  if (dbias != nullptr) {
    hipLaunchKernelGGL(dbias_reduce_kernel, dim3((unsigned)((N + 63) / 64)),
                       dim3(256), 0, stream, partial, dbias, bands, N, beta);
    AXN_HIP_TRY(hipGetLastError());
  }
  return AXN_OK;
}

}  // namespace axn
