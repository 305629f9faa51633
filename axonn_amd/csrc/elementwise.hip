// Backward of the fused bias/GELU epilogue for gfx950: one HBM pass computing
//   dZ = dY * gelu'(Z)   and   dbias[n] = sum_m dZ[m, n]
// which is what autograd derives from the reference's `x + bias`
// (axonn/intra_layer/fully_connected.py:348) followed by the caller's exact-erf
// nn.GELU.  Lanes move 16 bytes (8 bf16 columns); column sums are kept in
// registers over a band of rows, combined through LDS, written as one fp32
// partial row per band and reduced over bands in a fixed order by a second
// kernel, so the result does not depend on scheduling.
//
// Also here: the SwiGLU activation of the Llama MLP, h = silu(gate) * up, and its
// backward, each one HBM pass.  The reference's Llama patch
// (axonn/models/transformers/modify_llama.py:76-95) swaps the three projections
// for its Linear and leaves `act_fn(gate_proj(x)) * up_proj(x)` to separate
// elementwise kernels with a bf16 rounding in between; here the product is formed
// in fp32 and rounded once.
#include "axn_internal.h"

namespace axn {
namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int EW_TX = 64;          // lanes along columns (8 columns each)
constexpr int EW_TY = 4;           // row phases per workgroup
constexpr int EW_COLS = EW_TX * 8; // 512 columns per workgroup
constexpr int EW_BAND = 128;       // rows per workgroup (dGELU + dbias: column sums per band)
// Non-temporal loads of dY and Z: 12 % faster when the operands come from HBM (62 -> 55 us),
// 12 % slower when the memory-side cache holds them, which is the case in a training step
// (dY was written by the layer behind a moment ago): off.
constexpr bool DGELU_NT = false;
// SwiGLU has no sums to carry down the rows: one row piece per wave, the workgroups handed
// out in row-major order, so that the chip reads and writes one compact window of every
// operand (4096 x 14336 bf16 from HBM: forward 76 -> 59 us, backward 131 -> 98 us against
// 128-row bands, measured on MI355X).  Stores written through (nt + sc1), which gain 1 to
// 2 % in the optimizer's update kernel, change nothing in the forward and lose 6 % in the
// backward (two outputs): plain stores.
constexpr int SWIGLU_BAND = 4;

// 8 consecutive columns as floats, for bf16 / fp16 (16 bytes) and fp32 (32 bytes) rows.
// NT: non-temporal loads, for operands read once.  They are worth 15 % on the SwiGLU
// forward and 23 % on its backward and cost 12 % on dGELU (measured), so each kernel
// names its own.
template <bool NT, typename V>
__device__ __forceinline__ V load_vec(const void* p) {
  return NT ? __builtin_nontemporal_load((const V*)p) : *(const V*)p;
}
template <bool NT = false>
__device__ __forceinline__ void load8(const uint16_t* p, float (&x)[8]) {
  const bf16x8 v = load_vec<NT, bf16x8>(p);
#pragma unroll
  for (int e = 0; e < 8; ++e) x[e] = (float)v[e];
}
template <bool NT = false>
__device__ __forceinline__ void load8(const _Float16* p, float (&x)[8]) {
  const f16x8 v = load_vec<NT, f16x8>(p);
#pragma unroll
  for (int e = 0; e < 8; ++e) x[e] = (float)v[e];
}
template <bool NT = false>
__device__ __forceinline__ void load8(const float* p, float (&x)[8]) {
  const f32x4 a = load_vec<NT, f32x4>(p), b = load_vec<NT, f32x4>(p + 4);
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
__device__ __forceinline__ void store8(_Float16* p, float (&x)[8]) {
  f16x8 v;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    v[e] = (_Float16)x[e];
    x[e] = (float)v[e];
  }
  *(f16x8*)p = v;
}
__device__ __forceinline__ void store8(float* p, float (&x)[8]) {
  *(f32x4*)p = f32x4{x[0], x[1], x[2], x[3]};
  *(f32x4*)(p + 4) = f32x4{x[4], x[5], x[6], x[7]};
}

// Raw 8-column pieces of a row, so that a group of rows can be in flight as loads before
// any of it is converted.
template <typename T> struct Raw8;
template <> struct Raw8<uint16_t> { typedef bf16x8 type; };
template <> struct Raw8<_Float16> { typedef f16x8 type; };
template <> struct Raw8<float> { struct type { f32x4 lo, hi; }; };
template <typename T>
__device__ __forceinline__ typename Raw8<T>::type load_raw8(const T* p) {
  if constexpr (DGELU_NT && sizeof(T) == 2) {
    return __builtin_nontemporal_load((const typename Raw8<T>::type*)p);
  } else {
    return *(const typename Raw8<T>::type*)p;
  }
}
__device__ __forceinline__ void widen8(const bf16x8& v, float (&x)[8]) {
#pragma unroll
  for (int e = 0; e < 8; ++e) x[e] = (float)v[e];
}
__device__ __forceinline__ void widen8(const f16x8& v, float (&x)[8]) {
#pragma unroll
  for (int e = 0; e < 8; ++e) x[e] = (float)v[e];
}
__device__ __forceinline__ void widen8(const Raw8<float>::type& v, float (&x)[8]) {
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    x[e] = v.lo[e];
    x[4 + e] = v.hi[e];
  }
}

// A thread walks its rows in groups of EW_GROUP: the loads of the next group are issued
// before the stores of this one.  The memory counter of a wave is in order, so a load
// behind a store returns only after the store is acknowledged; with the loads in front,
// a wave waits for one store round trip per group and not per row.  Worth 3 % at
// 8192 x 5120 bf16 (56.7 -> 55.1 us on MI355X): with 2.5 waves per SIMD the kernel is
// bound by its arithmetic (about 24 operations per element) and by how little there is to
// hide latency with, not by the memory system.  Shorter bands do not help (32 rows:
// 68 us; the column sums then cost more than the better balance gains).  Rows of different
// groups never overlap, so dZ may still alias dY.
constexpr int EW_GROUP = 4;

template <typename T, bool HAS_Z>
__global__ void __launch_bounds__(EW_TX* EW_TY)
    dgelu_dbias_kernel(const T* dY, const T* Z, T* dZ, float* partial, int64_t M,
                       int64_t N, int64_t ld) {
  typedef typename Raw8<T>::type raw;
  const int tx = threadIdx.x % EW_TX, ty = threadIdx.x / EW_TX;
  const int64_t col = (int64_t)blockIdx.x * EW_COLS + tx * 8;
  const int64_t r0 = (int64_t)blockIdx.y * EW_BAND;
  int64_t r1 = r0 + EW_BAND;
  if (r1 > M) r1 = M;
  float s[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  if (col < N) {
    raw gy[EW_GROUP], gz[EW_GROUP];
    auto fetch = [&](int64_t first) {
#pragma unroll
      for (int u = 0; u < EW_GROUP; ++u) {
        const int64_t r = first + u * EW_TY;
        if (r < r1) {
          gy[u] = load_raw8(dY + r * ld + col);
          if (HAS_Z) gz[u] = load_raw8(Z + r * ld + col);
        }
      }
    };
    int64_t first = r0 + ty;
    fetch(first);
    while (first < r1) {
      float g[EW_GROUP][8];
#pragma unroll
      for (int u = 0; u < EW_GROUP; ++u) {
        widen8(gy[u], g[u]);
        if (HAS_Z) {
          float z[8];
          widen8(gz[u], z);
#pragma unroll
          for (int e = 0; e < 8; ++e) g[u][e] *= dgelu_exact(z[e]);
        }
      }
      const int64_t next = first + EW_GROUP * EW_TY;
      if (next < r1) fetch(next);
#pragma unroll
      for (int u = 0; u < EW_GROUP; ++u) {
        const int64_t r = first + u * EW_TY;
        if (r < r1) {
          // g becomes what was stored: the sum of what wgrad reads
          if (HAS_Z) store8(dZ + r * ld + col, g[u]);
#pragma unroll
          for (int e = 0; e < 8; ++e) s[e] += g[u][e];
        }
      }
      first = next;
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

template <typename T>
__global__ void __launch_bounds__(EW_TX* EW_TY)
    swiglu_fwd_kernel(const T* gate, const T* up, T* out, int64_t M, int64_t N, int64_t ld) {
  const int tx = threadIdx.x % EW_TX, ty = threadIdx.x / EW_TX;
  const int64_t col_blocks = (N + EW_COLS - 1) / EW_COLS;
  const int64_t band = blockIdx.x / col_blocks;
  const int64_t col = (int64_t)(blockIdx.x - band * col_blocks) * EW_COLS + tx * 8;
  if (col >= N) return;
  const int64_t r0 = band * SWIGLU_BAND;
  const int64_t r1 = (r0 + SWIGLU_BAND < M) ? r0 + SWIGLU_BAND : M;
  for (int64_t r = r0 + ty; r < r1; r += EW_TY) {
    const int64_t o = r * ld + col;
    float g[8], u[8];
    load8<true>(gate + o, g);
    load8<true>(up + o, u);
#pragma unroll
    for (int e = 0; e < 8; ++e) g[e] = g[e] * sigmoid_f(g[e]) * u[e];
    store8(out + o, g);
  }
}

// dgate = dout * up * silu'(gate),  dup = dout * silu(gate),
// silu'(x) = s (1 + x (1 - s)) with s = sigmoid(x).
template <typename T>
__global__ void __launch_bounds__(EW_TX* EW_TY)
    swiglu_bwd_kernel(const T* dout, const T* gate, const T* up, T* dgate, T* dup, int64_t M,
                      int64_t N, int64_t ld, int64_t ld_out) {
  const int tx = threadIdx.x % EW_TX, ty = threadIdx.x / EW_TX;
  const int64_t col_blocks = (N + EW_COLS - 1) / EW_COLS;
  const int64_t band = blockIdx.x / col_blocks;
  const int64_t col = (int64_t)(blockIdx.x - band * col_blocks) * EW_COLS + tx * 8;
  if (col >= N) return;
  const int64_t r0 = band * SWIGLU_BAND;
  const int64_t r1 = (r0 + SWIGLU_BAND < M) ? r0 + SWIGLU_BAND : M;
  for (int64_t r = r0 + ty; r < r1; r += EW_TY) {
    const int64_t o = r * ld + col;
    float d[8], g[8], u[8], dg[8], du[8];
    load8<true>(dout + o, d);
    load8<true>(gate + o, g);
    load8<true>(up + o, u);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float sg = sigmoid_f(g[e]);
      du[e] = d[e] * g[e] * sg;
      dg[e] = d[e] * u[e] * sg * (1.0f + g[e] * (1.0f - sg));
    }
    store8(dgate + r * ld_out + col, dg);
    store8(dup + r * ld_out + col, du);
  }
}

}  // namespace

int launch_swiglu_fwd(const void* gate, const void* up, void* out, int dtype, int64_t M,
                      int64_t N, int64_t ld, hipStream_t stream) {
  const int64_t bands = (M + SWIGLU_BAND - 1) / SWIGLU_BAND;
  const int64_t blocks = bands * ((N + EW_COLS - 1) / EW_COLS);
  if (blocks > 0x7fffffffLL) {
    set_error("swiglu: too many elements (%lld x %lld)", (long long)M, (long long)N);
    return AXN_ELIMIT;
  }
  const dim3 grid((unsigned)blocks), block(EW_TX * EW_TY);
  if (dtype == AXN_F32)
    hipLaunchKernelGGL(swiglu_fwd_kernel<float>, grid, block, 0, stream, (const float*)gate,
                       (const float*)up, (float*)out, M, N, ld);
  else if (dtype == AXN_F16)
    hipLaunchKernelGGL(swiglu_fwd_kernel<_Float16>, grid, block, 0, stream, (const _Float16*)gate,
                       (const _Float16*)up, (_Float16*)out, M, N, ld);
  else
    hipLaunchKernelGGL(swiglu_fwd_kernel<uint16_t>, grid, block, 0, stream, (const uint16_t*)gate,
                       (const uint16_t*)up, (uint16_t*)out, M, N, ld);
  AXN_HIP_TRY(hipGetLastError());
  return AXN_OK;
}

int launch_swiglu_bwd(const void* dout, const void* gate, const void* up, void* dgate, void* dup,
                      int dtype, int64_t M, int64_t N, int64_t ld, int64_t ld_out,
                      hipStream_t stream) {
  const int64_t bands = (M + SWIGLU_BAND - 1) / SWIGLU_BAND;
  const int64_t blocks = bands * ((N + EW_COLS - 1) / EW_COLS);
  if (blocks > 0x7fffffffLL) {
    set_error("swiglu: too many elements (%lld x %lld)", (long long)M, (long long)N);
    return AXN_ELIMIT;
  }
  const dim3 grid((unsigned)blocks), block(EW_TX * EW_TY);
  if (dtype == AXN_F32)
    hipLaunchKernelGGL(swiglu_bwd_kernel<float>, grid, block, 0, stream, (const float*)dout,
                       (const float*)gate, (const float*)up, (float*)dgate, (float*)dup, M, N, ld, ld_out);
  else if (dtype == AXN_F16)
    hipLaunchKernelGGL(swiglu_bwd_kernel<_Float16>, grid, block, 0, stream, (const _Float16*)dout,
                       (const _Float16*)gate, (const _Float16*)up, (_Float16*)dgate,
                       (_Float16*)dup, M, N, ld, ld_out);
  else
    hipLaunchKernelGGL(swiglu_bwd_kernel<uint16_t>, grid, block, 0, stream, (const uint16_t*)dout,
                       (const uint16_t*)gate, (const uint16_t*)up, (uint16_t*)dgate,
                       (uint16_t*)dup, M, N, ld, ld_out);
  AXN_HIP_TRY(hipGetLastError());
  return AXN_OK;
}

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
  } else if (dtype == AXN_F16) {
    const _Float16 *y = (const _Float16*)dY, *z = (const _Float16*)Z;
    if (Z != nullptr)
      hipLaunchKernelGGL((dgelu_dbias_kernel<_Float16, true>), grid, block, 0, stream, y, z,
                         (_Float16*)dZ, partial, M, N, ld);
    else
      hipLaunchKernelGGL((dgelu_dbias_kernel<_Float16, false>), grid, block, 0, stream, y, z,
                         (_Float16*)dZ, partial, M, N, ld);
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
