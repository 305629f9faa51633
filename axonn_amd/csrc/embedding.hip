// Embedding table lookup and its dense weight gradient for gfx950.
//
// Forward is a row gather, out[t, :] = W[ids[t], :]: one wave per 64 x 16 bytes of
// an output row, 16-byte loads and stores.
//
// Backward is dW[v, :] (+)= sum over the tokens t with ids[t] == v of dY[t, :].
// It is written as a gather as well, so that it needs no floating-point atomics
// and its result does not depend on the order in which workgroups run:
//   1. the token positions are sorted by id (stable LSD radix sort over the bits
//      of the vocabulary size; rocPRIM's device routine - the one library call);
//   2. the first sorted slot of every id present is recorded in row_start[V];
//   3. one wave per 64 x 16 bytes of a dW row walks that row's run of sorted
//      slots, adds the dY rows in ascending token order in fp32 and stores the
//      row once; rows no token names are stored as zeros (beta = 0) or left alone
//      (beta = 1).  Every dW byte is written exactly once and never read unless
//      beta = 1, so a fresh gradient needs no separate clear.
// The max_norm renormalisation of the looked-up rows reuses steps 1 and 2: one
// wave per row that occurs, so a row named by many tokens is scaled once.
#include "axn_internal.h"

#include <cstring>
#include <rocprim/device/device_radix_sort.hpp>

namespace axn {
namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int WAVES_PER_BLOCK = 4;
// LDS the weight-gradient kernel reserves per workgroup and never touches: 36 KB hold it at
// 16 waves per CU, where its stores stream best (all 32 resident: 263 us at 16384 tokens x 2048
// into 128256 rows; 16 to 20: 238 us; 12: 323 us; measured on MI355X).
constexpr int EMB_BWD_LDS = 36864;

// ---- forward ----------------------------------------------------------------
// Rows are moved as opaque 16-byte pieces: the element type only sets how many
// pieces a row has.  `pieces` = row bytes / 16, ld* in 16-byte pieces.
__global__ void __launch_bounds__(64 * WAVES_PER_BLOCK)
    embedding_fwd_kernel(const int64_t* __restrict__ ids, const u32x4* __restrict__ W,
                         u32x4* __restrict__ out, int64_t T, int64_t V, int64_t pieces,
                         int64_t ldw, int64_t ldo, int units_per_row, int* status) {
  const int lane = threadIdx.x & 63;
  const int64_t unit = (int64_t)blockIdx.x * WAVES_PER_BLOCK + (threadIdx.x >> 6);
  const int64_t t = unit / units_per_row;
  if (t >= T) return;
  const int64_t piece = (unit % units_per_row) * 64 + lane;
  if (piece >= pieces) return;
  const int64_t id = ids[t];
  u32x4 v = {0u, 0u, 0u, 0u};
  if (id >= 0 && id < V)
    v = W[id * ldw + piece];
  else if (status != nullptr && piece == 0)
    *status = 1;
  __builtin_nontemporal_store(v, out + t * ldo + piece);
}

// ---- sorting the token positions by id ---------------------------------------
// keys[i] = ids[i] (V for an id outside [0, V): those sort behind every row),
// vals[i] = i, row_start[v] = -1, status = 0.
__global__ void __launch_bounds__(256)
    embedding_keys_kernel(const int64_t* __restrict__ ids, int* __restrict__ keys,
                          int* __restrict__ vals, int* __restrict__ row_start, int* status,
                          int64_t T, int64_t V) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < T) {
    const int64_t id = ids[i];
    keys[i] = (id >= 0 && id < V) ? (int)id : (int)V;
    vals[i] = (int)i;
  }
  if (i < V) row_start[i] = -1;
  if (i == 0) *status = 0;
}

__global__ void __launch_bounds__(256)
    embedding_row_start_kernel(const int* __restrict__ keys, int* __restrict__ row_start,
                               int* status, int64_t T, int64_t V) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= T) return;
  const int k = keys[i];
  if (i != 0 && keys[i - 1] == k) return;
  if (k < V)
    row_start[k] = (int)i;
  else
    *status = 1;
}

// ---- backward ------------------------------------------------------------------
// One 16-byte vector of a table row as fp32 values.
// One 16-byte store, non-temporal and written through (nt + sc1): the dense weight gradient
// is written once, row after row, and read much later.  (The s_nop: the wait states a store
// of more than 8 bytes needs before its data registers are written again are the
// compiler's to insert for its own stores, not for this one.)
template <typename V>
__device__ __forceinline__ void store_through(V v, void* p) {
  static_assert(sizeof(V) == 16, "one 16-byte store");
  asm volatile("global_store_dwordx4 %0, %1, off sc1 nt\n\ts_nop 1" ::"v"(p), "v"(v) : "memory");
}

template <typename T>
struct Vec;
template <>
struct Vec<float> {
  static constexpr int N = 4;
  static __device__ __forceinline__ void load_cached(const float* p, float (&x)[4]) {
    const f32x4 v = *(const f32x4*)p;
#pragma unroll
    for (int e = 0; e < 4; ++e) x[e] = v[e];
  }
  static __device__ __forceinline__ void store(float* p, const float (&x)[4]) {
    store_through(f32x4{x[0], x[1], x[2], x[3]}, p);
  }
  static __device__ __forceinline__ void store_cached(float* p, const float (&x)[4]) {
    *(f32x4*)p = f32x4{x[0], x[1], x[2], x[3]};
  }
};
template <>
struct Vec<uint16_t> {
  static constexpr int N = 8;
  static __device__ __forceinline__ void load_cached(const uint16_t* p, float (&x)[8]) {
    const bf16x8 v = *(const bf16x8*)p;
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] = (float)v[e];
  }
  static __device__ __forceinline__ void store(uint16_t* p, const float (&x)[8]) {
    bf16x8 v;
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = (__bf16)x[e];
    store_through(v, p);
  }
  static __device__ __forceinline__ void store_cached(uint16_t* p, const float (&x)[8]) {
    bf16x8 v;
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = (__bf16)x[e];
    *(bf16x8*)p = v;
  }
};

template <>
struct Vec<_Float16> {
  static constexpr int N = 8;
  typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
  static __device__ __forceinline__ void load_cached(const _Float16* p, float (&x)[8]) {
    const f16x8 v = *(const f16x8*)p;
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] = (float)v[e];
  }
  static __device__ __forceinline__ void store(_Float16* p, const float (&x)[8]) {
    f16x8 v;
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = (_Float16)x[e];
    store_through(v, p);
  }
  static __device__ __forceinline__ void store_cached(_Float16* p, const float (&x)[8]) {
    f16x8 v;
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = (_Float16)x[e];
    *(f16x8*)p = v;
  }
};

// Loads VEC consecutive elements as fp32 (VEC = 4 or 8), 16 bytes per instruction
// where the type allows.  Gradient rows are read once: non-temporal.
template <int VEC>
__device__ __forceinline__ void load_row_piece(const float* p, float (&x)[VEC]) {
#pragma unroll
  for (int h = 0; h < VEC / 4; ++h) {
    const f32x4 v = __builtin_nontemporal_load((const f32x4*)p + h);
#pragma unroll
    for (int e = 0; e < 4; ++e) x[4 * h + e] = v[e];
  }
}
template <int VEC>
__device__ __forceinline__ void load_row_piece(const uint16_t* p, float (&x)[VEC]) {
  typedef __bf16 bf16xv __attribute__((ext_vector_type(VEC)));
  const bf16xv v = __builtin_nontemporal_load((const bf16xv*)p);
#pragma unroll
  for (int e = 0; e < VEC; ++e) x[e] = (float)v[e];
}
template <int VEC>
__device__ __forceinline__ void add_old(const float* p, float (&x)[VEC]) {
  const f32x4 v = *(const f32x4*)p;
#pragma unroll
  for (int e = 0; e < 4; ++e) x[e] += v[e];
}
template <int VEC>
__device__ __forceinline__ void add_old(const uint16_t* p, float (&x)[VEC]) {
  const bf16x8 v = *(const bf16x8*)p;
#pragma unroll
  for (int e = 0; e < 8; ++e) x[e] += (float)v[e];
}

// One wave per (row, U x 64 x VEC columns): VEC = one 16-byte store of the dW type
// per lane, U such pieces per lane, 64 x VEC columns apart, so that a wave has U
// independent loads in flight per gradient row and U KiB of stores behind one
// look-up of row_start (with one piece per wave the 8192 resident waves of the chip
// covered 8 MB per memory latency: 4.2 TB/s on a gradient that is mostly zeros).
template <typename TY, typename TW, int U>
__global__ void __launch_bounds__(64 * WAVES_PER_BLOCK)
    embedding_bwd_kernel(const int* __restrict__ keys, const int* __restrict__ vals,
                         const int* __restrict__ row_start, const TY* __restrict__ dY, TW* dW,
                         int64_t T, int64_t V, int64_t H, int64_t lddy, int64_t lddw,
                         int units_per_row, int64_t padding_idx, int scale_by_freq, int beta) {
  constexpr int VEC = 16 / (int)sizeof(TW);
  const int lane = threadIdx.x & 63;
  const int64_t unit = (int64_t)blockIdx.x * WAVES_PER_BLOCK + (threadIdx.x >> 6);
  const int64_t row = unit / units_per_row;
  if (row >= V) return;
  const int64_t col0 = ((unit % units_per_row) * U * 64 + lane) * VEC;
  float acc[U][VEC];
#pragma unroll
  for (int u = 0; u < U; ++u)
#pragma unroll
    for (int q = 0; q < VEC; ++q) acc[u][q] = 0.f;
  const int s = row_start[row];
  if (s >= 0 && row != padding_idx) {
    float inv = 1.0f;
    if (scale_by_freq) {
      int e = s + 1;
      while (e < T && keys[e] == (int)row) ++e;
      inv = 1.0f / (float)(e - s);
    }
    for (int j = s; j < T; ++j) {
      if (j != s && keys[j] != (int)row) break;
      const TY* src = dY + (int64_t)vals[j] * lddy + col0;
      float g[U][VEC];
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (col0 + u * 64 * VEC < H) load_row_piece<VEC>(src + u * 64 * VEC, g[u]);
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (col0 + u * 64 * VEC < H) {
#pragma unroll
          for (int q = 0; q < VEC; ++q)
            acc[u][q] = scale_by_freq ? __fmaf_rn(g[u][q], inv, acc[u][q]) : acc[u][q] + g[u][q];
        }
    }
  } else if (beta != 0) {
    return;  // nothing to add to this row
  }
  TW* dst = dW + row * lddw + col0;
#pragma unroll
  for (int u = 0; u < U; ++u) {
    if (col0 + u * 64 * VEC >= H) break;
    if (beta != 0) add_old<VEC>(dst + u * 64 * VEC, acc[u]);
    Vec<TW>::store(dst + u * 64 * VEC, acc[u]);
  }
}

// ---- max_norm ------------------------------------------------------------------
// One wave per row of the table; rows no token names are left alone.
// norm = (sum |w|^p)^(1/p) in fp32; rows with norm > max_norm are scaled by
// max_norm / (norm + 1e-7), as torch.embedding_renorm_ does.
template <typename TW>
__global__ void __launch_bounds__(64 * WAVES_PER_BLOCK)
    embedding_renorm_kernel(const int* __restrict__ row_start, TW* W, int64_t V, int64_t H,
                            int64_t ldw, float max_norm, float norm_type) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * WAVES_PER_BLOCK + (threadIdx.x >> 6);
  if (row >= V) return;
  if (row_start[row] < 0) return;
  constexpr int N = Vec<TW>::N;
  TW* w = W + row * ldw;
  float sum = 0.f;
  for (int64_t c = (int64_t)lane * N; c < H; c += 64 * N) {
    float x[N];
    Vec<TW>::load_cached(w + c, x);
#pragma unroll
    for (int e = 0; e < N; ++e) {
      const float a = fabsf(x[e]);
      if (norm_type == 1.0f)
        sum += a;
      else if (norm_type == 2.0f)
        sum = fmaf(a, a, sum);
      else
        sum += powf(a, norm_type);
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
  float norm;
  if (norm_type == 1.0f)
    norm = sum;
  else if (norm_type == 2.0f)
    norm = sqrtf(sum);
  else
    norm = powf(sum, 1.0f / norm_type);
  if (!(norm > max_norm)) return;
  const float scale = max_norm / (norm + 1e-7f);
  for (int64_t c = (int64_t)lane * N; c < H; c += 64 * N) {
    float x[N];
    Vec<TW>::load_cached(w + c, x);
#pragma unroll
    for (int e = 0; e < N; ++e) x[e] *= scale;
    Vec<TW>::store_cached(w + c, x);   // the lookup reads the row next
  }
}

// ---- workspace ---------------------------------------------------------------
constexpr size_t ALIGN = 256;
inline size_t round_up(size_t n) { return (n + ALIGN - 1) / ALIGN * ALIGN; }

struct Workspace {
  int *keys_a, *keys_b, *vals_a, *vals_b, *row_start, *status;
  void* sort_temp;
  size_t sort_temp_bytes;
};

// The sort's own temporary storage is bounded here by arithmetic, so that the size
// query needs no device: 16 bytes per token and 4 MiB cover rocPRIM's histograms
// and block descriptors with a wide margin; the launch checks the real need.
inline size_t sort_temp_bound(int64_t T) { return round_up((size_t)T * 16 + (4u << 20)); }

inline bool carve(void* ws, size_t ws_bytes, int64_t T, int64_t V, Workspace* out) {
  char* p = (char*)ws;
  const size_t tok = round_up((size_t)T * sizeof(int));
  out->keys_a = (int*)p; p += tok;
  out->keys_b = (int*)p; p += tok;
  out->vals_a = (int*)p; p += tok;
  out->vals_b = (int*)p; p += tok;
  out->row_start = (int*)p; p += round_up((size_t)V * sizeof(int));
  out->status = (int*)p; p += ALIGN;
  out->sort_temp = p;
  out->sort_temp_bytes = sort_temp_bound(T);
  return (size_t)(p - (char*)ws) + out->sort_temp_bytes <= ws_bytes;
}

int bits_for(int64_t V) {  // keys run over [0, V]
  int b = 1;
  while ((1LL << b) <= V) ++b;
  return b;
}

// Fills ws with the sorted (key, position) pairs and row_start; on return
// *keys and *vals point at the sorted arrays.
int sort_token_positions(const int64_t* ids, int64_t T, int64_t V, const Workspace& w,
                         const int** keys, const int** vals, hipStream_t stream) {
  const int64_t span = T > V ? T : V;
  hipLaunchKernelGGL(embedding_keys_kernel, dim3((unsigned)((span + 255) / 256)), dim3(256), 0,
                     stream, ids, w.keys_a, w.vals_a, w.row_start, w.status, T, V);
  AXN_HIP_TRY(hipGetLastError());
  *keys = w.keys_a;
  *vals = w.vals_a;
  if (T == 0) return AXN_OK;
  rocprim::double_buffer<int> k(w.keys_a, w.keys_b), v(w.vals_a, w.vals_b);
  size_t need = 0;
  AXN_HIP_TRY(rocprim::radix_sort_pairs(nullptr, need, k, v, (size_t)T, 0, (unsigned)bits_for(V),
                                        stream));
  if (need > w.sort_temp_bytes) {
    set_error("embedding: the sort needs %zu bytes of temporary storage, %zu reserved", need,
              w.sort_temp_bytes);
    return AXN_ELIMIT;
  }
  need = w.sort_temp_bytes;
  AXN_HIP_TRY(rocprim::radix_sort_pairs(w.sort_temp, need, k, v, (size_t)T, 0,
                                        (unsigned)bits_for(V), stream));
  *keys = k.current();
  *vals = v.current();
  hipLaunchKernelGGL(embedding_row_start_kernel, dim3((unsigned)((T + 255) / 256)), dim3(256), 0,
                     stream, *keys, w.row_start, w.status, T, V);
  AXN_HIP_TRY(hipGetLastError());
  return AXN_OK;
}

}  // namespace

size_t embedding_workspace_bytes(int64_t T, int64_t V) {
  if (T < 0 || V <= 0) return 0;
  return 4 * round_up((size_t)T * sizeof(int)) + round_up((size_t)V * sizeof(int)) + ALIGN +
         sort_temp_bound(T);
}

int launch_embedding_fwd(const int64_t* ids, const void* W, void* out, int elem_bytes, int64_t T,
                         int64_t V, int64_t H, int64_t ldw, int64_t ldo, int* status,
                         hipStream_t stream) {
  const int per_piece = 16 / elem_bytes;
  const int64_t pieces = H / per_piece;
  const int upr = (int)((pieces + 63) / 64);
  const int64_t blocks = (T * upr + WAVES_PER_BLOCK - 1) / WAVES_PER_BLOCK;
  if (blocks == 0) return AXN_OK;
  if (blocks >= (1LL << 31)) {
    set_error("embedding_fwd: too many tokens x columns (%lld blocks)", (long long)blocks);
    return AXN_ELIMIT;
  }
  hipLaunchKernelGGL(embedding_fwd_kernel, dim3((unsigned)blocks), dim3(64 * WAVES_PER_BLOCK), 0,
                     stream, ids, (const u32x4*)W, (u32x4*)out, T, V, pieces, ldw / per_piece,
                     ldo / per_piece, upr, status);
  AXN_HIP_TRY(hipGetLastError());
  return AXN_OK;
}

int launch_embedding_bwd(const int64_t* ids, const void* dY, void* dW, int dy_dtype, int dw_dtype,
                         int64_t T, int64_t V, int64_t H, int64_t lddy, int64_t lddw,
                         int64_t padding_idx, int scale_by_freq, int beta, void* ws,
                         size_t ws_bytes, hipStream_t stream) {
  Workspace w;
  if (ws == nullptr || !carve(ws, ws_bytes, T, V, &w)) {
    set_error("embedding_bwd: workspace too small (%zu bytes given, %zu needed)", ws_bytes,
              embedding_workspace_bytes(T, V));
    return AXN_EINVAL;
  }
  // pieces of 64 lanes x one 16-byte dW vector per row; up to 4 of them per wave
  const int vec = dw_dtype == AXN_F32 ? 4 : 8;
  const int64_t pieces = (H / vec + 63) / 64;
  const int U = pieces >= 4 ? 4 : pieces >= 2 ? 2 : 1;
  const int upr = (int)((pieces + U - 1) / U);
  const int64_t blocks = (V * upr + WAVES_PER_BLOCK - 1) / WAVES_PER_BLOCK;
  if (blocks >= (1LL << 31)) {
    set_error("embedding_bwd: too many rows x columns (%lld blocks)", (long long)blocks);
    return AXN_ELIMIT;
  }
  const int *keys = nullptr, *vals = nullptr;
  int rc = sort_token_positions(ids, T, V, w, &keys, &vals, stream);
  if (rc) return rc;
  const dim3 grid((unsigned)blocks), block(64 * WAVES_PER_BLOCK);
#define AXN_EMB_BWD_U(TY, TW, UU)                                                               \
  hipLaunchKernelGGL((embedding_bwd_kernel<TY, TW, UU>), grid, block, EMB_BWD_LDS, stream, keys, vals,    \
                     w.row_start, (const TY*)dY, (TW*)dW, T, V, H, lddy, lddw, upr, padding_idx, \
                     scale_by_freq, beta)
#define AXN_EMB_BWD(TY, TW)                 \
  do {                                      \
    if (U == 4)                             \
      AXN_EMB_BWD_U(TY, TW, 4);             \
    else if (U == 2)                        \
      AXN_EMB_BWD_U(TY, TW, 2);             \
    else                                    \
      AXN_EMB_BWD_U(TY, TW, 1);             \
  } while (0)
  if (dy_dtype == AXN_F32 && dw_dtype == AXN_F32)
    AXN_EMB_BWD(float, float);
  else if (dy_dtype == AXN_F32)
    AXN_EMB_BWD(float, uint16_t);
  else if (dw_dtype == AXN_F32)
    AXN_EMB_BWD(uint16_t, float);
  else
    AXN_EMB_BWD(uint16_t, uint16_t);
#undef AXN_EMB_BWD_U
#undef AXN_EMB_BWD
  AXN_HIP_TRY(hipGetLastError());
  return AXN_OK;
}

int launch_embedding_renorm(const int64_t* ids, void* W, int dtype, int64_t T, int64_t V,
                            int64_t H, int64_t ldw, float max_norm, float norm_type, void* ws,
                            size_t ws_bytes, hipStream_t stream) {
  Workspace w;
  if (ws == nullptr || !carve(ws, ws_bytes, T, V, &w)) {
    set_error("embedding_renorm: workspace too small (%zu bytes given, %zu needed)", ws_bytes,
              embedding_workspace_bytes(T, V));
    return AXN_EINVAL;
  }
  const int *keys = nullptr, *vals = nullptr;
  int rc = sort_token_positions(ids, T, V, w, &keys, &vals, stream);
  if (rc) return rc;
  const dim3 grid((unsigned)((V + WAVES_PER_BLOCK - 1) / WAVES_PER_BLOCK)),
      block(64 * WAVES_PER_BLOCK);
  if (dtype == AXN_F32)
    hipLaunchKernelGGL(embedding_renorm_kernel<float>, grid, block, 0, stream, w.row_start,
                       (float*)W, V, H, ldw, max_norm, norm_type);
  else if (dtype == AXN_F16)
    hipLaunchKernelGGL(embedding_renorm_kernel<_Float16>, grid, block, 0, stream, w.row_start,
                       (_Float16*)W, V, H, ldw, max_norm, norm_type);
  else
    hipLaunchKernelGGL(embedding_renorm_kernel<uint16_t>, grid, block, 0, stream, w.row_start,
                       (uint16_t*)W, V, H, ldw, max_norm, norm_type);
  AXN_HIP_TRY(hipGetLastError());
  return AXN_OK;
}

}  // namespace axn
