// Embedding table lookup and its dense weight gradient for gfx950.
//
// Forward is a row gather, out[t, :] = W[ids[t], :]: one wave per 64 x 16 bytes of
// an output row, 16-byte loads and stores.
//
// Backward is dW[v, :] (+)= sum over the tokens t with ids[t] == v of dY[t, :].
// It is written as a gather as well, so that it needs no floating-point atomics
// and its result does not depend on the order in which workgroups run:
//   1. the token positions are sorted by id (stable LSD radix sort over the bits
//      of the vocabulary size, kernels below: no library call, no atomics on
//      floating-point data, nothing but kernel launches);
//   2. the first sorted slot of every id present is recorded in row_start[V] (by the
//      sort's last pass: the smallest slot a row's tokens land in);
//   3. one wave per 64 x 16 bytes of a dW row walks that row's run of sorted
//      slots, adds the dY rows in ascending token order in fp32 and stores the
//      row once; rows no token names are stored as zeros (beta = 0) or left alone
//      (beta = 1).  Every dW byte is written exactly once and never read unless
//      beta = 1, so a fresh gradient needs no separate clear.
// The max_norm renormalisation of the looked-up rows reuses steps 1 and 2: one
// wave per row that occurs, so a row named by many tokens is scaled once.
#include "axn_internal.h"

#include <cstring>

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
// Stable least-significant-digit radix sort of (key, position) pairs, keys over [0, V]
// (V for an id outside [0, V): those sort behind every row), in 1 to 4 passes of at most
// 10 bits.  A workgroup of 4 waves owns 256 G consecutive slots, wave w the w-th quarter of
// them (G = 2 for batches up to 2^15 tokens, where short pieces give the sort more waves,
// G = 8 beyond, where they keep the count arrays small).  Per pass:
//   counts   hist[digit][workgroup] = slots of the workgroup whose key has that digit (pass
//            0: counted by the kernel that writes the keys; later passes: counted by the
//            previous pass's scatter with integer atomics, which add up to the same counts
//            in any order)
//   scan     exclusive prefix sum over the digit-major array: where the workgroup's slots
//            of a digit go (a launch of its own beyond 2^17 tokens; up to there the array is
//            small and every workgroup of the scatter sums what lies in front of it itself)
//   scatter  every wave counts the digits of its quarter, which places the quarters of a
//            digit one behind the other; then a wave walks its quarter 64 slots at a time
//            in slot order: lanes with equal digits find one another with one ballot per
//            digit bit, and a slot goes to (the running count of its digit) + (equal-digit
//            lanes before it).  Slots of equal digit keep their order, which is what makes
//            the sort stable and the order of every row's tokens ascending.
constexpr int SORT_SHORT_BATCH = 1 << 15;   // tokens up to which a wave's quarter is 128 slots
constexpr int SORT_FUSED_BATCH = 1 << 17;   // tokens (at most 64 workgroups) up to which no scan is launched
constexpr int SORT_WAVES = 4;        // waves per workgroup
constexpr int SORT_MAX_BITS = 10;    // digit width: 1024 counters per wave in LDS
constexpr int SORT_MAX_PASSES = 4;

struct SortPlan {
  int passes;
  int bits[SORT_MAX_PASSES], shift[SORT_MAX_PASSES];
  int groups;                         // 64-slot groups per wave
  bool fused_scan;                    // the scatter derives the prefix sums itself
  int64_t nblk;                       // workgroups = units of the count arrays
  size_t hist_ofs[SORT_MAX_PASSES];   // in ints, from the start of the histogram area
  size_t hist_ints;
};

__device__ __forceinline__ int key_of_id(int64_t id, int64_t V) {
  return (id >= 0 && id < V) ? (int)id : (int)V;
}

// keys[i], vals[i] = i, pass 0's counts; row_start[v] = -1, status = 0, the later passes'
// counts cleared.
template <int G>
__global__ void __launch_bounds__(64 * SORT_WAVES)
    embedding_sort_prepare_kernel(const int64_t* __restrict__ ids, int* __restrict__ keys,
                                  int* __restrict__ vals, int* __restrict__ row_start, int* status,
                                  int* __restrict__ hist0, int* __restrict__ hist_rest,
                                  int64_t hist_rest_ints, int64_t T, int64_t V, int64_t nblk,
                                  int bits0, bool block_major) {
  __shared__ int cnt[1 << SORT_MAX_BITS];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int64_t gtid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t nthreads = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = gtid; i < hist_rest_ints; i += nthreads) hist_rest[i] = 0;
  for (int64_t i = gtid; i < V; i += nthreads) row_start[i] = -1;
  if (gtid == 0) *status = 0;
  const int nd = 1 << bits0;
  for (int d = threadIdx.x; d < nd; d += 64 * SORT_WAVES) cnt[d] = 0;
  __syncthreads();
  const int64_t blk = blockIdx.x;
  if (blk < nblk) {
    const int64_t first = (blk * SORT_WAVES + w) * (64 * G);
    int64_t id[G];   // all loads of the wave in flight at once
#pragma unroll
    for (int g = 0; g < G; ++g) {
      const int64_t i = first + g * 64 + lane;
      id[g] = i < T ? ids[i] : 0;
    }
#pragma unroll
    for (int g = 0; g < G; ++g) {
      const int64_t i = first + g * 64 + lane;
      if (i < T) {
        const int key = key_of_id(id[g], V);
        keys[i] = key;
        vals[i] = (int)i;
        atomicAdd(&cnt[key & (nd - 1)], 1);
      }
    }
  }
  __syncthreads();
  if (blk < nblk)
    for (int d = threadIdx.x; d < nd; d += 64 * SORT_WAVES)
      hist0[block_major ? blk * nd + d : (int64_t)d * nblk + blk] = cnt[d];
}

// Inclusive prefix sum across the 64 lanes in six data-parallel-primitive adds (no LDS
// round trip): shifts by 1, 2, 4, 8 inside the rows of 16 lanes (a lane the shift leaves
// without a source adds 0), then lane 15's total into rows 1 and 3, then lane 31's into
// rows 2 and 3.
__device__ __forceinline__ int wave_inclusive_sum(int v) {
  v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, true);    // row_shr:1
  v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, true);    // row_shr:2
  v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, true);    // row_shr:4
  v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, true);    // row_shr:8
  v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false);   // row_bcast:15 into rows 1, 3
  v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false);   // row_bcast:31 into rows 2, 3
  return v;
}

// In-place exclusive prefix sum over n ints, one workgroup of 1024 threads: tiles of 65536
// entries, 4096 consecutive ones per wave held in registers as 16 rows of 64 lanes x 4 (every
// access of a wave covers 1 KiB of consecutive bytes, every load of a tile in flight at
// once, nothing read twice); rows are scanned across the lanes, the rows' totals along the
// wave, the waves' totals across the workgroup, and a running total goes from tile to tile.
__global__ void __launch_bounds__(1024) embedding_sort_scan_kernel(int* __restrict__ h, int64_t n) {
  typedef int i32x4 __attribute__((ext_vector_type(4)));
  constexpr int ROWS = 16;                // 16-byte vectors per thread and tile
  __shared__ int wave_total[16];
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  int carry = 0;
  for (int64_t tile = 0; tile < n; tile += 1024 * ROWS * 4) {
    const int64_t lo = tile + (int64_t)w * (64 * ROWS * 4) + lane * 4;
    i32x4 v[ROWS];
#pragma unroll
    for (int j = 0; j < ROWS; ++j) {
      const int64_t i = lo + 256 * j;
      if (i + 3 < n) {
        v[j] = *(const i32x4*)(h + i);
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) v[j][e] = i + e < n ? h[i + e] : 0;
      }
    }
    int excl[ROWS];   // sum of everything of this wave's part in front of v[j]
    int wave_sum = 0;
#pragma unroll
    for (int j = 0; j < ROWS; ++j) {
      const int s = v[j][0] + v[j][1] + v[j][2] + v[j][3];
      const int incl = wave_inclusive_sum(s);
      excl[j] = wave_sum + incl - s;
      wave_sum += __builtin_amdgcn_readlane(incl, 63);
    }
    __syncthreads();   // the previous tile's totals have been read
    if (lane == 0) wave_total[w] = wave_sum;
    __syncthreads();
    int before = carry, all = 0;
    for (int k = 0; k < 16; ++k) {
      if (k < w) before += wave_total[k];
      all += wave_total[k];
    }
#pragma unroll
    for (int j = 0; j < ROWS; ++j) {
      const int64_t i = lo + 256 * j;
      i32x4 o;
      o[0] = before + excl[j];
      o[1] = o[0] + v[j][0];
      o[2] = o[1] + v[j][1];
      o[3] = o[2] + v[j][2];
      if (i + 3 < n) {
        *(i32x4*)(h + i) = o;
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (i + e < n) h[i + e] = o[e];
      }
    }
    carry += all;
  }
}

// SCANNED: `base` holds the exclusive prefix sums of the counts (embedding_sort_scan_kernel
// has run); otherwise it holds the counts themselves and every workgroup derives its own
// part of the prefix sums from them - all digit-major rows in front of a digit's row and
// the row up to this workgroup - which for few workgroups costs less than a launch.
template <int G, bool SCANNED>
__global__ void __launch_bounds__(64 * SORT_WAVES)
    embedding_sort_scatter_kernel(const int* __restrict__ keys_in, const int* __restrict__ vals_in,
                                  int* __restrict__ keys_out, int* __restrict__ vals_out,
                                  const int* __restrict__ base, int* __restrict__ next_hist,
                                  int* __restrict__ row_start, int* status, int64_t T, int64_t V,
                                  int64_t nblk, int shift, int bits, int next_shift, int next_bits) {
  __shared__ int cnt[SORT_WAVES][1 << SORT_MAX_BITS];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int64_t blk = blockIdx.x;
  const int nd = 1 << bits;
  for (int d = threadIdx.x; d < SORT_WAVES * nd; d += 64 * SORT_WAVES) cnt[d / nd][d % nd] = 0;
  const int64_t first = (blk * SORT_WAVES + w) * (64 * G);
  int kreg[G], vreg[G];   // all loads of the wave in flight at once
#pragma unroll
  for (int g = 0; g < G; ++g) {
    const int64_t i = first + g * 64 + lane;
    const bool active = i < T;
    kreg[g] = active ? keys_in[i] : 0;
    vreg[g] = active ? vals_in[i] : 0;
  }
  __syncthreads();
  // the digits of this wave's quarter
#pragma unroll
  for (int g = 0; g < G; ++g)
    if (first + g * 64 + lane < T) atomicAdd(&cnt[w][(kreg[g] >> shift) & (nd - 1)], 1);
  __syncthreads();
  // counts -> first destination of each wave's slots of a digit; a thread sees to the
  // digits t, t + 256, t + 512, t + 768 (at most 1024 digits, 256 threads)
  int first_dest[4] = {0, 0, 0, 0};
  if constexpr (SCANNED) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int d = threadIdx.x + 256 * e;
      if (d < nd) first_dest[e] = base[(int64_t)d * nblk + blk];
    }
  } else {
    // The counts lie workgroup-major here ([workgroup][digit]: consecutive lanes read
    // consecutive words).  A digit's slots start behind every slot of a smaller digit (the
    // digits' totals, scanned over the workgroup in digit order) and behind the digit's
    // slots of the workgroups in front of this one.
    __shared__ int wave_total[4][SORT_WAVES];
    int tot[4] = {0, 0, 0, 0}, pre[4] = {0, 0, 0, 0};
#pragma unroll 8
    for (int64_t b = 0; b < nblk; ++b) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int d = threadIdx.x + 256 * e;
        const int c = d < nd ? base[b * nd + d] : 0;
        tot[e] += c;
        pre[e] += b < blk ? c : 0;
      }
    }
    int incl[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      incl[e] = wave_inclusive_sum(tot[e]);
      if (lane == 63) wave_total[e][w] = incl[e];
    }
    __syncthreads();
    int run = 0;   // slots of the digits in front of digit 256 e + 64 w
#pragma unroll
    for (int e = 0; e < 4; ++e) {
#pragma unroll
      for (int k = 0; k < SORT_WAVES; ++k) {
        if (k == w) first_dest[e] = run + incl[e] - tot[e] + pre[e];
        run += wave_total[e][k];
      }
    }
  }
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int d = threadIdx.x + 256 * e;
    if (d < nd) {
      int run = first_dest[e];
#pragma unroll
      for (int k = 0; k < SORT_WAVES; ++k) {
        const int c = cnt[k][d];
        cnt[k][d] = run;
        run += c;
      }
    }
  }
  __syncthreads();
  const uint64_t below = lane == 0 ? 0ull : (~0ull >> (64 - lane));
#pragma unroll
  for (int g = 0; g < G; ++g) {   // (every wave makes every trip: the barriers below)
    const bool active = first + g * 64 + lane < T;
    const int key = kreg[g];
    const int val = vreg[g];
    const int d = (key >> shift) & (nd - 1);
    uint64_t same = __ballot(active);   // the lanes whose slot has this lane's digit
    for (int b = 0; b < bits; ++b) {
      const bool bit = (d >> b) & 1;
      const uint64_t with = __ballot(active && bit);
      same &= bit ? with : ~with;
    }
    const int off = active ? cnt[w][d] : 0;
    __syncthreads();   // every lane has read its digit's count before any lane moves one on
    if (active && lane == 63 - __builtin_clzll(same)) cnt[w][d] = off + __builtin_popcountll(same);
    __syncthreads();
    if (active) {
      const int dest = off + __builtin_popcountll(same & below);
      keys_out[dest] = key;
      vals_out[dest] = val;
      if (next_hist != nullptr) {
        const int nx = (key >> next_shift) & ((1 << next_bits) - 1);
        const int64_t nb = dest / (64 * G * SORT_WAVES);
        atomicAdd(&next_hist[SCANNED ? (int64_t)nx * nblk + nb : (nb << next_bits) + nx], 1);
      } else if (key < V) {
        // last pass: the slots are final, and a row's run starts at the smallest of them
        // (row_start holds -1 = the largest unsigned value until a slot arrives)
        atomicMin((unsigned*)&row_start[key], (unsigned)dest);
      } else {
        *status = 1;   // an id outside the table
      }
    }
  }
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
  int *keys_a, *keys_b, *vals_a, *vals_b, *row_start, *status, *hist;
};

int bits_for(int64_t V) {  // keys run over [0, V]
  int b = 1;
  while ((1LL << b) <= V) ++b;
  return b;
}

// The passes of the sort: the key's bits in equal parts of at most SORT_MAX_BITS, and one
// digit-major count array [2^bits][segments] per pass.
SortPlan plan_sort(int64_t T, int64_t V) {
  SortPlan pl;
  const int total = bits_for(V);
  pl.passes = (total + SORT_MAX_BITS - 1) / SORT_MAX_BITS;
  pl.groups = T <= SORT_SHORT_BATCH ? 2 : 8;
  pl.fused_scan = T <= SORT_FUSED_BATCH;
  const int64_t per_block = 64 * pl.groups * SORT_WAVES;
  pl.nblk = (T + per_block - 1) / per_block;
  int shift = 0;
  size_t ofs = 0;
  for (int p = 0; p < SORT_MAX_PASSES; ++p) {
    pl.bits[p] = p < pl.passes ? total / pl.passes + (p < total % pl.passes ? 1 : 0) : 0;
    pl.shift[p] = shift;
    pl.hist_ofs[p] = ofs;
    shift += pl.bits[p];
    if (p < pl.passes) ofs += ((size_t)1 << pl.bits[p]) * (size_t)pl.nblk;
  }
  pl.hist_ints = ofs;
  return pl;
}

inline bool carve(void* ws, size_t ws_bytes, int64_t T, int64_t V, Workspace* out) {
  char* p = (char*)ws;
  const size_t tok = round_up((size_t)T * sizeof(int));
  out->keys_a = (int*)p; p += tok;
  out->keys_b = (int*)p; p += tok;
  out->vals_a = (int*)p; p += tok;
  out->vals_b = (int*)p; p += tok;
  out->row_start = (int*)p; p += round_up((size_t)V * sizeof(int));
  out->status = (int*)p; p += ALIGN;
  out->hist = (int*)p; p += round_up(plan_sort(T, V).hist_ints * sizeof(int));
  return (size_t)(p - (char*)ws) <= ws_bytes;
}

// Fills ws with the sorted (key, position) pairs and row_start; on return
// *keys and *vals point at the sorted arrays.
int sort_token_positions(const int64_t* ids, int64_t T, int64_t V, const Workspace& w,
                         const int** keys, const int** vals, hipStream_t stream) {
  const SortPlan pl = plan_sort(T, V);
  if (pl.nblk >= (1LL << 31) ||
      pl.hist_ints >= ((size_t)1 << 40)) {
    set_error("embedding: too many tokens to sort (%lld)", (long long)T);
    return AXN_ELIMIT;
  }
  const dim3 block(64 * SORT_WAVES);
  const int64_t seg_blocks = pl.nblk;
  // (at least enough workgroups to fill row_start at a good rate when the batch is short)
  int64_t fill_blocks = (V + 4 * 256 - 1) / (4 * 256);
  if (fill_blocks > 1024) fill_blocks = 1024;
  const int64_t prep_blocks = seg_blocks > fill_blocks ? seg_blocks : (fill_blocks > 0 ? fill_blocks : 1);
  int* hist_rest = w.hist + pl.hist_ofs[1];
  const int64_t hist_rest_ints = pl.passes > 1 ? (int64_t)(pl.hist_ints - pl.hist_ofs[1]) : 0;
  if (pl.groups == 2)
    hipLaunchKernelGGL(embedding_sort_prepare_kernel<2>, dim3((unsigned)prep_blocks), block, 0, stream, ids,
                       w.keys_a, w.vals_a, w.row_start, w.status, w.hist, hist_rest, hist_rest_ints, T, V,
                       pl.nblk, pl.bits[0], pl.fused_scan);
  else
    hipLaunchKernelGGL(embedding_sort_prepare_kernel<8>, dim3((unsigned)prep_blocks), block, 0, stream, ids,
                       w.keys_a, w.vals_a, w.row_start, w.status, w.hist, hist_rest, hist_rest_ints, T, V,
                       pl.nblk, pl.bits[0], pl.fused_scan);
  AXN_HIP_TRY(hipGetLastError());
  const int *kin = w.keys_a, *vin = w.vals_a;
  int *kout = w.keys_b, *vout = w.vals_b;
  if (T > 0) {
    for (int p = 0; p < pl.passes; ++p) {
      int* hist = w.hist + pl.hist_ofs[p];
      const int64_t n = ((int64_t)1 << pl.bits[p]) * pl.nblk;
      if (!pl.fused_scan) {
        hipLaunchKernelGGL(embedding_sort_scan_kernel, dim3(1), dim3(1024), 0, stream, hist, n);
        AXN_HIP_TRY(hipGetLastError());
      }
      const bool more = p + 1 < pl.passes;
      void (*scatter)(const int*, const int*, int*, int*, const int*, int*, int*, int*, int64_t, int64_t,
                      int64_t, int, int, int, int) =
          pl.fused_scan ? (pl.groups == 2 ? embedding_sort_scatter_kernel<2, false>
                                          : embedding_sort_scatter_kernel<8, false>)
                        : embedding_sort_scatter_kernel<8, true>;
      hipLaunchKernelGGL(scatter, dim3((unsigned)seg_blocks), block, 0, stream, kin, vin, kout, vout,
                         (const int*)hist, more ? w.hist + pl.hist_ofs[p + 1] : nullptr, w.row_start,
                         w.status, T, V, pl.nblk, pl.shift[p], pl.bits[p], more ? pl.shift[p + 1] : 0,
                         more ? pl.bits[p + 1] : 0);
      AXN_HIP_TRY(hipGetLastError());
      const int* tk = kin; kin = kout; kout = (int*)tk;
      const int* tv = vin; vin = vout; vout = (int*)tv;
    }
  }
  *keys = kin;
  *vals = vin;
  return AXN_OK;
}

}  // namespace

size_t embedding_workspace_bytes(int64_t T, int64_t V) {
  if (T < 0 || V <= 0) return 0;
  return 4 * round_up((size_t)T * sizeof(int)) + round_up((size_t)V * sizeof(int)) + ALIGN +
         round_up(plan_sort(T, V).hist_ints * sizeof(int));
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
