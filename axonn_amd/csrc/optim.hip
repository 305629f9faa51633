// Mixed-precision optimizer step for gfx950 (MI355X): multi-tensor, HBM
// streaming.  Three kernels share one addressing scheme:
//   mt_scan   one read pass over the low-precision gradients: overflow check
//             (axonn/inter_layer.py:435-445) + sum of squares of the unscaled
//             gradients (axonn/intra_layer/gradient_normalization.py:18-34)
//   mt_adam   one read-modify-write pass: unscale, clip, Adam on the fp32
//             master weights and moments, low-precision copy of the weights
//             (axonn/optim.py:157-190)
//   mt_scale  in-place scaling of the gradients
//             (axonn/inter_layer.py:458, gradient_normalization.py:88-93)
//
// Addressing.  The tensors of one launch (at most MT_MAX) travel in the kernel
// argument block: pointers, sizes and a prefix sum of per-tensor chunk counts.
// Workgroup b finds its tensor in that prefix sum with scalar loads from the argument
// block (binary search; the update kernel's two-step search is described there) and owns
// one chunk of consecutive elements of it.
// Tensors are views into flat buffers at arbitrary element offsets
// (axonn/utils.py:11-30), so each tensor starts with a scalar "head" of up to 63
// elements after which every pointer of the tensor is 16-byte aligned (and on a
// cache line when the buffers allow it); the body is then moved as 16-byte vectors
// (8-byte ones for 16-bit streams of the update kernel).  A
// tensor whose pointers cannot be aligned by one common head is processed with
// scalar accesses.
#include "axn_internal.h"

#include <cmath>
#include <mutex>

namespace axn {
namespace {

constexpr int MT_MAX = 64;         // tensors per launch
constexpr int MT_THREADS = 256;    // threads per workgroup
constexpr int MT_VEC = 8;          // elements per lane per step
// Elements per workgroup.  The read-only scan streams best in long runs with
// non-temporal loads; the read-modify-write update does best with one-wave workgroups
// that make one trip of ADAM_VECS 4-element vectors per lane (see mt_adam_kernel).  Both
// measured on MI355X.
constexpr int SCAN_CHUNK = 65536;
constexpr int SCALE_CHUNK = 16384;
constexpr int ADAM_VEC = 4;                     // elements per vector of the update kernel
constexpr int ADAM_THREADS = 64;                // lanes per workgroup of the update kernel
constexpr int ADAM_VECS = 1;                    // vectors per lane
constexpr int ADAM_CHUNK = ADAM_THREADS * ADAM_VEC * ADAM_VECS;
// LDS the update kernel reserves per workgroup and never touches: it bounds the
// workgroups that are resident on a CU (160 KB per CU), see mt_adam_kernel.
constexpr int ADAM_LDS = 15360;
// Cache policy bits of the update kernel's buffer accesses (1 sc0, 2 nt, 16 sc1).  Loads
// non-temporal; stores non-temporal and written through (nt + sc1): 1 to 2 % over nt
// alone, 10 % over plain stores, measured on MI355X.
constexpr int ADAM_LOAD_POLICY = 2, ADAM_STORE_POLICY = 2 | 16;
static_assert(ADAM_THREADS >= 64 && ADAM_THREADS % 64 == 0, "a tensor's scalar head (up to 63 elements) is one element per lane");
static_assert(ADAM_CHUNK % MT_VEC == 0, "chunks keep the 16-byte alignment of the tensor's body");
static_assert(ADAM_LDS <= 65536, "dynamic LDS a launch may ask for without a function attribute");

// Memory access policies, compile-time per call site.
template <bool NT, typename T>
__device__ __forceinline__ T ld(const T* p) {
  if (NT) return __builtin_nontemporal_load(p);
  return *p;
}
template <bool NT, typename T>
__device__ __forceinline__ void st(T v, T* p) {
  if (NT) __builtin_nontemporal_store(v, p); else *p = v;
}

typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;

struct MtTable {
  const void* g[MT_MAX];
  void* p[MT_MAX];
  void* m[MT_MAX];
  void* v[MT_MAX];
  void* plow[MT_MAX];
  int64_t size[MT_MAX];
  int32_t chunk_start[MT_MAX + 1];  // prefix sum of chunks per tensor
  int32_t meta[MT_MAX];             // bits 0-7: scalar elements before the aligned body;
                                    // bit 8: vector accesses allowed
  int32_t n;
  int32_t chunk;                    // elements per workgroup (multiple of MT_VEC)
};

struct ScanPartial {
  float sumsq;
  float sum;
  int32_t nonfinite;
  int32_t pad;
};

__device__ __forceinline__ int head_of(const MtTable& t, int i) { return t.meta[i] & 0xff; }
__device__ __forceinline__ bool vec_ok_of(const MtTable& t, int i) { return (t.meta[i] & 0x100) != 0; }

__device__ __forceinline__ int find_tensor(const MtTable& t, int block) {
  int lo = 0, hi = t.n;  // chunk_start[lo] <= block < chunk_start[hi]
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (t.chunk_start[mid] <= block) lo = mid; else hi = mid;
  }
  return lo;
}

template <int DT> struct Lowp;
template <> struct Lowp<AXN_BF16> {
  typedef uint16_t raw;
  __device__ static float to_float(raw x) { return __uint_as_float((uint32_t)x << 16); }
  __device__ static raw from_float(float f) {
    return __builtin_bit_cast(uint16_t, (__bf16)f);
  }
  __device__ static bool nonfinite(raw x) { return (x & 0x7F80u) == 0x7F80u; }
};
template <> struct Lowp<AXN_F16> {
  typedef uint16_t raw;
  __device__ static float to_float(raw x) { return (float)__builtin_bit_cast(_Float16, x); }
  __device__ static raw from_float(float f) {
    return __builtin_bit_cast(uint16_t, (_Float16)f);
  }
  __device__ static bool nonfinite(raw x) { return (x & 0x7C00u) == 0x7C00u; }
};
template <> struct Lowp<AXN_F32> {
  typedef uint32_t raw;
  __device__ static float to_float(raw x) { return __uint_as_float(x); }
  __device__ static raw from_float(float f) { return __float_as_uint(f); }
  __device__ static bool nonfinite(raw x) { return (x & 0x7F800000u) == 0x7F800000u; }
};

// 8 consecutive low-precision elements from a 16-byte aligned address.
template <int DT, bool NT>
__device__ __forceinline__ void load8(const void* base, int64_t i,
                                      typename Lowp<DT>::raw (&r)[8]) {
  typedef typename Lowp<DT>::raw raw;
  const raw* p = (const raw*)base + i;
  if (sizeof(raw) == 2) {
    const u32x4 w = ld<NT>((const u32x4*)p);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      r[2 * e] = (raw)(w[e] & 0xFFFFu);
      r[2 * e + 1] = (raw)(w[e] >> 16);
    }
  } else {
    const u32x4 w0 = ld<NT>((const u32x4*)p);
    const u32x4 w1 = ld<NT>((const u32x4*)p + 1);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      r[e] = (raw)w0[e];
      r[4 + e] = (raw)w1[e];
    }
  }
}

template <int DT, bool NT>
__device__ __forceinline__ void store8(void* base, int64_t i,
                                       const typename Lowp<DT>::raw (&r)[8]) {
  typedef typename Lowp<DT>::raw raw;
  raw* p = (raw*)base + i;
  if (sizeof(raw) == 2) {
    u32x4 w;
#pragma unroll
    for (int e = 0; e < 4; ++e)
      w[e] = (uint32_t)r[2 * e] | ((uint32_t)r[2 * e + 1] << 16);
    st<NT>(w, (u32x4*)p);
  } else {
    u32x4 w0, w1;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      w0[e] = (uint32_t)r[e];
      w1[e] = (uint32_t)r[4 + e];
    }
    st<NT>(w0, (u32x4*)p);
    st<NT>(w1, (u32x4*)p + 1);
  }
}

template <bool NT>
__device__ __forceinline__ void loadf8(const float* p, float (&x)[8]) {
  const f32x4 a = ld<NT>((const f32x4*)p);
  const f32x4 b = ld<NT>((const f32x4*)p + 1);
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    x[e] = a[e];
    x[4 + e] = b[e];
  }
}
template <bool NT>
__device__ __forceinline__ void storef8(float* p, const float (&x)[8]) {
  f32x4 a = {x[0], x[1], x[2], x[3]}, b = {x[4], x[5], x[6], x[7]};
  st<NT>(a, (f32x4*)p);
  st<NT>(b, (f32x4*)p + 1);
}

// Element range [begin, end) of tensor `t` owned by chunk `c`.  Chunk 0 also
// owns the scalar head [0, head).
struct Range {
  int64_t begin, end;
};
__device__ __forceinline__ Range chunk_range(const MtTable& tab, int t, int c) {
  const int64_t head = head_of(tab, t);
  Range r;
  r.begin = head + (int64_t)c * tab.chunk;
  r.end = r.begin + tab.chunk;
  if (r.end > tab.size[t]) r.end = tab.size[t];
  if (r.begin > r.end) r.begin = r.end;
  return r;
}

// ---------------------------------------------------------------- scan ------
__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) x += __shfl_xor(x, o, 64);
  return x;
}
__device__ __forceinline__ int wave_or(int x) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) x |= __shfl_xor(x, o, 64);
  return x;
}

// |u|^p of the norm's order p, by mode: the 2-norm and the 1-norm have their own
// instructions, order 0 counts the non-zero elements (torch.norm's meaning of p = 0),
// any other order goes through exp2(p log2 |u|) (|0|^p is 0 for p > 0 and +inf for p < 0,
// as in torch).
// Orders +inf and -inf are the largest and the smallest |u|: their terms are combined by
// max / min instead of a sum, a NaN staying a NaN as in torch.
enum NormMode { NORM_2 = 0, NORM_1 = 1, NORM_0 = 2, NORM_P = 3, NORM_MAX = 4, NORM_MIN = 5 };
template <int MODE>
__device__ __forceinline__ float norm_term(float u, float p) {
  if (MODE == NORM_2) return u * u;
  if (MODE == NORM_1 || MODE == NORM_MAX || MODE == NORM_MIN) return fabsf(u);
  if (MODE == NORM_0) return u != 0.0f ? 1.0f : 0.0f;
  return powf(fabsf(u), p);
}
// How two partial results of a mode meet, and the value that changes nothing.
template <int MODE, typename T>
__device__ __forceinline__ T norm_join(T a, T b) {
  if (MODE == NORM_MAX) return (a >= b || a != a) ? a : b;
  if (MODE == NORM_MIN) return (a <= b || a != a) ? a : b;
  return a + b;
}
template <int MODE>
__device__ __forceinline__ float norm_identity() {
  return MODE == NORM_MIN ? __builtin_inff() : 0.0f;
}

template <int DT, int MODE>
__global__ void __launch_bounds__(MT_THREADS)
    mt_scan_kernel(const MtTable tab, float inv_scale, float norm_type, ScanPartial* partial,
                   int block_base) {
  typedef typename Lowp<DT>::raw raw;
  const int t = find_tensor(tab, blockIdx.x);
  const int c = blockIdx.x - tab.chunk_start[t];
  const Range rg = chunk_range(tab, t, c);
  const void* g = tab.g[t];
  const int tid = threadIdx.x;

  float sq = norm_identity<MODE>(), sm = 0.f;
  int bad = 0;
  auto one = [&](raw x) {
    bad |= Lowp<DT>::nonfinite(x) ? 1 : 0;
    const float f = Lowp<DT>::to_float(x);
    sm += f;
    sq = norm_join<MODE>(sq, norm_term<MODE>(f * inv_scale, norm_type));
  };
  if (vec_ok_of(tab, t)) {
    if (c == 0 && tid < head_of(tab, t)) one(((const raw*)g)[tid]);
    const int64_t nvec = (rg.end - rg.begin) / MT_VEC;
    for (int64_t i = tid; i < nvec; i += MT_THREADS) {
      raw r[8];
      load8<DT, true>(g, rg.begin + i * MT_VEC, r);
#pragma unroll
      for (int e = 0; e < 8; ++e) one(r[e]);
    }
    const int64_t tail = rg.begin + nvec * MT_VEC;
    if (tail + tid < rg.end) one(((const raw*)g)[tail + tid]);
  } else {
    const int64_t b = (c == 0) ? 0 : rg.begin;
    for (int64_t i = b + tid; i < rg.end; i += MT_THREADS) one(((const raw*)g)[i]);
  }

  __shared__ float s_sq[MT_THREADS / 64], s_sm[MT_THREADS / 64];
  __shared__ int s_bad[MT_THREADS / 64];
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) sq = norm_join<MODE>(sq, __shfl_xor(sq, o, 64));
  sm = wave_sum(sm);
  bad = wave_or(bad);
  if ((tid & 63) == 0) {
    s_sq[tid >> 6] = sq;
    s_sm[tid >> 6] = sm;
    s_bad[tid >> 6] = bad;
  }
  __syncthreads();
  if (tid == 0) {
    ScanPartial p;
    p.sumsq = norm_identity<MODE>();
    p.sum = 0.f;
    p.nonfinite = 0;
#pragma unroll
    for (int w = 0; w < MT_THREADS / 64; ++w) {  // fixed order: deterministic
      p.sumsq = norm_join<MODE>(p.sumsq, s_sq[w]);
      p.sum += s_sm[w];
      p.nonfinite |= s_bad[w];
    }
    p.pad = 0;
    partial[block_base + blockIdx.x] = p;
  }
}

__device__ __forceinline__ double wave_sum_d(double x) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) x += __shfl_xor(x, o, 64);
  return x;
}

// One workgroup of 1024 threads reduces the partials of one launch group in a
// fixed order: wave w takes tensors w, w + 16, ...; lanes stride over that
// tensor's chunks.  `first` initialises the result, later groups accumulate.
template <int MODE>
__global__ void __launch_bounds__(1024)
    mt_scan_finalize_kernel(const MtTable tab, const ScanPartial* partial,
                            int block_base, double sum_limit, float max_norm,
                            float norm_type, int first, axn_scan_result* out) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  __shared__ double s_sq[16];
  __shared__ int s_bad[16];
  double sq = (double)norm_identity<MODE>();
  int bad = 0;
  for (int t = wave; t < tab.n; t += 16) {
    double tsq = (double)norm_identity<MODE>(), tsm = 0.0;
    int tbad = 0;
    for (int b = tab.chunk_start[t] + lane; b < tab.chunk_start[t + 1]; b += 64) {
      const ScanPartial p = partial[block_base + b];
      tsq = norm_join<MODE>(tsq, (double)p.sumsq);
      tsm += (double)p.sum;
      tbad |= p.nonfinite;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) tsq = norm_join<MODE>(tsq, __shfl_xor(tsq, o, 64));
    tsm = wave_sum_d(tsm);
    tbad = wave_or(tbad);
    // The tensor's sum, rounded to the gradient dtype, is non-finite.
    if (!(fabs(tsm) < sum_limit)) tbad = 1;
    // order 0: the norm over the stacked per-tensor norms counts the tensors whose own
    // count of non-zero elements is not zero
    if (MODE == NORM_0) tsq = tsq != 0.0 ? 1.0 : 0.0;
    sq = norm_join<MODE>(sq, tsq);
    bad |= tbad;
  }
  if (lane == 0) {
    s_sq[wave] = sq;
    s_bad[wave] = bad;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    double total = first ? (double)norm_identity<MODE>() : out->sumsq;
    int flag = first ? 0 : out->found_inf;
    for (int w = 0; w < 16; ++w) {
      total = norm_join<MODE>(total, s_sq[w]);
      flag |= s_bad[w];
    }
    const float norm = MODE == NORM_2 ? (float)sqrt(total)
                       : MODE == NORM_P ? (float)pow(total, 1.0 / (double)norm_type)
                                        : (float)total;
    float coef = 1.0f;
    if (max_norm > 0.0f) {
      coef = max_norm / (norm + 1e-6f);
      if (coef > 1.0f) coef = 1.0f;  // a NaN coefficient stays NaN, as torch.clamp keeps it
    }
    out->sumsq = total;
    out->total_norm = norm;
    out->clip_coef = coef;
    out->found_inf = flag;
    out->reserved[0] = out->reserved[1] = out->reserved[2] = 0;
  }
}

// ---------------------------------------------------------------- adam ------
struct AdamScalars {
  axn_adam_hparams hp;
  float inv_scale;
};

__device__ __forceinline__ void adam_math(float g, float& p, float& m, float& v,
                                          const AdamScalars& s, float gmul) {
  g = g * s.inv_scale;
  g = g * gmul;
  if (s.hp.weight_decay != 0.0f) g = g + s.hp.weight_decay * p;
  m = m + (g - m) * s.hp.one_minus_beta1;
  v = v * s.hp.beta2 + s.hp.one_minus_beta2 * g * g;
  const float denom = sqrtf(v) * s.hp.inv_sqrt_bc2 + s.hp.eps;
  p = p - s.hp.lr_over_bc1 * (m / denom);
  // The low-precision copy must be the rounding of the fp32 value that is
  // stored, not of the unrounded expression: keep the compiler from folding
  // the conversion into the last multiply-add (a mixed-precision FMA rounds once).
  asm volatile("" : "+v"(p));
}

typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

// One tensor's row of the table, in scalar registers.
struct TensorRow {
  const void* g;
  float* p;
  float* m;
  float* v;
  void* plow;
  int64_t size;
  int first_chunk;
  int meta;
};

// The row of the tensor that owns chunk `block`, through the scalar cache only: three
// pivots pick a quarter of the table, fifteen scalar compares on that quarter's starts pick
// the tensor, its row follows - three rounds of scalar loads from the argument block,
// which every wave of the launch repeats and the scalar cache holds.  Rows past the last
// tensor start at 2^31 - 1, which no chunk index reaches.  (Fetching row i in lane i with
// vector loads and voting is one round only, but those loads queue behind the streaming
// loads of the CU's other waves: 5.9 against 6.3 TB/s for the update.)
__device__ __forceinline__ TensorRow row_by_scalar_search(const MtTable& tab, int block) {
  static_assert(MT_MAX == 64, "four quarters of sixteen rows");
  // start <= block as the sign bit of start - block - 1 (both in [0, 2^31)): scalar adds only
  auto at_or_before = [block](int start) -> int { return (int)((uint32_t)(start - block - 1) >> 31); };
  const int q = at_or_before(tab.chunk_start[16]) + at_or_before(tab.chunk_start[32]) +
                at_or_before(tab.chunk_start[48]);
  const int base = q * 16;
  int t = base;
#pragma unroll
  for (int j = 1; j < 16; ++j) t += at_or_before(tab.chunk_start[base + j]);
  TensorRow r;
  r.g = tab.g[t];
  r.p = (float*)tab.p[t];
  r.m = (float*)tab.m[t];
  r.v = (float*)tab.v[t];
  r.plow = tab.plow[t];
  r.size = tab.size[t];
  r.first_chunk = tab.chunk_start[t];
  r.meta = tab.meta[t];
  return r;
}

// What the update's rate hangs on, measured on MI355X (1.3e9 elements, 64 tensors, 28 bytes
// per element; 6.5 to 6.6 TB/s as it stands):
//  - every access a wave makes covers consecutive bytes (one 4-element vector per lane:
//    16 bytes of each fp32 stream, 8 of each 16-bit one); loads non-temporal, stores
//    non-temporal and written through (nt + sc1: 1 to 2 % over nt alone, 10 % over plain
//    stores); 8 elements per lane in one access lose 6 %, cached loads of the state 13 %;
//  - all loads of a wave in front of its first store, and a wave that ends after its
//    stores: a wave that loops waits for its own stores before its next loads return
//    (the memory counter is in order; 16 trips per wave lose 6 %);
//  - one chunk per workgroup, handed out by the dispatcher in order, so that the chip
//    works on one compact window of every stream; resident workgroups that stride over
//    the chunks lose 8 to 12 %;
//  - FEWER waves in flight than the registers allow: with all 32 one-wave workgroups of a
//    CU resident the five streams thrash one another in the memory system (5.7 TB/s);
//    ten or eleven waves of one vector per lane are the best found (14 to 16 KB reserved
//    per workgroup: within 0.5 %; 12 KB: -2 %, 18 KB: -2.5 %).  The launch reserves ADAM_LDS
//    bytes of LDS per workgroup, which the kernel never touches, to hold the count there.
//    Several vectors per lane (ADAM_VECS) need fewer waves and make a skipped step cheaper
//    (1.27 M instead of 5.1 M workgroups that leave at once), but move 6 % less;
//  - a short way from the wave's start to its loads, because with few waves nothing hides
//    it: the table lookup stays on the scalar path, the scan result is loaded beside it,
//    not in front of it, and the accesses are buffer accesses (one descriptor per stream
//    in scalar registers, one 32-bit offset per lane: +3 to 4 % over 64-bit addresses
//    computed per lane).
template <int GDT, int PDT, bool HAS_PLOW, bool HAS_SCAN>
__global__ void __launch_bounds__(ADAM_THREADS)
    mt_adam_kernel(const MtTable tab, const AdamScalars s, const axn_scan_result* scan) {
  typedef typename Lowp<GDT>::raw graw;
  typedef typename Lowp<PDT>::raw praw;
  const int tid = threadIdx.x;
  const int b = blockIdx.x;
  const TensorRow row = row_by_scalar_search(tab, b);
  int found_inf = 0;
  float gmul = 1.0f;
  if (HAS_SCAN) {
    found_inf = scan->found_inf;
    gmul = scan->clip_coef;
  }
  const int c = b - row.first_chunk;
  // Overflow: the whole step is skipped.  As an empty range rather than an early return,
  // so that the scan result's load runs beside the table's and not in front of it.
  const int head = found_inf != 0 ? 0 : row.meta & 0xff;
  const int64_t size = found_inf != 0 ? 0 : row.size;
  Range rg;
  rg.begin = head + (int64_t)c * ADAM_CHUNK;
  rg.end = rg.begin + ADAM_CHUNK;
  if (rg.end > size) rg.end = size;
  if (rg.begin > rg.end) rg.begin = rg.end;
  const void* g = row.g;
  float* p = row.p;
  float* m = row.m;
  float* v = row.v;
  void* plow = row.plow;

  auto one = [&](int64_t i) {
    float pp = p[i], mm = m[i], vv = v[i];
    adam_math(Lowp<GDT>::to_float(((const graw*)g)[i]), pp, mm, vv, s, gmul);
    p[i] = pp;
    m[i] = mm;
    v[i] = vv;
    if (HAS_PLOW) ((praw*)plow)[i] = Lowp<PDT>::from_float(pp);
  };

  if (row.meta & 0x100) {
    if (c == 0 && tid < head) one(tid);
    const int nvec = (int)((rg.end - rg.begin) / ADAM_VEC);
    // ADAM_VECS vectors per lane, ADAM_THREADS vectors apart (every access of the wave
    // covers consecutive bytes), all loads in front of the first store.  Vector by vector
    // (g p m v, g p m v, ...); stream by stream (p p p p, m m m m, ...) measured the same on
    // constant data and 2 % slower on random data.
    // Each stream of the chunk is a buffer of exactly the bytes of its nvec vectors: the
    // hardware drops the accesses of the lanes behind the end (loads return zero, stores
    // do nothing), so a ragged last chunk runs the same code, and a lane needs one 32-bit
    // offset per access instead of a 64-bit address.
    constexpr int GSZ = (int)sizeof(graw), PSZ = (int)sizeof(praw);
    auto stream = [&](const void* base, int elem) {
      return __builtin_amdgcn_make_buffer_rsrc((void*)((const char*)base + rg.begin * elem), 0,
                                               nvec * ADAM_VEC * elem, 0x00020000);
    };
    if (nvec > 0) {   // (a skipped step's waves leave here)
    const __amdgpu_buffer_rsrc_t bg = stream(g, GSZ), bp = stream(p, 4), bm = stream(m, 4),
                                 bv = stream(v, 4), bl = stream(HAS_PLOW ? plow : p, PSZ);
    graw gr[ADAM_VECS][4];
    f32x4 pp[ADAM_VECS], mm[ADAM_VECS], vv[ADAM_VECS];
#pragma unroll
    for (int k = 0; k < ADAM_VECS; ++k) {
      const int e0 = (tid + k * ADAM_THREADS) * ADAM_VEC;
      if (GSZ == 2) {
        const u32x2 w = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(bg, e0 * 2, 0, ADAM_LOAD_POLICY));
        gr[k][0] = (graw)(w[0] & 0xFFFFu);
        gr[k][1] = (graw)(w[0] >> 16);
        gr[k][2] = (graw)(w[1] & 0xFFFFu);
        gr[k][3] = (graw)(w[1] >> 16);
      } else {
        const u32x4 w = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(bg, e0 * 4, 0, ADAM_LOAD_POLICY));
#pragma unroll
        for (int e = 0; e < 4; ++e) gr[k][e] = (graw)w[e];
      }
      pp[k] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(bp, e0 * 4, 0, ADAM_LOAD_POLICY));
      mm[k] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(bm, e0 * 4, 0, ADAM_LOAD_POLICY));
      vv[k] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(bv, e0 * 4, 0, ADAM_LOAD_POLICY));
    }
    __builtin_amdgcn_sched_barrier(0);   // every load is issued before the arithmetic of the first vector
#pragma unroll
    for (int k = 0; k < ADAM_VECS; ++k) {
      const int e0 = (tid + k * ADAM_THREADS) * ADAM_VEC;
      praw pl[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float pe = pp[k][e], me = mm[k][e], ve = vv[k][e];
        adam_math(Lowp<GDT>::to_float(gr[k][e]), pe, me, ve, s, gmul);
        pp[k][e] = pe;
        mm[k][e] = me;
        vv[k][e] = ve;
        if (HAS_PLOW) pl[e] = Lowp<PDT>::from_float(pe);
      }
      __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, pp[k]), bp, e0 * 4, 0, ADAM_STORE_POLICY);
      __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, mm[k]), bm, e0 * 4, 0, ADAM_STORE_POLICY);
      __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, vv[k]), bv, e0 * 4, 0, ADAM_STORE_POLICY);
      if (HAS_PLOW) {
        if (PSZ == 2) {
          u32x2 w;
          w[0] = (uint32_t)pl[0] | ((uint32_t)pl[1] << 16);
          w[1] = (uint32_t)pl[2] | ((uint32_t)pl[3] << 16);
          __builtin_amdgcn_raw_buffer_store_b64(w, bl, e0 * 2, 0, ADAM_STORE_POLICY);
        } else {
          u32x4 w;
#pragma unroll
          for (int e = 0; e < 4; ++e) w[e] = (uint32_t)pl[e];
          __builtin_amdgcn_raw_buffer_store_b128(w, bl, e0 * 4, 0, ADAM_STORE_POLICY);
        }
      }
    }
    }
    const int64_t tail = rg.begin + (int64_t)nvec * ADAM_VEC;
    if (tail + tid < rg.end) one(tail + tid);
  } else {
    const int64_t b0 = (c == 0) ? 0 : rg.begin;
    for (int64_t i = b0 + tid; i < rg.end; i += ADAM_THREADS) one(i);
  }
}

// --------------------------------------------------------------- scale ------
template <int DT>
__global__ void __launch_bounds__(MT_THREADS)
    mt_scale_kernel(const MtTable tab, float inv_scale,
                    const axn_scan_result* scan, int use_clip) {
  typedef typename Lowp<DT>::raw raw;
  const float coef = use_clip ? scan->clip_coef : 1.0f;
  const int t = find_tensor(tab, blockIdx.x);
  const int c = blockIdx.x - tab.chunk_start[t];
  const Range rg = chunk_range(tab, t, c);
  void* g = const_cast<void*>(tab.g[t]);
  const int tid = threadIdx.x;
  // Two roundings, as the reference's separate div_ and mul_ passes make.
  auto f = [&](raw x) -> raw {
    raw y = Lowp<DT>::from_float(Lowp<DT>::to_float(x) * inv_scale);
    if (use_clip) y = Lowp<DT>::from_float(Lowp<DT>::to_float(y) * coef);
    return y;
  };
  if (vec_ok_of(tab, t)) {
    if (c == 0 && tid < head_of(tab, t)) ((raw*)g)[tid] = f(((raw*)g)[tid]);
    const int64_t nvec = (rg.end - rg.begin) / MT_VEC;
    for (int64_t i = tid; i < nvec; i += MT_THREADS) {
      raw r[8];
      load8<DT, false>(g, rg.begin + i * MT_VEC, r);
#pragma unroll
      for (int e = 0; e < 8; ++e) r[e] = f(r[e]);
      store8<DT, true>(g, rg.begin + i * MT_VEC, r);
    }
    const int64_t tail = rg.begin + nvec * MT_VEC;
    if (tail + tid < rg.end) ((raw*)g)[tail + tid] = f(((raw*)g)[tail + tid]);
  } else {
    const int64_t b = (c == 0) ? 0 : rg.begin;
    for (int64_t i = b + tid; i < rg.end; i += MT_THREADS) ((raw*)g)[i] = f(((raw*)g)[i]);
  }
}

// ------------------------------------------------------------- host side ----
int dtype_size(int dt) { return dt == AXN_F32 ? 4 : 2; }

// Number of leading scalar elements after which every given pointer of a
// tensor is 16-byte aligned, or -1 when no common count exists.  The pointer
// with the narrowest element decides the count; the others must agree.
int common_head(const void* const* ptrs, const int* elem_sizes, int count) {
  int best = 0;
  for (int i = 0; i < count; ++i) {
    if (ptrs[i] == nullptr) continue;
    const uintptr_t a = (uintptr_t)ptrs[i];
    const int es = elem_sizes[i];
    if (a % es != 0) return -1;
    const int h = (int)(((16 - a % 16) % 16) / es);
    if (h > best) best = h;
  }
  for (int i = 0; i < count; ++i) {
    if (ptrs[i] == nullptr) continue;
    const uintptr_t a = (uintptr_t)ptrs[i] + (uintptr_t)best * elem_sizes[i];
    if (a % 16 != 0) return -1;
  }
  // Prefer a head after which every pointer sits on a 128-byte cache line, so that
  // the chunks of different workgroups do not share lines (views at one common
  // element offset into line-aligned flat buffers always have one, of at most 63
  // elements).  Steps of 8 elements keep the 16-byte alignment found above.
  for (int h = best; h < 64; h += 8) {
    bool all = true;
    for (int i = 0; i < count && all; ++i)
      if (ptrs[i] != nullptr)
        all = ((uintptr_t)ptrs[i] + (uintptr_t)h * elem_sizes[i]) % 128 == 0;
    if (all) return h;
  }
  return best;
}

struct Group {
  MtTable tab;
  int blocks;
};

// Walks the tensor list in launch groups (at most MT_MAX tensors, below 2^31 chunks)
// and hands each filled argument table to `emit`, which returns a status; the first
// non-zero status ends the walk.  `ptr_sets[k][i]` is pointer k of tensor i (k = 0 is
// always the gradient).  Nothing is allocated: the one table lives on the stack.
template <class Emit>
int for_each_group(const void* const* const* ptr_sets, const int* elem_sizes, int nsets,
                   const int64_t* h_sizes, int64_t n, int chunk, Emit&& emit) {
  Group cur;
  cur.tab = MtTable();
  cur.blocks = 0;
  int k = 0;
  auto flush = [&]() -> int {
    if (k == 0) return AXN_OK;
    cur.tab.n = k;
    cur.tab.chunk = chunk;
    // past the last tensor: a start no workgroup index reaches, so that a lookup need
    // not know the count
    for (int j = k; j <= MT_MAX; ++j) cur.tab.chunk_start[j] = j == k ? cur.blocks : 0x7fffffff;
    const int rc = emit(cur);
    cur.tab = MtTable();
    cur.blocks = 0;
    k = 0;
    return rc;
  };
  for (int64_t i = 0; i < n; ++i) {
    const int64_t sz = h_sizes[i];
    if (sz == 0) continue;
    const void* ptrs[5] = {nullptr, nullptr, nullptr, nullptr, nullptr};
    for (int s = 0; s < nsets; ++s) ptrs[s] = ptr_sets[s] ? ptr_sets[s][i] : nullptr;
    int head = common_head(ptrs, elem_sizes, nsets);
    const bool vec_ok = head >= 0;
    if (!vec_ok) head = 0;
    if (head > sz) head = (int)sz;
    const int64_t body = sz - head;
    int64_t chunks = (body + chunk - 1) / chunk;
    if (chunks == 0) chunks = 1;  // the head still needs a workgroup
    if (chunks > 0x3fffffff) {
      set_error("multi-tensor: tensor %lld has too many elements (%lld)",
                (long long)i, (long long)sz);
      return AXN_ELIMIT;
    }
    if (k == MT_MAX || (long long)cur.blocks + chunks > 0x7fffffffLL) {
      const int rc = flush();
      if (rc != AXN_OK) return rc;
    }
    cur.tab.g[k] = ptrs[0];
    cur.tab.p[k] = const_cast<void*>(ptrs[1]);
    cur.tab.m[k] = const_cast<void*>(ptrs[2]);
    cur.tab.v[k] = const_cast<void*>(ptrs[3]);
    cur.tab.plow[k] = const_cast<void*>(ptrs[4]);
    cur.tab.size[k] = sz;
    cur.tab.chunk_start[k] = cur.blocks;
    cur.tab.meta[k] = head | (vec_ok ? 0x100 : 0);
    cur.blocks += (int)chunks;
    ++k;
  }
  return flush();
}

double sum_limit_of(int dt) {
  // Smallest magnitude that rounds (to nearest even) to infinity in the dtype.
  switch (dt) {
    case AXN_F16: return 65520.0;
    case AXN_BF16: return 3.3961775292304601e38;   // 2^127 * (2 - 2^-8)
    default: return 3.4028235677973366e38;         // 2^127 * (2 - 2^-24)
  }
}

int norm_mode_host(float p) {
  return p == 2.0f ? NORM_2 : p == 1.0f ? NORM_1 : p == 0.0f ? NORM_0
         : p == INFINITY ? NORM_MAX : p == -INFINITY ? NORM_MIN : NORM_P;
}

template <int DT>
void scan_dispatch(const Group& gr, float inv_scale, float norm_type, ScanPartial* partial,
                   int base, hipStream_t stream) {
  const dim3 grid(gr.blocks), block(MT_THREADS);
  switch (norm_mode_host(norm_type)) {
#define AXN_SCAN_CASE(MODE)                                                                     \
  case MODE:                                                                                    \
    hipLaunchKernelGGL((mt_scan_kernel<DT, MODE>), grid, block, 0, stream, gr.tab, inv_scale,   \
                       norm_type, partial, base);                                               \
    break;
    AXN_SCAN_CASE(NORM_2)
    AXN_SCAN_CASE(NORM_1)
    AXN_SCAN_CASE(NORM_0)
    AXN_SCAN_CASE(NORM_MAX)
    AXN_SCAN_CASE(NORM_MIN)
    default:
    AXN_SCAN_CASE(NORM_P)
#undef AXN_SCAN_CASE
  }
}

void finalize_dispatch(const MtTable& tab, const ScanPartial* partial, int base, double sum_limit,
                       float max_norm, float norm_type, int first, axn_scan_result* result,
                       hipStream_t stream) {
  switch (norm_mode_host(norm_type)) {
#define AXN_FIN_CASE(MODE)                                                                       \
  case MODE:                                                                                     \
    hipLaunchKernelGGL(mt_scan_finalize_kernel<MODE>, dim3(1), dim3(1024), 0, stream, tab,       \
                       partial, base, sum_limit, max_norm, norm_type, first, result);            \
    break;
    AXN_FIN_CASE(NORM_2)
    AXN_FIN_CASE(NORM_1)
    AXN_FIN_CASE(NORM_0)
    AXN_FIN_CASE(NORM_MAX)
    AXN_FIN_CASE(NORM_MIN)
    default:
    AXN_FIN_CASE(NORM_P)
#undef AXN_FIN_CASE
  }
}

}  // namespace
}  // namespace axn

// Scratch of axn_mt_scan_noalloc: the per-chunk partial results of the scan, in device
// memory that exists for the life of the process (1 MiB per GPU the library runs on).
// This name is a host-side handle only; the device address is looked up per device.
static __device__ __align__(256) unsigned char scratch[AXN_MT_SCAN_SCRATCH_BYTES];

namespace axn {
namespace {

// Device address of `scratch` on the current device, looked up once per device.
int scan_scratch(void** out) {
  static std::mutex mu;
  static void* ptrs[64];
  int dev = 0;
  AXN_HIP_TRY(hipGetDevice(&dev));
  if (dev < 0 || dev >= 64) {
    set_error("axn_mt_scan_noalloc: device index %d out of range", dev);
    return AXN_ELIMIT;
  }
  std::lock_guard<std::mutex> lock(mu);
  if (ptrs[dev] == nullptr) {
    void* p = nullptr;
    AXN_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (p == nullptr) {
      set_error("axn_mt_scan_noalloc: no device address for the scratch array");
      return AXN_EHIP;
    }
    ptrs[dev] = p;
  }
  *out = ptrs[dev];
  return AXN_OK;
}

}  // namespace

size_t mt_scan_workspace_bytes(int64_t n, int64_t total) {
  if (n < 0 || total < 0) return 0;
  // One partial per chunk; a tensor adds at most one ragged chunk.
  const int64_t blocks = total / SCAN_CHUNK + 2 * n + 1;
  return (size_t)blocks * sizeof(ScanPartial);
}

int launch_mt_scan(const void* const* h_g, const int64_t* h_sizes, int64_t n,
                   int g_dtype, float inv_scale, float max_norm, float norm_type,
                   int accumulate, axn_scan_result* result, void* ws, size_t ws_bytes,
                   hipStream_t stream) {
  const void* const* sets[1] = {h_g};
  const int es[1] = {dtype_size(g_dtype)};
  // first walk: what the partial results need
  int64_t need = 0;
  int rc = for_each_group(sets, es, 1, h_sizes, n, SCAN_CHUNK, [&](const Group& gr) {
    need += gr.blocks;
    return (int)AXN_OK;
  });
  if (rc != AXN_OK) return rc;
  if ((size_t)need * sizeof(ScanPartial) > ws_bytes) {
    set_error("mt_scan: workspace too small (%zu bytes given, %zu needed)",
              ws_bytes, (size_t)need * sizeof(ScanPartial));
    return AXN_EINVAL;
  }
  ScanPartial* partial = (ScanPartial*)ws;
  if (need == 0) {
    // Nothing to scan: norm 0, no overflow.
    MtTable empty = MtTable();
    empty.n = 0;
    empty.chunk = SCAN_CHUNK;
    // (nothing scanned and nothing to add to: every order's norm is 0)
    finalize_dispatch(empty, partial, 0, sum_limit_of(g_dtype), max_norm, accumulate ? norm_type : 2.0f,
                      accumulate ? 0 : 1, result, stream);
    AXN_HIP_TRY(hipGetLastError());
    return AXN_OK;
  }
  int base = 0;
  bool first = !accumulate;
  return for_each_group(sets, es, 1, h_sizes, n, SCAN_CHUNK, [&](const Group& gr) {
    switch (g_dtype) {
      case AXN_BF16: scan_dispatch<AXN_BF16>(gr, inv_scale, norm_type, partial, base, stream); break;
      case AXN_F16: scan_dispatch<AXN_F16>(gr, inv_scale, norm_type, partial, base, stream); break;
      default: scan_dispatch<AXN_F32>(gr, inv_scale, norm_type, partial, base, stream); break;
    }
    AXN_HIP_TRY(hipGetLastError());
    finalize_dispatch(gr.tab, partial, base, sum_limit_of(g_dtype), max_norm, norm_type, first ? 1 : 0,
                      result, stream);
    AXN_HIP_TRY(hipGetLastError());
    base += gr.blocks;
    first = false;
    return (int)AXN_OK;
  });
}

int launch_mt_scan_noalloc(const void* const* h_g, const int64_t* h_sizes, int64_t n,
                           int g_dtype, float inv_scale, float max_norm, float norm_type,
                           int accumulate, axn_scan_result* result, hipStream_t stream) {
  // the size limit is checked before anything touches the device
  const void* const* sets[1] = {h_g};
  const int es[1] = {dtype_size(g_dtype)};
  int64_t need = 0;
  int rc = for_each_group(sets, es, 1, h_sizes, n, SCAN_CHUNK, [&](const Group& gr) {
    need += gr.blocks;
    return (int)AXN_OK;
  });
  if (rc != AXN_OK) return rc;
  if ((size_t)need * sizeof(ScanPartial) > (size_t)AXN_MT_SCAN_SCRATCH_BYTES) {
    set_error("axn_mt_scan_noalloc: the gradients make %lld chunks of %d elements, the built-in "
              "scratch holds %lld; use axn_mt_scan with a workspace",
              (long long)need, SCAN_CHUNK,
              (long long)(AXN_MT_SCAN_SCRATCH_BYTES / sizeof(ScanPartial)));
    return AXN_ELIMIT;
  }
  void* ws = nullptr;
  rc = scan_scratch(&ws);
  if (rc != AXN_OK) return rc;
  return launch_mt_scan(h_g, h_sizes, n, g_dtype, inv_scale, max_norm, norm_type, accumulate,
                        result, ws, (size_t)AXN_MT_SCAN_SCRATCH_BYTES, stream);
}

namespace {
template <int GDT, bool HAS_SCAN>
int adam_launch(const Group& gr, const AdamScalars& s, int plow_dtype, bool has_plow,
                const axn_scan_result* scan, hipStream_t stream) {
  const dim3 grid((unsigned)gr.blocks), block(ADAM_THREADS);
  if (!has_plow) {
    hipLaunchKernelGGL((mt_adam_kernel<GDT, AXN_BF16, false, HAS_SCAN>), grid, block, ADAM_LDS,
                       stream, gr.tab, s, scan);
  } else if (plow_dtype == AXN_BF16) {
    hipLaunchKernelGGL((mt_adam_kernel<GDT, AXN_BF16, true, HAS_SCAN>), grid, block, ADAM_LDS,
                       stream, gr.tab, s, scan);
  } else {
    hipLaunchKernelGGL((mt_adam_kernel<GDT, AXN_F16, true, HAS_SCAN>), grid, block, ADAM_LDS,
                       stream, gr.tab, s, scan);
  }
  AXN_HIP_TRY(hipGetLastError());
  return AXN_OK;
}
template <int GDT>
int adam_dispatch(const Group& gr, const AdamScalars& s, int plow_dtype,
                  bool has_plow, const axn_scan_result* scan, hipStream_t stream) {
  return scan != nullptr ? adam_launch<GDT, true>(gr, s, plow_dtype, has_plow, scan, stream)
                         : adam_launch<GDT, false>(gr, s, plow_dtype, has_plow, scan, stream);
}
}  // namespace

int launch_mt_adam(const void* const* h_g, void* const* h_p, void* const* h_m,
                   void* const* h_v, void* const* h_plow, const int64_t* h_sizes,
                   int64_t n, int g_dtype, int plow_dtype, float inv_scale,
                   const axn_scan_result* scan, const axn_adam_hparams& hp,
                   hipStream_t stream) {
  const void* const* sets[5] = {h_g, (const void* const*)h_p, (const void* const*)h_m,
                                (const void* const*)h_v, (const void* const*)h_plow};
  const int es[5] = {dtype_size(g_dtype), 4, 4, 4, dtype_size(plow_dtype)};
  AdamScalars s;
  s.hp = hp;
  s.inv_scale = inv_scale;
  const bool has_plow = h_plow != nullptr;
  return for_each_group(sets, es, 5, h_sizes, n, ADAM_CHUNK, [&](const Group& gr) {
    switch (g_dtype) {
      case AXN_BF16: return adam_dispatch<AXN_BF16>(gr, s, plow_dtype, has_plow, scan, stream);
      case AXN_F16: return adam_dispatch<AXN_F16>(gr, s, plow_dtype, has_plow, scan, stream);
      default: return adam_dispatch<AXN_F32>(gr, s, plow_dtype, has_plow, scan, stream);
    }
  });
}

int launch_mt_scale(void* const* h_g, const int64_t* h_sizes, int64_t n,
                    int g_dtype, float inv_scale, const axn_scan_result* scan,
                    int use_clip, hipStream_t stream) {
  const void* const* sets[1] = {(const void* const*)h_g};
  const int es[1] = {dtype_size(g_dtype)};
  return for_each_group(sets, es, 1, h_sizes, n, SCALE_CHUNK, [&](const Group& gr) {
    const dim3 grid(gr.blocks), block(MT_THREADS);
    switch (g_dtype) {
      case AXN_BF16:
        hipLaunchKernelGGL(mt_scale_kernel<AXN_BF16>, grid, block, 0, stream,
                           gr.tab, inv_scale, scan, use_clip);
        break;
      case AXN_F16:
        hipLaunchKernelGGL(mt_scale_kernel<AXN_F16>, grid, block, 0, stream,
                           gr.tab, inv_scale, scan, use_clip);
        break;
      default:
        hipLaunchKernelGGL(mt_scale_kernel<AXN_F32>, grid, block, 0, stream,
                           gr.tab, inv_scale, scan, use_clip);
        break;
    }
    AXN_HIP_TRY(hipGetLastError());
    return (int)AXN_OK;
  });
}

}  // namespace axn
