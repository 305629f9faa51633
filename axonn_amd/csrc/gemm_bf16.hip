// bf16 MFMA GEMM for gfx950 (MI355X): the three shard GEMMs of the
// tensor-parallel Linear layer,
//   forward  Y  = X  W^T   (axonn/intra_layer/fully_connected.py:118)
//   dgrad    dX = dY W     (fully_connected.py:140)
//   wgrad    dW = dY^T X   (fully_connected.py:147-151)
// as one templated kernel over the operand storage orders.
//
// Structure
//   * v_mfma_f32_32x32x16_bf16, fp32 accumulate in registers.
//   * A workgroup owns a BM x BN output tile and walks the contraction in
//     steps of 64; operand tiles are staged global -> VGPR -> LDS, double
//     buffered, one workgroup barrier per step.
//   * LDS layouts are chosen per storage order so that fragment reads are free
//     of bank conflicts on the 64-bank LDS:
//       K-major  tile [rows][64]   : 16-byte chunk c of row r lives at chunk
//                                    c ^ ((r >> 1) & 7); read with ds_read_b128.
//       MN-major tile [64][rows]   : 64-byte chunk c of contraction row k lives
//                                    at chunk c ^ (k & 3); read with the
//                                    transposing ds_read_b64_tr_b16, which hands
//                                    every lane 4 consecutive contraction
//                                    elements of one output row/column.
//   * The MFMA is issued with the operands swapped (D^T = B^T A^T) so a lane
//     ends up with 4 consecutive output columns per register quad; the
//     epilogue transposes through LDS once more so every lane writes 16
//     contiguous bytes and a row segment of 128 bytes is written by 8 lanes.
//   * Workgroup ids are remapped so that each of the 8 XCDs (private L2 each)
//     works on a compact block of neighbouring tiles.
#include "axn_internal.h"

namespace axn {
namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

constexpr int BK = 64;          // contraction elements per step
constexpr int NUM_XCD = 8;      // MI355X: 8 accelerator dies, round-robin dispatch
constexpr int EPI_LD = 68;      // floats per row of the epilogue staging buffer

#define LDS_PTR(T, p) ((__attribute__((address_space(3))) T*)(p))

__device__ __forceinline__ float gelu_exact(float z) {
  return 0.5f * z * (1.0f + erff(z * 0.70710678118654752440f));
}

// Workgroup id -> output tile, XCD aware.  Consecutive workgroup ids go to
// different XCDs, so ids are first regrouped per XCD into contiguous ranges and
// then walked in bands of GROUP_M tile rows.
__device__ __forceinline__ void tile_of_workgroup(int pid, int tiles_m,
                                                  int tiles_n, int& tm,
                                                  int& tn) {
  const int nwg = tiles_m * tiles_n;
  const int per = (nwg + NUM_XCD - 1) / NUM_XCD;
  int tall = nwg % NUM_XCD;
  if (tall == 0) tall = NUM_XCD;
  const int xcd = pid % NUM_XCD;
  const int local = pid / NUM_XCD;
  int t = (xcd < tall) ? xcd * per + local
                       : tall * per + (xcd - tall) * (per - 1) + local;
  constexpr int GROUP_M = 8;
  const int in_group = GROUP_M * tiles_n;
  const int group = t / in_group;
  const int first_m = group * GROUP_M;
  const int gsz = (tiles_m - first_m < GROUP_M) ? tiles_m - first_m : GROUP_M;
  const int r = t - group * in_group;
  tm = first_m + r % gsz;
  tn = r / gsz;
}

// One operand tile: global -> registers -> LDS, and fragment reads.
//   ROWS     rows/columns of the output covered by the tile (BM or BN)
//   KMAJOR   storage order (see file header)
//   NT       threads in the workgroup
template <int ROWS, bool KMAJOR, int NT, bool EDGE>
struct OperandTile {
  static constexpr int CHUNKS = ROWS * BK / 8;       // 16-byte chunks per tile
  static constexpr int PER_THREAD = CHUNKS / NT;     // chunks per thread
  static constexpr int BYTES = ROWS * BK * 2;
  static_assert(CHUNKS % NT == 0, "tile must divide evenly over the threads");

  // Global load of this thread's chunks of the tile starting at contraction
  // index k0; out-of-range chunks read as zero when EDGE.
  __device__ __forceinline__ static void load(u32x4 (&r)[PER_THREAD],
                                              const uint16_t* base, int64_t ld,
                                              int row0, int row_max, int k0,
                                              int k_max, int tid) {
#pragma unroll
    for (int i = 0; i < PER_THREAD; ++i) {
      const int id = i * NT + tid;
      int row, k;
      if (KMAJOR) {
        row = id >> 3;
        k = (id & 7) * 8;
      } else {
        k = id / (ROWS / 8);
        row = (id % (ROWS / 8)) * 8;
      }
      const int gr = row0 + row, gk = k0 + k;
      const uint16_t* p = KMAJOR ? base + (int64_t)gr * ld + gk
                                 : base + (int64_t)gk * ld + gr;
      if (EDGE) {
        if (gr < row_max && gk < k_max) {
          r[i] = *(const u32x4*)p;
        } else {
          r[i] = u32x4{0u, 0u, 0u, 0u};
        }
      } else {
        r[i] = *(const u32x4*)p;
      }
    }
  }

  __device__ __forceinline__ static void store(const u32x4 (&r)[PER_THREAD],
                                               char* lds, int tid) {
#pragma unroll
    for (int i = 0; i < PER_THREAD; ++i) {
      const int id = i * NT + tid;
      int off;
      if (KMAJOR) {
        const int row = id >> 3, c = id & 7;
        off = row * 128 + ((c ^ ((row >> 1) & 7)) << 4);
      } else {
        const int k = id / (ROWS / 8), c16 = id % (ROWS / 8);
        off = k * (ROWS * 2) + ((((c16 >> 2) ^ (k & 3)) << 6) | ((c16 & 3) << 4));
      }
      *(u32x4*)(lds + off) = r[i];
    }
  }

  // MFMA operand fragment for 32 rows starting at `row` (multiple of 32 within
  // the tile) and the 16 contraction elements starting at 16 * kk.
  __device__ __forceinline__ static bf16x8 frag(const char* lds, int row,
                                                int kk, int lane) {
    if (KMAJOR) {
      const int r = row + (lane & 31);
      const int swz = ((lane & 31) >> 1) & 7;
      const int c = (kk * 2 + (lane >> 5)) ^ swz;
      return *(const bf16x8*)(lds + r * 128 + (c << 4));
    } else {
      const int kq = (lane & 15) >> 2;  // == k & 3 for both halves
      const int k = kk * 16 + 8 * (lane >> 5) + kq;
      const int colbyte = (row + 16 * ((lane >> 4) & 1) + 4 * (lane & 3)) * 2;
      const int off = k * (ROWS * 2) + ((((colbyte >> 6) ^ kq) << 6) | (colbyte & 63));
      s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(s16x4, lds + off));
      s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
          LDS_PTR(s16x4, lds + off + 4 * (ROWS * 2)));
      typedef __attribute__((ext_vector_type(8))) short s16x8;
      s16x8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
      return __builtin_bit_cast(bf16x8, v);
    }
  }
};

template <int BM, int BN, int WAVES_M, int WAVES_N, bool A_KMAJOR, bool B_KMAJOR,
          int EPI, bool OUT_F32, bool EDGE>
__global__ void __launch_bounds__(WAVES_M* WAVES_N * 64)
    gemm_bf16_kernel(const GemmArgs g) {
  constexpr int NT = WAVES_M * WAVES_N * 64;
  constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
  constexpr int FM = WTM / 32, FN = WTN / 32;
  static_assert(WTM % 32 == 0 && WTN % 32 == 0, "wave tile must be 32-aligned");
  using TA = OperandTile<BM, A_KMAJOR, NT, EDGE>;
  using TB = OperandTile<BN, B_KMAJOR, NT, EDGE>;
  constexpr int STAGE = TA::BYTES + TB::BYTES;

  extern __shared__ __attribute__((aligned(16))) char lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;

  int tm, tn;
  tile_of_workgroup(blockIdx.x, g.tiles_m, g.tiles_n, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;

  f32x16 acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  u32x4 ra[TA::PER_THREAD], rb[TB::PER_THREAD];
  const int KT = (g.Kc + BK - 1) / BK;

  TA::load(ra, g.A, g.lda, m0, g.M, 0, g.Kc, tid);
  TB::load(rb, g.B, g.ldb, n0, g.N, 0, g.Kc, tid);
  TA::store(ra, lds, tid);
  TB::store(rb, lds + TA::BYTES, tid);
  __syncthreads();

  for (int kt = 0; kt < KT; ++kt) {
    const char* sA = lds + (kt & 1) * STAGE;
    const char* sB = sA + TA::BYTES;
    const bool more = kt + 1 < KT;
    if (more) {
      TA::load(ra, g.A, g.lda, m0, g.M, (kt + 1) * BK, g.Kc, tid);
      TB::load(rb, g.B, g.ldb, n0, g.N, (kt + 1) * BK, g.Kc, tid);
    }
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
      bf16x8 fa[FM], fb[FN];
#pragma unroll
      for (int i = 0; i < FM; ++i) fa[i] = TA::frag(sA, wm * WTM + i * 32, kk, lane);
#pragma unroll
      for (int j = 0; j < FN; ++j) fb[j] = TB::frag(sB, wn * WTN + j * 32, kk, lane);
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[j], fa[i],
                                                              acc[i][j], 0, 0, 0);
    }
    if (more) {
      char* nA = lds + ((kt + 1) & 1) * STAGE;
      TA::store(ra, nA, tid);
      TB::store(rb, nA + TA::BYTES, tid);
    }
    __syncthreads();
  }

  // ---- epilogue -----------------------------------------------------------
  // With the operands swapped, lane l register r of acc[i][j] is the output
  // element  row = l % 32,  col = 8 * (r / 4) + 4 * (l / 32) + r % 4  of the
  // 32 x 32 block (i, j) of this wave's tile.
  constexpr int EPC = (WTN < 64) ? WTN : 64;  // columns per staging pass
  constexpr int JP = EPC / 32;                // fragments per pass
  constexpr int LPR = EPC / 8;                // lanes per row on read-back
  constexpr int RPI = 64 / LPR;               // rows per read-back iteration
  static_assert(32 * EPI_LD * 4 * WAVES_M * WAVES_N <= 2 * STAGE,
                "epilogue staging must fit in the operand buffers");
  float* E = (float*)lds + wave * (32 * EPI_LD);

#pragma unroll
  for (int i = 0; i < FM; ++i) {
#pragma unroll
    for (int jp = 0; jp < FN / JP; ++jp) {
#pragma unroll
      for (int jj = 0; jj < JP; ++jj) {
        const f32x16 a = acc[i][jp * JP + jj];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          f32x4 v = {a[4 * q], a[4 * q + 1], a[4 * q + 2], a[4 * q + 3]};
          *(f32x4*)&E[(lane & 31) * EPI_LD + jj * 32 + 8 * q + 4 * (lane >> 5)] = v;
        }
      }
#pragma unroll
      for (int it = 0; it < 32 / RPI; ++it) {
        const int r = it * RPI + lane / LPR;
        const int c = (lane % LPR) * 8;
        const f32x4 v0 = *(const f32x4*)&E[r * EPI_LD + c];
        const f32x4 v1 = *(const f32x4*)&E[r * EPI_LD + c + 4];
        float v[8] = {v0[0], v0[1], v0[2], v0[3], v1[0], v1[1], v1[2], v1[3]};
        const int row = m0 + wm * WTM + i * 32 + r;
        const int col = n0 + wn * WTN + jp * EPC + c;
        if (EDGE && (row >= g.M || col >= g.N)) continue;
        const int64_t o = (int64_t)row * g.ldc + col;
        if (EPI == AXN_EPI_BIAS || EPI == AXN_EPI_BIAS_GELU) {
          const f32x4 b0 = *(const f32x4*)(g.bias + col);
          const f32x4 b1 = *(const f32x4*)(g.bias + col + 4);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            v[e] += b0[e];
            v[4 + e] += b1[e];
          }
        }
        if (EPI == AXN_EPI_BIAS_GELU || EPI == AXN_EPI_GELU) {
          if (g.Z != nullptr) {
            bf16x8 z;
#pragma unroll
            for (int e = 0; e < 8; ++e) z[e] = (__bf16)v[e];
            *(bf16x8*)(g.Z + o) = z;
          }
#pragma unroll
          for (int e = 0; e < 8; ++e) v[e] = gelu_exact(v[e]);
        }
        if (OUT_F32) {
          float* C = (float*)g.C + o;
          f32x4 o0 = {v[0], v[1], v[2], v[3]}, o1 = {v[4], v[5], v[6], v[7]};
          if (g.beta) {
            o0 += *(const f32x4*)C;
            o1 += *(const f32x4*)(C + 4);
          }
          *(f32x4*)C = o0;
          *(f32x4*)(C + 4) = o1;
        } else {
          uint16_t* C = (uint16_t*)g.C + o;
          if (g.beta) {
            const bf16x8 old = *(const bf16x8*)C;
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] += (float)old[e];
          }
          bf16x8 y;
#pragma unroll
          for (int e = 0; e < 8; ++e) y[e] = (__bf16)v[e];
          *(bf16x8*)C = y;
        }
      }
    }
  }
}

template <int BM, int BN, int WAVES_M, int WAVES_N, bool AK, bool BKM, int EPI,
          bool OUT_F32, bool EDGE>
int launch_cfg(const GemmArgs& in, hipStream_t stream) {
  GemmArgs g = in;
  g.tiles_m = (g.M + BM - 1) / BM;
  g.tiles_n = (g.N + BN - 1) / BN;
  constexpr int NT = WAVES_M * WAVES_N * 64;
  constexpr size_t lds = 2 * (size_t)(BM + BN) * BK * 2;
  auto kern = gemm_bf16_kernel<BM, BN, WAVES_M, WAVES_N, AK, BKM, EPI, OUT_F32, EDGE>;
  static thread_local bool attr_set = false;
  if (!attr_set) {
    AXN_HIP_TRY(hipFuncSetAttribute((const void*)kern,
                                    hipFuncAttributeMaxDynamicSharedMemorySize,
                                    (int)lds));
    attr_set = true;
  }
  const long long nwg = (long long)g.tiles_m * g.tiles_n;
  if (nwg > 0x7fffffffLL) {
    set_error("gemm: too many output tiles (%lld)", nwg);
    return AXN_ELIMIT;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)nwg), dim3(NT), lds, stream, g);
  AXN_HIP_TRY(hipGetLastError());
  return AXN_OK;
}

// Tile selection.  Large aligned problems take 256 x 256 tiles on 8 waves;
// problems that would leave most of the 256 CUs idle at that size, and ragged
// ones, take 128 x 128 tiles with bounds checks.
template <bool AK, bool BKM, int EPI, bool OUT_F32>
int launch_shape(const GemmArgs& g, hipStream_t stream) {
  const bool aligned256 = (g.M % 256 == 0) && (g.N % 256 == 0) && (g.Kc % BK == 0);
  const long long tiles256 = (long long)((g.M + 255) / 256) * ((g.N + 255) / 256);
  if (aligned256 && tiles256 >= 192)
    return launch_cfg<256, 256, 2, 4, AK, BKM, EPI, OUT_F32, false>(g, stream);
  const bool aligned128 = (g.M % 128 == 0) && (g.N % 128 == 0) && (g.Kc % BK == 0);
  if (aligned128)
    return launch_cfg<128, 128, 2, 2, AK, BKM, EPI, OUT_F32, false>(g, stream);
  return launch_cfg<128, 128, 2, 2, AK, BKM, EPI, OUT_F32, true>(g, stream);
}

}  // namespace

int launch_gemm_bf16(GemmLayout layout, const GemmArgs& g, int epilogue,
                     bool out_f32, hipStream_t stream) {
  switch (layout) {
    case GEMM_NT:
      if (out_f32) break;
      switch (epilogue) {
        case AXN_EPI_NONE:
          return launch_shape<true, true, AXN_EPI_NONE, false>(g, stream);
        case AXN_EPI_BIAS:
          return launch_shape<true, true, AXN_EPI_BIAS, false>(g, stream);
        case AXN_EPI_BIAS_GELU:
          return launch_shape<true, true, AXN_EPI_BIAS_GELU, false>(g, stream);
        case AXN_EPI_GELU:
          return launch_shape<true, true, AXN_EPI_GELU, false>(g, stream);
      }
      break;
    case GEMM_NN:
      if (out_f32 || epilogue != AXN_EPI_NONE) break;
      return launch_shape<true, false, AXN_EPI_NONE, false>(g, stream);
    case GEMM_TN:
      if (epilogue != AXN_EPI_NONE) break;
      return out_f32 ? launch_shape<false, false, AXN_EPI_NONE, true>(g, stream)
                     : launch_shape<false, false, AXN_EPI_NONE, false>(g, stream);
  }
  set_error("gemm: unsupported layout/epilogue/output combination");
  return AXN_EINVAL;
}

}  // namespace axn
