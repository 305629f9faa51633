// bf16 MFMA GEMM for gfx950 (MI355X): the three shard GEMMs of the
// tensor-parallel Linear layer,
//   forward  Y  = X  W^T   (axonn/intra_layer/fully_connected.py:118)
//   dgrad    dX = dY W     (fully_connected.py:140)
//   wgrad    dW = dY^T X   (fully_connected.py:147-151)
// templated over the operand storage orders: an operand is "K-major" when the
// contraction index is contiguous in memory ([rows][Kc]) and "MN-major" when it
// is strided ([Kc][rows]).  No transposed copy of an operand is ever made.
//
// Common to both kernel families in this file
//   * fp32 accumulation in registers; a workgroup owns a BM x BN output tile and
//     walks the contraction through LDS tiles.
//   * LDS layouts per storage order such that fragment reads are free of bank
//     conflicts on the 64-bank LDS; MN-major tiles are read with the transposing
//     ds_read_b64_tr_b16.
//   * The MFMA is issued with the operands swapped (D^T = B^T A^T), so that a lane
//     holds consecutive output columns of a row and writes 16 contiguous bytes.
//   * Workgroup ids are remapped so that each of the 8 XCDs (private L2 each)
//     works on a compact block of neighbouring tiles.
//
// One-wave-per-SIMD kernels (solo_gemm: gemm_*_solo_kernel at 256 x 256 and 128 x 128
// tiles, gemm_*_rest_kernel at 256 x 128, gemm_*_swiglu_kernel; shapes made of whole
// tiles, contraction % 64 == 0, operands below 2 GiB): 4 waves, one per SIMD, each a
// quarter of the tile on v_mfma_f32_16x16x32_{bf16,f16}; operand tiles go global -> LDS
// directly (buffer loads to LDS, 16 bytes per lane, no registers) into a ring of five
// 64-deep tiles; each wave pipelines its share of the copies and its LDS fragment reads
// between its own MFMAs; a permuted row order of the column operand's fragments leaves
// a lane with 8 consecutive output columns, stored straight from the accumulators.
// launch_shape / launch_whole choose the tile and cut a problem whose last round of
// large tiles would be at most half full into full rounds and a rest; a workspace
// variant splits the contraction of problems with few tiles over workgroups; the
// gate/up forward of a gated MLP gathers its column operand from two weight matrices
// and applies silu(gate) * up in the epilogue.
//
// Register-staged kernel (gemm_*_kernel: any shape with N % 8 == 0 and K % 8 == 0):
// 128 x 128 tiles, v_mfma_f32_32x32x16, operand tiles staged global -> VGPR -> LDS with
// bounds checks, one barrier per step, epilogue transposed through LDS; ragged shapes,
// contractions that are not multiples of 64, operands of 2 GiB and more.
#include <atomic>
#include <cmath>
#include <functional>
#include <queue>
#include <vector>
#include <utility>

#include "axn_internal.h"

namespace axn {
namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(8))) short s16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

constexpr int BK = 64;          // contraction elements per step
constexpr int NUM_XCD = 8;      // MI355X: 8 accelerator dies, round-robin dispatch
constexpr int EPI_LD = 68;      // floats per row of the epilogue staging buffer
// Internal epilogue of the gate/up forward: the tile's B rows are 64 gate rows and 64 up
// rows per wave, and the output is silu(gate) * up (not part of the public axn_epilogue).
constexpr int EPI_SWIGLU = 100;
// Internal: no epilogue, but the contraction runs through two operand pairs one after the
// other (C = A B + A2 B2).
constexpr int EPI_PAIR = 101;
#define LDS_PTR(T, p) ((__attribute__((address_space(3))) T*)(p))

template <int... I, class F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F&& f) {
  (f(std::integral_constant<int, I>{}), ...);
}
// Calls f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>).
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(std::make_integer_sequence<int, N>{}, f);
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
      s16x8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
      return __builtin_bit_cast(bf16x8, v);
    }
  }
};

// Epilogue of 8 consecutive columns of one output row, held in fp32: bias,
// exact GELU with optional save of the pre-activation, accumulation into the
// existing output (beta), conversion and one 16- or 32-byte store.
// HALF: the 16-bit storage type is IEEE half instead of bfloat16.
template <int EPI, bool OUT_F32, bool HALF>
__device__ __forceinline__ void store_row8(float (&v)[8], const GemmArgs& g, int row, int col) {
  using lp = std::conditional_t<HALF, _Float16, __bf16>;
  using lpx8 = std::conditional_t<HALF, f16x8, bf16x8>;
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
      lpx8 z;
#pragma unroll
      for (int e = 0; e < 8; ++e) z[e] = (lp)v[e];
      *(lpx8*)(g.Z + o) = z;
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
      const lpx8 old = *(const lpx8*)C;
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] += (float)old[e];
    }
    lpx8 y;
#pragma unroll
    for (int e = 0; e < 8; ++e) y[e] = (lp)v[e];
    *(lpx8*)C = y;
  }
}

// Epilogue of the gate/up forward for 8 consecutive columns of one row: both
// pre-activations are rounded to the 16-bit type (and stored, if asked for: the backward
// pass reads them), and the output is computed from the rounded values, so that it equals
// the separate activation kernel applied to the stored pre-activations bit for bit.
template <bool HALF>
__device__ __forceinline__ void store_swiglu8(const float (&vg)[8], const float (&vu)[8],
                                              const GemmArgs& g, int row, int col) {
  using lp = std::conditional_t<HALF, _Float16, __bf16>;
  using lpx8 = std::conditional_t<HALF, f16x8, bf16x8>;
  const int64_t o = (int64_t)row * g.ldc + col;
  lpx8 gate, up, out;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    gate[e] = (lp)vg[e];
    up[e] = (lp)vu[e];
    const float x = (float)gate[e];
    out[e] = (lp)(x * sigmoid_f(x) * (float)up[e]);
  }
  if (g.G != nullptr) *(lpx8*)(g.G + o) = gate;
  if (g.U != nullptr) *(lpx8*)(g.U + o) = up;
  *(lpx8*)((uint16_t*)g.C + o) = out;
}

// Writes a wave's accumulators to C with the fused epilogue.  With the operands
// swapped, lane l register r of acc[i][j] is the output element
//   row = l % 32,  col = 8 * (r / 4) + 4 * (l / 32) + r % 4
// of the 32 x 32 block (i, j) of the wave's tile.  Blocks are transposed through
// a per-wave LDS buffer (32 rows x 64 fp32 columns, padded) so that every lane
// then owns 8 consecutive columns of one row.  The caller must have made sure
// that no wave still reads operand tiles from LDS.
template <int FM, int FN, int EPI, bool OUT_F32, bool EDGE, bool HALF>
__device__ __forceinline__ void store_tile(const f32x16 (&acc)[FM][FN], const GemmArgs& g,
                                           char* lds, int wave, int lane, int row0,
                                           int col0) {
  constexpr int WTN = FN * 32;
  constexpr int EPC = (WTN < 64) ? WTN : 64;  // columns per staging pass
  constexpr int JP = EPC / 32;                // fragments per pass
  constexpr int LPR = EPC / 8;                // lanes per row on read-back
  constexpr int RPI = 64 / LPR;               // rows per read-back iteration
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
        const int row = row0 + i * 32 + r;
        const int col = col0 + jp * EPC + c;
        if (EDGE && (row >= g.M || col >= g.N)) continue;
        store_row8<EPI, OUT_F32, HALF>(v, g, row, col);
      }
    }
  }
}

// ---------------------------------------------------------------------------
// LDS fragment reads as inline assembly: the compiler neither waits for them nor
// orders them behind outstanding copies; the kernels place the waits themselves.
// ---------------------------------------------------------------------------
template <int IMM>
__device__ __forceinline__ bf16x8 lds_read_b128(uint32_t addr) {
  bf16x8 v;
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(IMM));
  return v;
}
template <int IMM>
__device__ __forceinline__ s16x4 lds_read_tr16_b64(uint32_t addr) {
  s16x4 v;
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(IMM));
  return v;
}

// ---------------------------------------------------------------------------
// One-wave-per-SIMD kernel: 64-deep operand tiles, v_mfma_f32_16x16x32_bf16.
// ---------------------------------------------------------------------------
// Measured on MI355X, which runs these kernels power-limited: at equal FLOPs the
// 16x16x32 MFMA sustains about 10 % more clock than 32x32x16 (half the
// accumulator traffic per FLOP), and LDS fragment reads cost clock rather than
// issue slots.
//
// One operand tile: 256 rows x 64 deep (32 KiB), copied by 4 waves (8 copies
// each) and read as 16-row x 32-deep MFMA fragments (lane l: row l % 16,
// contraction elements 8 (l / 16) .. + 8).
//   K-major  tile [256][64] : 128-byte rows = whole cache lines of the operand;
//                             16-byte chunk c of row r lives at chunk c ^ ((r >> 1) & 7),
//                             which spreads the 16 lanes of a fragment quarter over
//                             all 64 banks
//   MN-major tile [64][256] : 512-byte rows; 64-byte chunk c of contraction row k
//                             lives at chunk c ^ (k & 3); read with the transposing
//                             ds_read_b64_tr_b16 (two per fragment)
//
// PERMUTED (the operand that supplies the output columns): fragment j holds the
// tile rows 32 (j / 2) + 8 (q / 4) + 4 (j % 2) + q % 4 in its lane-rows
// q = 0..15 instead of 16 j + q.  The MFMA result then leaves lane l with
// columns 8 (l / 16) .. + 3 of a 32-column group in block 2t and .. + 4 .. + 7
// in block 2t + 1: eight consecutive output columns per lane, stored from
// registers without a transpose through LDS.  Its K-major swizzle is
// chunk ^ (((r >> 1) & 1) | ((r >> 3) & 3) << 1), which again gives the 16 rows
// of a fragment quarter 16 distinct (row parity, chunk) pairs.
template <bool KMAJOR, bool PERMUTED, int ROWS_ /* 256 or 128 */>
struct DeepOperand {
  static constexpr int ROWS = ROWS_;
  static constexpr int PK = 64;
  static constexpr int BYTES = ROWS * PK * 2;      // 32 or 16 KiB
  static constexpr int NW = 4;
  static constexpr int DMA_N = BYTES / 1024 / NW;  // 8 or 4 copies per wave
  static constexpr int FR = ROWS / 32;             // 16-row fragments of a wave's half of the rows
  static constexpr int NADDR = KMAJOR ? 2 : FR / 2;
  static constexpr int LPR = ROWS / 8;             // MN-major: lanes per contraction row of a copy

  __device__ __forceinline__ static int kmajor_swizzle(int row) {
    return PERMUTED ? (((row >> 1) & 1) | (((row >> 3) & 3) << 1)) : ((row >> 1) & 7);
  }

  // Byte offset of this lane's 16 bytes for copy 0 of the tile at contraction
  // offset 0, and the uniform stride from copy i to i + 1.  Lane l of copy i
  // lands at tile + (4 i + wave) * 1024 + 16 l; the swizzle is applied here.
  __device__ __forceinline__ static uint32_t dma_offset(int64_t ld, int row0, int wave,
                                                        int lane, uint32_t& istride) {
    if (KMAJOR) {
      const int row = wave * 8 + (lane >> 3);              // + 32 i
      const int c = (lane & 7) ^ kmajor_swizzle(row);      // 32 i does not change the swizzle
      istride = (uint32_t)(32 * ld * 2);
      return (uint32_t)(((int64_t)(row0 + row) * ld + c * 8) * 2);
    } else {
      constexpr int KPI = 64 / LPR;                    // contraction rows per copy: 2 or 4
      const int k = wave * KPI + lane / LPR;           // + 4 KPI i
      const int p16 = lane % LPR;
      const int c64 = (p16 >> 2) ^ (k & 3);            // 4 KPI i does not change k & 3
      istride = (uint32_t)(4 * KPI * ld * 2);
      return (uint32_t)(((int64_t)k * ld + row0 + (c64 * 4 + (p16 & 3)) * 8) * 2);
    }
  }

  // Copy I of the tile (LDS kilobytes 4 I .. 4 I + 3); it reads the operand IO copy strides
  // behind copy 0 (IO = I unless the tile's rows are gathered from two places).
  template <int I, int IO = I>
  __device__ __forceinline__ static void dma_one(__amdgpu_buffer_rsrc_t rsrc, uint32_t voff,
                                                 uint32_t tile_ofs, uint32_t istride,
                                                 char* lds_tile, int wave) {
    static_assert(I >= 0 && I < DMA_N && IO >= 0 && IO < DMA_N, "copy index");
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, LDS_PTR(void, lds_tile + (NW * I + wave) * 1024),
                                             16, (int)voff, (int)(tile_ofs + IO * istride), 0, 0);
  }

  // Per-lane LDS byte offsets (relative to the tile) the fragment reads start from.
  //   K-major : a[s] for the 32-deep step s; fragments add whole rows (frag_offset),
  //             which leave the swizzle unchanged.
  //   MN-major: a[i >> 1] for fragment i, step s adds 32 rows.  The 16 lanes of a
  //             block address contraction rows 8 (l / 16) + (l & 15) / 4 and 4
  //             columns each; the transposing read hands lane i of the block the
  //             column that lane 4 (i / 4) .. addressed, rows 8 (l / 16) + 0..3
  //             (second read: + 4..7).
  __device__ __forceinline__ static void read_bases(uint32_t (&a)[NADDR], int wrow0, int lane) {
    const int q = lane & 15;
    if (KMAJOR) {
      const int r = wrow0 + (PERMUTED ? 8 * (q >> 2) + (q & 3) : q);
      const int swz = kmajor_swizzle(r);
#pragma unroll
      for (int st = 0; st < 2; ++st)
        a[st] = (uint32_t)(r * 128 + (((st * 4 + (lane >> 4)) ^ swz) << 4));
    } else {
      const int kq = q >> 2;
      const int k = 8 * (lane >> 4) + kq;
#pragma unroll
      for (int h = 0; h < NADDR; ++h) {
        const int colbyte = (wrow0 + h * 32 + (PERMUTED ? 8 : 4) * (lane & 3)) * 2;
        a[h] = (uint32_t)(k * (ROWS * 2) + ((((colbyte >> 6) ^ kq) << 6) | (colbyte & 63)));
      }
    }
  }

  // Fragment I of the 32-deep step ST of the tile.
  template <int ST, int I>
  __device__ __forceinline__ static void read_frag(bf16x8& f, const uint32_t (&a)[NADDR]) {
    if constexpr (KMAJOR) {
      constexpr int row_ofs = PERMUTED ? 32 * (I >> 1) + 4 * (I & 1) : 16 * I;
      f = lds_read_b128<row_ofs * 128>(a[ST]);
    } else {
      constexpr int col_ofs = PERMUTED ? 4 * (I & 1) : 16 * (I & 1);  // elements
      const s16x4 lo = lds_read_tr16_b64<ST * 32 * ROWS * 2 + col_ofs * 2>(a[I >> 1]);
      const s16x4 hi = lds_read_tr16_b64<(ST * 32 + 4) * ROWS * 2 + col_ofs * 2>(a[I >> 1]);
      f = __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
    }
  }
};

// Waits for every outstanding LDS read; the fragments flow through the
// statement, so no MFMA on them can move above the wait.
__device__ __forceinline__ void wait_all_fragments(bf16x8 (&fa)[8], bf16x8 (&fb)[8]) {
  asm volatile("s_waitcnt lgkmcnt(0)"
               : "+v"(fa[0]), "+v"(fa[1]), "+v"(fa[2]), "+v"(fa[3]), "+v"(fa[4]), "+v"(fa[5]),
                 "+v"(fa[6]), "+v"(fa[7]), "+v"(fb[0]), "+v"(fb[1]), "+v"(fb[2]), "+v"(fb[3]),
                 "+v"(fb[4]), "+v"(fb[5]), "+v"(fb[6]), "+v"(fb[7]));
}
__device__ __forceinline__ void wait_all_fragments(bf16x8 (&fa)[8], bf16x8 (&fb)[4]) {
  asm volatile("s_waitcnt lgkmcnt(0)"
               : "+v"(fa[0]), "+v"(fa[1]), "+v"(fa[2]), "+v"(fa[3]), "+v"(fa[4]), "+v"(fa[5]),
                 "+v"(fa[6]), "+v"(fa[7]), "+v"(fb[0]), "+v"(fb[1]), "+v"(fb[2]), "+v"(fb[3]));
}
__device__ __forceinline__ void wait_all_fragments(bf16x8 (&fa)[4], bf16x8 (&fb)[4]) {
  asm volatile("s_waitcnt lgkmcnt(0)"
               : "+v"(fa[0]), "+v"(fa[1]), "+v"(fa[2]), "+v"(fa[3]), "+v"(fb[0]), "+v"(fb[1]),
                 "+v"(fb[2]), "+v"(fb[3]));
}
// Passes a row of accumulators through a statement (see the end of the kernel).
__device__ __forceinline__ void settle_accumulators(f32x4 (&a)[8]) {
  asm volatile("s_nop 3"
               : "+a"(a[0]), "+a"(a[1]), "+a"(a[2]), "+a"(a[3]), "+a"(a[4]), "+a"(a[5]),
                 "+a"(a[6]), "+a"(a[7]));
}
__device__ __forceinline__ void settle_accumulators(f32x4 (&a)[4]) {
  asm volatile("s_nop 3" : "+a"(a[0]), "+a"(a[1]), "+a"(a[2]), "+a"(a[3]));
}
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// TILE = 256: 4 waves, one per SIMD, each owning 128 x 128 of the 256 x 256 tile:
// 8 x 8 blocks of 16 x 16, 256 accumulator registers, 64 MFMAs per 32-deep step.
// A wave pipelines against itself: while the MFMAs of one step run on one
// register set (8 + 8 fragments), the fragments of the next step are read into
// the other, one fragment between two MFMAs.
//
// LDS holds a ring of 5 operand tiles (160 KiB); the tiles A0 B0 A1 B1 A2 ... of
// the contraction stages take the slots 0 1 2 3 4 0 1 ...  Stage p (64 deep):
//   step 0 : MFMAs | this wave's 8 copies of A(p+2) | reads of (p, 1)
//   step 1 : wait for own copies of A(p+1), B(p+1); barrier;
//            MFMAs | this wave's 8 copies of B(p+2) | reads of (p+1, 0)
// At the barrier every wave holds the last fragments of stage p in registers, so
// both of its slots are free: B(p+2) takes A(p)'s, A(p+3) (next step 0) B(p)'s.
// The copies come first in a step, the reads second: a tile has at least a whole
// stage (128 MFMAs per wave) to land.
//
// TILE = 128 is the same schedule on a 128 x 128 tile for problems that do not
// fill the chip with 256 x 256 tiles: 64 x 64 per wave (4 x 4 blocks, 16 MFMAs per
// step, 4 copies per tile and wave), an 80 KiB ring, two workgroups per CU.
//
// BM x BN = 256 x 128 is the tile of the launches that finish a problem after its full
// rounds of 256 x 256 tiles: a rest of r <= 128 large tiles makes 2 r <= 256 of these,
// one per CU, and needs 3/4 of the global -> LDS bytes per MFMA of the 128 x 128 tile.
// Its ring has five slots of the larger (A) tile's size.
template <int BM, int BN, bool A_KMAJOR, bool B_KMAJOR, int EPI, bool OUT_F32, bool HALF>
__device__ __forceinline__ void solo_gemm(const GemmArgs& g) {
  constexpr int WTM = BM / 2, WTN = BN / 2, FRM = BM / 32, FRN = BN / 32;
  constexpr int PK = 64, NSLOT = 5;
  constexpr int NM = FRM * FRN;         // MFMAs per step
  using OA = DeepOperand<A_KMAJOR, false, BM>;
  using OB = DeepOperand<B_KMAJOR, true, BN>;
  constexpr uint32_t SLOT = OA::BYTES > OB::BYTES ? OA::BYTES : OB::BYTES;  // 32 or 16 KiB
  constexpr int NCA = OA::DMA_N, NCB = OB::DMA_N;  // copies per tile and wave
  constexpr int NFRAG = FRM + FRN;                 // fragment reads per step
  constexpr int READ_EVERY = (NM / 2) / NFRAG;     // a fragment read every .. MFMAs, first half of a step
  constexpr int COPY_EVERY_A = (NM / 2) / NCA;     // a copy every .. MFMAs, second half
  constexpr int COPY_EVERY_B = (NM / 2) / NCB;
  static_assert((BM == 256 || BM == 128) && (BN == 256 || BN == 128) && BM >= BN,
                "tile sizes with a schedule below");
  static_assert(READ_EVERY >= 1 && COPY_EVERY_A >= 1 && COPY_EVERY_B >= 1, "schedule fits a step");
  // Gate/up forward: the B tile's 256 rows are, per 128-row half (one wave column), 64
  // rows of the gate weights and the 64 rows of the up weights with the same indices, so
  // that a lane ends with a gate value in accumulator block j and the up value of the
  // same output element in block j + 4.  The tile covers 128 output columns.
  constexpr bool SWIGLU = EPI == EPI_SWIGLU;
  // Two-term product: stages 0 .. k_first / 64 - 1 copy from (A, B), the others from
  // (A2, B2); everything behind the copies is unchanged.
  constexpr bool PAIR = EPI == EPI_PAIR;
  static_assert(!PAIR || (A_KMAJOR && !B_KMAJOR), "the two-term product is the dgrad layout");
  static_assert(!SWIGLU || (BM == 256 && BN == 256 && A_KMAJOR && B_KMAJOR && !OUT_F32),
                "the gate/up forward runs on the 256 x 256 tile with contraction-contiguous operands");

  extern __shared__ __attribute__((aligned(16))) char lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;

  f32x4 acc[FRM][FRN];

  const uint32_t a_bytes = (uint32_t)((int64_t)(A_KMAJOR ? g.M : g.Kc) * g.lda * 2);
  const uint32_t b_bytes = (uint32_t)((int64_t)(B_KMAJOR ? g.N : (PAIR ? g.k_first : g.Kc)) * g.ldb * 2);
  const __amdgpu_buffer_rsrc_t ra_rsrc =
      __builtin_amdgcn_make_buffer_rsrc((void*)g.A, 0, (int)a_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t rb_rsrc =
      __builtin_amdgcn_make_buffer_rsrc((void*)g.B, 0, (int)b_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t rb2_rsrc =
      __builtin_amdgcn_make_buffer_rsrc((void*)(SWIGLU ? g.B2 : g.B), 0, (int)b_bytes, 0x00020000);
  // the pair the copies read from (PAIR only: switched once, two stages before the
  // first stage of the second pair)
  __amdgpu_buffer_rsrc_t ra_cur = ra_rsrc, rb_cur = rb_rsrc;
  uint32_t a_is = 0, b_is = 0, va = 0, vb = 0;   // per-lane copy offsets of the current tile
  const uint32_t a_step = (uint32_t)((A_KMAJOR ? (int64_t)PK : (int64_t)PK * g.lda) * 2);
  const uint32_t b_step = (uint32_t)((B_KMAJOR ? (int64_t)PK : (int64_t)PK * g.ldb) * 2);
  uint32_t ka = 0, kb = 0;  // byte offsets of the next A / B tile to copy
  uint32_t wslot = 0;       // ring slot (byte offset) the next copied tile takes

  const uint32_t lds0 = (uint32_t)(uintptr_t)LDS_PTR(char, lds);
  uint32_t ra0[OA::NADDR], rb0[OB::NADDR];
  OA::read_bases(ra0, wm * WTM, lane);
  OB::read_bases(rb0, wn * WTN, lane);
#pragma unroll
  for (int i = 0; i < OA::NADDR; ++i) ra0[i] += lds0;
#pragma unroll
  for (int i = 0; i < OB::NADDR; ++i) rb0[i] += lds0;

  auto next_slot = [&](uint32_t s_) { return s_ + SLOT == NSLOT * SLOT ? 0u : s_ + SLOT; };
  auto copy_a = [&](auto c_) {
    if constexpr (PAIR)
      OA::template dma_one<decltype(c_)::value>(ra_cur, va, ka, a_is, lds + wslot, wave);
    else
      OA::template dma_one<decltype(c_)::value>(ra_rsrc, va, ka, a_is, lds + wslot, wave);
  };
  auto copy_b = [&](auto c_) {
    constexpr int I = decltype(c_)::value;
    if constexpr (SWIGLU) {
      // copies 4 h + {0, 1} of a half h bring 64 gate rows, 4 h + {2, 3} the 64 up rows
      // with the same indices: both are rows 64 h + 32 (I % 2) .. of their matrix
      constexpr int IO = 2 * (I / 4) + I % 2;
      OB::template dma_one<I, IO>(I % 4 < 2 ? rb_rsrc : rb2_rsrc, vb, kb, b_is, lds + wslot, wave);
    } else if constexpr (PAIR) {
      OB::template dma_one<I>(rb_cur, vb, kb, b_is, lds + wslot, wave);
    } else {
      OB::template dma_one<I>(rb_rsrc, vb, kb, b_is, lds + wslot, wave);
    }
  };
  auto a_done = [&]() { ka += a_step; wslot = next_slot(wslot); };
  auto b_done = [&]() { kb += b_step; wslot = next_slot(wslot); };

  bf16x8 fa0[FRM], fb0[FRN], fa1[FRM], fb1[FRN];  // register sets of steps 0 / 1
  // fragment f of FRM + FRN (A fragments, then B fragments) of step ST of the stage
  // whose tiles sit at sa / sb, into register set ST
  auto read = [&](auto st_, auto f_, uint32_t sa, uint32_t sb) {
    constexpr int ST = decltype(st_)::value, f = decltype(f_)::value;
    bf16x8(&fa)[FRM] = ST ? fa1 : fa0;
    bf16x8(&fb)[FRN] = ST ? fb1 : fb0;
    if constexpr (f < FRM) {
      uint32_t ra[OA::NADDR];
#pragma unroll
      for (int i = 0; i < OA::NADDR; ++i) ra[i] = ra0[i] + sa;
      OA::template read_frag<ST, f>(fa[f], ra);
    } else {
      uint32_t rb[OB::NADDR];
#pragma unroll
      for (int i = 0; i < OB::NADDR; ++i) rb[i] = rb0[i] + sb;
      OB::template read_frag<ST, f - FRM>(fb[f - FRM], rb);
    }
  };
  uint32_t sa = 0, sb = SLOT;  // slots of the current stage's tiles

  // HAS2: stage p + 2 exists (its tiles are copied during this stage);
  // LAST: no stage follows.
  auto stage = [&](auto has2_, auto last_) {
    constexpr bool HAS2 = decltype(has2_)::value;
    constexpr bool LAST = decltype(last_)::value;
    const uint32_t na = next_slot(sb), nb = next_slot(na);  // slots of stage p + 1
    static_for<2>([&](auto st_) {
      constexpr int ST = decltype(st_)::value;
      bf16x8(&fa)[FRM] = ST ? fa1 : fa0;
      bf16x8(&fb)[FRN] = ST ? fb1 : fb0;
      wait_all_fragments(fa, fb);  // every read of this set was issued during the previous step
      if constexpr (ST == 1 && !LAST) {
        if (HAS2) wait_vmcnt<NCA>();  // A(p+2) may be in flight
        else wait_vmcnt<0>();
        __builtin_amdgcn_s_barrier();
      }
      __builtin_amdgcn_sched_barrier(0);
      static_for<NM>([&](auto m_) {
        constexpr int m = decltype(m_)::value;
        constexpr int i = m / FRN, j = m % FRN;
        // Inline assembly pins the register classes (accumulators in AGPRs, fragments
        // in VGPRs): with the builtin the allocator moves two-instruction
        // (transposed) fragments through AGPRs and spills.  No MFMA hazard can arise:
        // fragments come from LDS behind s_waitcnt, and an accumulator is touched
        // again only NM - 1 (at least 15) independent MFMAs later.
        // (fragments are opaque 16-byte registers: the mnemonic alone names the type)
        if constexpr (HALF)
          asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0"
                       : "+a"(acc[i][j])
                       : "v"(fb[j]), "v"(fa[i]));
        else
          asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0"
                       : "+a"(acc[i][j])
                       : "v"(fb[j]), "v"(fa[i]));
        constexpr int CE = ST == 0 ? COPY_EVERY_A : COPY_EVERY_B;  // step 0 copies A, step 1 B
        constexpr int NCX = ST == 0 ? NCA : NCB;
        // Copies in the first half of a step, fragment reads in the second: a copy is issued
        // as soon as the barrier (step 1) or the previous step (step 0) has freed its slot,
        // which gives the tile a quarter of a stage more to arrive than the other order
        // (measured: +2.6 % on the step, +7 % on the MLP shard); the reads still have half
        // a step to return.
        constexpr int mc = m;            // position in the copying half
        constexpr int mr = m - NM / 2;   // position in the reading half
        if constexpr (mr >= 0 && mr < NM / 2 && mr % READ_EVERY == 0 && mr / READ_EVERY < NFRAG) {
          if constexpr (ST == 0) read(std::integral_constant<int, 1>{},
                                      std::integral_constant<int, mr / READ_EVERY>{}, sa, sb);
          else if constexpr (!LAST) read(std::integral_constant<int, 0>{},
                                         std::integral_constant<int, mr / READ_EVERY>{}, na, nb);
        }
        // (an independent statement: a read and a copy may fall behind the same MFMA)
        static_assert((NM / 2) / CE >= NCX, "every copy of the tile has a place in the half step");
        if constexpr (HAS2 && mc >= 0 && mc < NM / 2 && mc % CE == CE - 1 && mc / CE < NCX) {
          if constexpr (ST == 0) copy_a(std::integral_constant<int, mc / CE>{});
          else copy_b(std::integral_constant<int, mc / CE>{});
        }
        __builtin_amdgcn_sched_barrier(0);
      });
      if constexpr (HAS2 && ST == 0) a_done();
      if constexpr (HAS2 && ST == 1) b_done();
    });
    sa = na;
    sb = nb;
  };
  using T = std::true_type;
  using F = std::false_type;

  // This workgroup's tile and, for a split contraction, its part: KP stages from stage s0 on.
  int tm, tn, split = 0;
  {
    int pid = blockIdx.x - g.wg_first;
    if (g.splits > 1) {
      split = pid / (g.tiles_m * g.tiles_n);
      pid -= split * (g.tiles_m * g.tiles_n);
    }
    tile_of_workgroup(pid, g.tiles_m, g.tiles_n, tm, tn);
  }
  const int KP = (g.splits > 1 ? g.k_split : g.Kc) / PK;
  const int s0 = split * KP;
  const int m0 = tm * BM, n0 = tn * (SWIGLU ? BN / 2 : BN);
  va = OA::dma_offset(g.lda, m0, wave, lane, a_is);
  vb = OB::dma_offset(g.ldb, n0, wave, lane, b_is);
  ka = (uint32_t)s0 * a_step;
  kb = (uint32_t)s0 * b_step;

  // A0 B0 (A1 B1) up front.
  static_for<NCA>(copy_a); a_done();
  static_for<NCB>(copy_b); b_done();
  if (KP > 1) {
    static_for<NCA>(copy_a); a_done();
    static_for<NCB>(copy_b); b_done();
  }
  // The accumulators are cleared here, while the first tiles are on their way: left
  // to itself the compiler clears them where they are first used, behind the wait.
#pragma unroll
  for (int i = 0; i < FRM; ++i)
#pragma unroll
    for (int j = 0; j < FRN; ++j) acc[i][j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
  for (int i = 0; i < FRM; ++i) settle_accumulators(acc[i]);
  if (KP > 1) {
    wait_vmcnt<NCA + NCB>();
  } else {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  }
  __builtin_amdgcn_s_barrier();

  static_for<NFRAG>([&](auto f_) { read(std::integral_constant<int, 0>{}, f_, sa, sb); });

  if constexpr (PAIR) {
    const int kp1 = g.k_first / PK;  // >= 2: the stages copied up front are of the first pair
    const uint32_t b2_bytes = (uint32_t)((int64_t)(g.Kc - g.k_first) * g.ldb * 2);
    for (int p = 0; p < KP - 2; ++p) {
      if (p == kp1 - 2) {  // this stage copies the tiles of stage kp1, the second pair's first
        ra_cur = __builtin_amdgcn_make_buffer_rsrc((void*)g.A2, 0, (int)a_bytes, 0x00020000);
        rb_cur = __builtin_amdgcn_make_buffer_rsrc((void*)g.B2, 0, (int)b2_bytes, 0x00020000);
        ka = 0;
        kb = 0;
      }
      stage(T{}, F{});
    }
  } else {
    for (int p = 0; p < KP - 2; ++p) stage(T{}, F{});
  }
  if (KP > 1) stage(F{}, F{});
  stage(F{}, T{});
  // The compiler does not know that the statements above are MFMAs: left alone it
  // copies an accumulator out of its AGPRs right behind the MFMA that writes it,
  // before the result has left the pipeline.  Every accumulator is therefore
  // passed through a statement that follows the last MFMA by more than its
  // latency; the epilogue can only read the values these statements return.
  asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
#pragma unroll
  for (int i = 0; i < FRM; ++i) settle_accumulators(acc[i]);
  // With the permuted column fragments a lane owns, per block row i and block
  // pair t, the 8 consecutive columns 32 t + 8 (l / 16) .. + 7 of row 16 i + l % 16:
  // they go out straight from the registers, 64 contiguous bytes per row and
  // instruction.
  const int orow = m0 + wm * WTM + (lane & 15);
  const int ocol = n0 + wn * WTN + 8 * (lane >> 4);
  if constexpr (SWIGLU) {
    // blocks 0..3 of a lane's row hold 64 gate columns, blocks 4..7 the up values of the
    // same columns
    const int hcol = n0 + wn * (WTN / 2) + 8 * (lane >> 4);
#pragma unroll
    for (int i = 0; i < FRM; ++i)
#pragma unroll
      for (int t = 0; t < FRN / 4; ++t) {
        const f32x4 gl = acc[i][2 * t], gh = acc[i][2 * t + 1];
        const f32x4 ul = acc[i][2 * t + FRN / 2], uh = acc[i][2 * t + 1 + FRN / 2];
        const float vg[8] = {gl[0], gl[1], gl[2], gl[3], gh[0], gh[1], gh[2], gh[3]};
        const float vu[8] = {ul[0], ul[1], ul[2], ul[3], uh[0], uh[1], uh[2], uh[3]};
        store_swiglu8<HALF>(vg, vu, g, orow + 16 * i, hcol + 32 * t);
      }
  } else {
    GemmArgs go = g;  // a split writes its own fp32 partial product
    if (OUT_F32 && g.splits > 1) go.C = (float*)g.C + (int64_t)split * g.M * g.ldc;
#pragma unroll
    for (int i = 0; i < FRM; ++i)
#pragma unroll
      for (int t = 0; t < FRN / 2; ++t) {
        const f32x4 lo = acc[i][2 * t], hi = acc[i][2 * t + 1];
        float v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        store_row8<(PAIR ? (int)AXN_EPI_NONE : EPI), OUT_F32, HALF>(v, go, orow + 16 * i, ocol + 32 * t);
      }
  }
}

template <int TILE, bool A_KMAJOR, bool B_KMAJOR, int EPI, bool OUT_F32>
__global__ void __launch_bounds__(256) gemm_bf16_solo_kernel(const GemmArgs g) {
  solo_gemm<TILE, TILE, A_KMAJOR, B_KMAJOR, EPI, OUT_F32, false>(g);
}
template <int TILE, bool A_KMAJOR, bool B_KMAJOR, int EPI, bool OUT_F32>
__global__ void __launch_bounds__(256) gemm_f16_solo_kernel(const GemmArgs g) {
  solo_gemm<TILE, TILE, A_KMAJOR, B_KMAJOR, EPI, OUT_F32, true>(g);
}
// The 256 x 128 tile of the launches that finish a problem.
template <bool A_KMAJOR, bool B_KMAJOR, int EPI, bool OUT_F32>
__global__ void __launch_bounds__(256) gemm_bf16_rest_kernel(const GemmArgs g) {
  solo_gemm<256, 128, A_KMAJOR, B_KMAJOR, EPI, OUT_F32, false>(g);
}
template <bool A_KMAJOR, bool B_KMAJOR, int EPI, bool OUT_F32>
__global__ void __launch_bounds__(256) gemm_f16_rest_kernel(const GemmArgs g) {
  solo_gemm<256, 128, A_KMAJOR, B_KMAJOR, EPI, OUT_F32, true>(g);
}

// Weight gradient and input gradient of one layer in one launch, 256 x 256 tiles: the
// workgroups [gw.wg_first, gw.wg_first + gw's tiles) compute dW = dY^T X, the others dX = dY W.
// The host puts the problem with the longer tiles first; the dispatcher hands workgroups
// out in index order, so a CU takes a tile of the other product as soon as it is free.
template <bool HALF, bool DW_F32>
__global__ void __launch_bounds__(256) gemm_backward_kernel(const GemmArgs gw, const GemmArgs gd) {
  const int b = (int)blockIdx.x;
  if (b >= gw.wg_first && b < gw.wg_first + gw.tiles_m * gw.tiles_n)
    solo_gemm<256, 256, false, false, AXN_EPI_NONE, DW_F32, HALF>(gw);
  else
    solo_gemm<256, 256, true, false, AXN_EPI_NONE, false, HALF>(gd);
}

// The gate/up forward of a gated MLP: silu(A B^T) * (A B2^T), 256 rows x 128 columns of
// the output per workgroup (the MFMA work of a 256 x 256 tile).
__global__ void __launch_bounds__(256) gemm_bf16_swiglu_kernel(const GemmArgs g) {
  solo_gemm<256, 256, true, true, EPI_SWIGLU, false, false>(g);
}
__global__ void __launch_bounds__(256) gemm_f16_swiglu_kernel(const GemmArgs g) {
  solo_gemm<256, 256, true, true, EPI_SWIGLU, false, true>(g);
}

// ---------------------------------------------------------------------------
// Register-staged kernel.
// ---------------------------------------------------------------------------
template <int BM, int BN, int WAVES_M, int WAVES_N, bool A_KMAJOR, bool B_KMAJOR,
          int EPI, bool OUT_F32, bool EDGE, bool HALF>
__device__ __forceinline__ void staged_gemm(const GemmArgs& g) {
  constexpr int NT = WAVES_M * WAVES_N * 64;
  constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
  constexpr int FM = WTM / 32, FN = WTN / 32;
  static_assert(WTM % 32 == 0 && WTN % 32 == 0, "wave tile must be 32-aligned");
  using TA = OperandTile<BM, A_KMAJOR, NT, EDGE>;
  using TB = OperandTile<BN, B_KMAJOR, NT, EDGE>;
  constexpr int STAGE = TA::BYTES + TB::BYTES;
  static_assert(32 * EPI_LD * 4 * WAVES_M * WAVES_N <= 2 * STAGE,
                "epilogue staging must fit in the operand buffers");

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
  constexpr int KK = BK / 16;  // MFMA steps per staged tile

  TA::load(ra, g.A, g.lda, m0, g.M, 0, g.Kc, tid);
  TB::load(rb, g.B, g.ldb, n0, g.N, 0, g.Kc, tid);
  TA::store(ra, lds, tid);
  TB::store(rb, lds + TA::BYTES, tid);
  __syncthreads();

  // Fragments are double buffered in registers: while the MFMAs of step kk
  // run, the ds_reads of step kk + 1 are in flight.
  bf16x8 fa[2][FM], fb[2][FN];
  auto read_frags = [&](int buf, const char* sA, const char* sB, int kk) {
#pragma unroll
    for (int i = 0; i < FM; ++i) fa[buf][i] = TA::frag(sA, wm * WTM + i * 32, kk, lane);
#pragma unroll
    for (int j = 0; j < FN; ++j) fb[buf][j] = TB::frag(sB, wn * WTN + j * 32, kk, lane);
  };
  auto mfma_step = [&](int buf) {
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int j = 0; j < FN; ++j)
        if constexpr (HALF)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
              __builtin_bit_cast(f16x8, fb[buf][j]), __builtin_bit_cast(f16x8, fa[buf][i]),
              acc[i][j], 0, 0, 0);
        else
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[buf][j], fa[buf][i],
                                                              acc[i][j], 0, 0, 0);
  };

  read_frags(0, lds, lds + TA::BYTES, 0);
  for (int kt = 0; kt < KT; ++kt) {
    const char* sA = lds + (kt & 1) * STAGE;
    const char* sB = sA + TA::BYTES;
    char* nA = lds + ((kt + 1) & 1) * STAGE;
    const bool more = kt + 1 < KT;
    if (more) {
      TA::load(ra, g.A, g.lda, m0, g.M, (kt + 1) * BK, g.Kc, tid);
      TB::load(rb, g.B, g.ldb, n0, g.N, (kt + 1) * BK, g.Kc, tid);
    }
#pragma unroll
    for (int kk = 0; kk < KK - 1; ++kk) {
      read_frags((kk + 1) & 1, sA, sB, kk + 1);
      mfma_step(kk & 1);
    }
    // Last step of this tile: every read of the current buffer has been issued,
    // so the next tile can go to the other buffer while the MFMAs run.
    if (more) {
      TA::store(ra, nA, tid);
      TB::store(rb, nA + TA::BYTES, tid);
    }
    mfma_step((KK - 1) & 1);
    __syncthreads();
    if (more) read_frags(0, nA, nA + TA::BYTES, 0);
  }

  store_tile<FM, FN, EPI, OUT_F32, EDGE, HALF>(acc, g, lds, wave, lane, m0 + wm * WTM,
                                               n0 + wn * WTN);
}

template <int BM, int BN, int WAVES_M, int WAVES_N, bool A_KMAJOR, bool B_KMAJOR,
          int EPI, bool OUT_F32, bool EDGE>
__global__ void __launch_bounds__(WAVES_M* WAVES_N * 64) gemm_bf16_kernel(const GemmArgs g) {
  staged_gemm<BM, BN, WAVES_M, WAVES_N, A_KMAJOR, B_KMAJOR, EPI, OUT_F32, EDGE, false>(g);
}
template <int BM, int BN, int WAVES_M, int WAVES_N, bool A_KMAJOR, bool B_KMAJOR,
          int EPI, bool OUT_F32, bool EDGE>
__global__ void __launch_bounds__(WAVES_M* WAVES_N * 64) gemm_f16_kernel(const GemmArgs g) {
  staged_gemm<BM, BN, WAVES_M, WAVES_N, A_KMAJOR, B_KMAJOR, EPI, OUT_F32, EDGE, true>(g);
}

// The dynamic LDS size a kernel may ask for is an attribute of the kernel on a device: set
// on a kernel's first launch on each device, not on every launch.  `done` is the
// per-kernel-instance record (one bit per device).
int allow_lds(const void* kern, size_t lds, std::atomic<unsigned long long>& done) {
  int dev = 0;
  AXN_HIP_TRY(hipGetDevice(&dev));
  const unsigned long long bit = 1ull << (dev & 63);
  if (done.load(std::memory_order_acquire) & bit) return AXN_OK;
  AXN_HIP_TRY(hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  done.fetch_or(bit, std::memory_order_release);
  return AXN_OK;
}

template <int BM, int BN, int WAVES_M, int WAVES_N, bool AK, bool BKM, int EPI,
          bool OUT_F32, bool EDGE, bool HALF>
int launch_cfg(const GemmArgs& in, hipStream_t stream) {
  GemmArgs g = in;
  g.tiles_m = (g.M + BM - 1) / BM;
  g.tiles_n = (g.N + BN - 1) / BN;
  constexpr int NT = WAVES_M * WAVES_N * 64;
  constexpr size_t lds = 2 * (size_t)(BM + BN) * BK * 2;
  void (*kern)(const GemmArgs) =
      gemm_bf16_kernel<BM, BN, WAVES_M, WAVES_N, AK, BKM, EPI, OUT_F32, EDGE>;
  if constexpr (HALF) kern = gemm_f16_kernel<BM, BN, WAVES_M, WAVES_N, AK, BKM, EPI, OUT_F32, EDGE>;
  {
    static std::atomic<unsigned long long> lds_allowed{0};   // per template instance
    const int rc = allow_lds((const void*)kern, lds, lds_allowed);
    if (rc != AXN_OK) return rc;
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

template <int TILE, bool AK, bool BKM, int EPI, bool OUT_F32, bool HALF>
int launch_solo(const GemmArgs& in, hipStream_t stream) {
  GemmArgs g = in;
  g.tiles_m = g.M / TILE;
  g.tiles_n = g.N / TILE;
  // ring of 5 operand tiles: 160 KiB (all of a CU's LDS) or 80 KiB (two workgroups per CU)
  constexpr size_t lds = 5 * TILE * 64 * 2;
  void (*kern)(const GemmArgs) = gemm_bf16_solo_kernel<TILE, AK, BKM, EPI, OUT_F32>;
  if constexpr (HALF) kern = gemm_f16_solo_kernel<TILE, AK, BKM, EPI, OUT_F32>;
  {
    static std::atomic<unsigned long long> lds_allowed{0};   // per template instance
    const int rc = allow_lds((const void*)kern, lds, lds_allowed);
    if (rc != AXN_OK) return rc;
  }
  const int splits = g.splits > 1 ? g.splits : 1;
  hipLaunchKernelGGL(kern, dim3((unsigned)(g.tiles_m * g.tiles_n * splits)), dim3(256), lds, stream,
                     g);
  AXN_HIP_TRY(hipGetLastError());
  return AXN_OK;
}

template <bool AK, bool BKM, int EPI, bool OUT_F32, bool HALF>
int launch_rest(const GemmArgs& in, hipStream_t stream) {
  GemmArgs g = in;
  g.tiles_m = g.M / 256;
  g.tiles_n = g.N / 128;
  constexpr size_t lds = 5 * 256 * 64 * 2;  // five slots of the A tile's size
  void (*kern)(const GemmArgs) = gemm_bf16_rest_kernel<AK, BKM, EPI, OUT_F32>;
  if constexpr (HALF) kern = gemm_f16_rest_kernel<AK, BKM, EPI, OUT_F32>;
  {
    static std::atomic<unsigned long long> lds_allowed{0};   // per template instance
    const int rc = allow_lds((const void*)kern, lds, lds_allowed);
    if (rc != AXN_OK) return rc;
  }
  const int splits = g.splits > 1 ? g.splits : 1;
  hipLaunchKernelGGL(kern, dim3((unsigned)(g.tiles_m * g.tiles_n * splits)), dim3(256), lds, stream, g);
  AXN_HIP_TRY(hipGetLastError());
  return AXN_OK;
}

// Kernel selection.  Problems made of whole 256 x 256 tiles, more than 128 of
// them (half of the CUs) and not just above one round of 256, take the
// one-wave-per-SIMD kernel at that tile size, 65..128 of them take it at 256 x 128;
// other problems made of whole 128 x 128 tiles take it at 128 x 128; ragged
// shapes, and operands too large for 32-bit byte offsets, take the
// register-staged kernel.
template <bool AK, bool BKM, int EPI, bool OUT_F32, bool HALF>
int launch_whole(const GemmArgs& g, hipStream_t stream) {
  const bool deep = g.Kc % 64 == 0;
  const bool whole256 = (g.M % 256 == 0) && (g.N % 256 == 0) && deep;
  const bool whole128 = (g.M % 128 == 0) && (g.N % 128 == 0) && deep;
  const long long tiles256 = (long long)((g.M + 255) / 256) * ((g.N + 255) / 256);
  const long long tiles128 = (long long)((g.M + 127) / 128) * ((g.N + 127) / 128);
  // The one-wave-per-SIMD kernel addresses its operands with 32-bit byte offsets.
  const int64_t a_span = (int64_t)(AK ? g.M : g.Kc) * g.lda * 2;
  const int64_t b_span = (int64_t)(BKM ? g.N : g.Kc) * g.ldb * 2;
  const bool small_spans = a_span < (1LL << 31) && b_span < (1LL << 31);
  // Up to 128 large tiles the small tile wins: four times as many workgroups, two per CU, still
  // fit in one round.  Beyond that its second round costs more than the idle CUs of the large one,
  // except just above one full round (257..320 large tiles), where the large tile's second round
  // would leave three quarters of the chip idle (measured: +10..14 % at 272..304 tiles, -3 % at 336).
  const bool large_tile = tiles256 > 128 && !(tiles256 > 256 && tiles256 <= 320);
  if (small_spans && whole256 && large_tile)
    return launch_solo<256, AK, BKM, EPI, OUT_F32, HALF>(g, stream);
  // 65..128 large tiles: 256 x 128 tiles, one workgroup per CU on more than half of the CUs
  // (+4..11 % against the small tile, measured at 80, 96, 112 and 128 tiles).
  if (small_spans && whole256 && tiles256 > 64 && tiles256 <= 128)
    return launch_rest<AK, BKM, EPI, OUT_F32, HALF>(g, stream);
  if (small_spans && whole128 && tiles128 < (1LL << 31))
    return launch_solo<128, AK, BKM, EPI, OUT_F32, HALF>(g, stream);
  if constexpr (EPI == EPI_PAIR) {
    set_error("gemm_pair: needs whole 128 x 128 tiles, contractions that are multiples of 64 and "
              "operands below 2 GiB (got M=%d, N=%d, K=%d)", g.M, g.N, g.Kc);
    return AXN_ESHAPE;
  } else {
    if (whole128) return launch_cfg<128, 128, 2, 2, AK, BKM, EPI, OUT_F32, false, HALF>(g, stream);
    return launch_cfg<128, 128, 2, 2, AK, BKM, EPI, OUT_F32, true, HALF>(g, stream);
  }
}

// Full rounds and the rest.  A problem of k * 256 + r large tiles with 0 < r <= 128 ends
// in a round that leaves at least half of the CUs idle.  It is cut along one output
// dimension into a part of exactly k rounds of large tiles and the remaining r tiles,
// which go to 256 x 128 tiles (2 r workgroups, one per CU) or, for r <= 64, to the small
// tile (4 r workgroups).
// Measured on 4096-row problems, K = 4096: +8..12 % at 272..384 tiles, +11..13 % at
// 544..576, +4 % at 640, +10 % at 800, +1 % at 896; with r > 128 the cut loses 2..3 %.
// The two parts run one after the other on the caller's stream.
template <bool AK, bool BKM, int EPI, bool OUT_F32, bool HALF>
int launch_shape(const GemmArgs& g, hipStream_t stream) {
  if (g.M % 256 == 0 && g.N % 256 == 0 && g.Kc % 64 == 0 && g.splits <= 1) {
    const long long tm = g.M / 256, tn = g.N / 256, tiles = tm * tn;
    const long long full = tiles / 256 * 256, rest = tiles - full;
    if (full > 0 && rest > 0 && rest <= 128) {
      constexpr int64_t esz = OUT_F32 ? 4 : 2;
      GemmArgs g1 = g, g2 = g;
      bool cut = false;
      if (full % tm == 0) {  // whole tile columns
        const int64_t n1 = full / tm * 256;
        g1.N = (int)n1;
        g2.N = g.N - (int)n1;
        g2.B = BKM ? g.B + n1 * g.ldb : g.B + n1;
        if (g.B2 != nullptr) g2.B2 = BKM ? g.B2 + n1 * g.ldb : g.B2 + n1;
        g2.C = (char*)g.C + n1 * esz;
        if (g.bias != nullptr) g2.bias = g.bias + n1;
        if (g.Z != nullptr) g2.Z = g.Z + n1;
        cut = true;
      } else if (full % tn == 0) {  // whole tile rows
        const int64_t m1 = full / tn * 256;
        g1.M = (int)m1;
        g2.M = g.M - (int)m1;
        g2.A = AK ? g.A + m1 * g.lda : g.A + m1;
        if (g.A2 != nullptr) g2.A2 = AK ? g.A2 + m1 * g.lda : g.A2 + m1;
        g2.C = (char*)g.C + m1 * g.ldc * esz;
        if (g.Z != nullptr) g2.Z = g.Z + m1 * g.ldc;
        cut = true;
      }
      if (cut) {
        const int rc = launch_whole<AK, BKM, EPI, OUT_F32, HALF>(g1, stream);
        if (rc != AXN_OK) return rc;
        // More than 64 tiles left: 256 x 128 tiles, one per CU on more than half of the CUs
        // (qkv forward +5 %, down dgrad +3 % against the small tile); fewer: the small tile,
        // whose 4 r workgroups still give every CU at most one (MLP shard dgrad, r = 64: -7 %
        // with the 256 x 128 tile).
        const int64_t a_span = (int64_t)(AK ? g2.M : g2.Kc) * g2.lda * 2;
        const int64_t b_span = (int64_t)(BKM ? g2.N : g2.Kc) * g2.ldb * 2;
        if (rest > 64 && a_span < (1LL << 31) && b_span < (1LL << 31))
          return launch_rest<AK, BKM, EPI, OUT_F32, HALF>(g2, stream);
        return launch_whole<AK, BKM, EPI, OUT_F32, HALF>(g2, stream);
      }
    }
  }
  return launch_whole<AK, BKM, EPI, OUT_F32, HALF>(g, stream);
}

}  // namespace

namespace {

// Sum of the fp32 partial products of a split contraction, in split order, plus the
// old output if beta; one 16-byte store (two for fp32) of 8 columns per lane.
template <typename LP>
__global__ void __launch_bounds__(256)
    splitk_reduce_kernel(const float* __restrict__ ws, LP* out, int64_t M, int64_t N, int64_t ld,
                         int splits, int beta) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t per_row = N / 8;
  if (idx >= M * per_row) return;
  const int64_t row = idx / per_row, col = (idx - row * per_row) * 8;
  const float* p = ws + row * N + col;
  f32x4 a0 = __builtin_nontemporal_load((const f32x4*)p);
  f32x4 a1 = __builtin_nontemporal_load((const f32x4*)(p + 4));
  for (int s = 1; s < splits; ++s) {
    p += M * N;
    a0 += __builtin_nontemporal_load((const f32x4*)p);
    a1 += __builtin_nontemporal_load((const f32x4*)(p + 4));
  }
  LP* o = out + row * ld + col;
  if constexpr (sizeof(LP) == 4) {
    if (beta) {
      a0 += *(const f32x4*)o;
      a1 += *(const f32x4*)(o + 4);
    }
    *(f32x4*)o = a0;
    *(f32x4*)(o + 4) = a1;
  } else {
    typedef LP lpx8 __attribute__((ext_vector_type(8)));
    float v[8] = {a0[0], a0[1], a0[2], a0[3], a1[0], a1[1], a1[2], a1[3]};
    if (beta) {
      const lpx8 old = *(const lpx8*)o;
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] += (float)old[e];
    }
    lpx8 y;
#pragma unroll
    for (int e = 0; e < 8; ++e) y[e] = (LP)v[e];
    *(lpx8*)o = y;
  }
}

template <bool AK, bool BKM, bool HALF>
int launch_split(const GemmArgs& g, bool wide_tiles, hipStream_t stream) {
  if (wide_tiles) return launch_rest<AK, BKM, AXN_EPI_NONE, true, HALF>(g, stream);
  return launch_solo<128, AK, BKM, AXN_EPI_NONE, true, HALF>(g, stream);
}

template <bool HALF>
int launch_layout(GemmLayout layout, const GemmArgs& g, int epilogue, bool out_f32,
                  hipStream_t stream) {
  switch (layout) {
    case GEMM_NT:
      if (out_f32) {  // 16-bit product + fp32 bias promoted to fp32, as `x + bias` promotes it
        if (epilogue == AXN_EPI_BIAS) return launch_shape<true, true, AXN_EPI_BIAS, true, HALF>(g, stream);
        if (epilogue == AXN_EPI_BIAS_GELU)
          return launch_shape<true, true, AXN_EPI_BIAS_GELU, true, HALF>(g, stream);
        break;
      }
      switch (epilogue) {
        case AXN_EPI_NONE:
          return launch_shape<true, true, AXN_EPI_NONE, false, HALF>(g, stream);
        case AXN_EPI_BIAS:
          return launch_shape<true, true, AXN_EPI_BIAS, false, HALF>(g, stream);
        case AXN_EPI_BIAS_GELU:
          return launch_shape<true, true, AXN_EPI_BIAS_GELU, false, HALF>(g, stream);
        case AXN_EPI_GELU:
          return launch_shape<true, true, AXN_EPI_GELU, false, HALF>(g, stream);
      }
      break;
    case GEMM_NN:
      if (out_f32 || epilogue != AXN_EPI_NONE) break;
      return launch_shape<true, false, AXN_EPI_NONE, false, HALF>(g, stream);
    case GEMM_TN:
      if (epilogue != AXN_EPI_NONE) break;
      return out_f32 ? launch_shape<false, false, AXN_EPI_NONE, true, HALF>(g, stream)
                     : launch_shape<false, false, AXN_EPI_NONE, false, HALF>(g, stream);
  }
  set_error("gemm: unsupported layout/epilogue/output combination");
  return AXN_EINVAL;
}
}  // namespace

int launch_gemm_pair(const GemmArgs& g, bool half, hipStream_t stream) {
  if (g.k_first % 64 != 0 || g.k_first < 128 || (g.Kc - g.k_first) % 64 != 0 || g.Kc - g.k_first < 64 ||
      g.splits > 1) {
    set_error("gemm_pair: both contractions must be multiples of 64, the first at least 128 "
              "(got %d and %d)", g.k_first, g.Kc - g.k_first);
    return AXN_ESHAPE;
  }
  // the operand spans the kernels address with 32 bits, checked on the longer pair
  const int k_long = g.k_first > g.Kc - g.k_first ? g.k_first : g.Kc - g.k_first;
  if ((int64_t)k_long * g.ldb * 2 >= (1LL << 31)) {
    set_error("gemm_pair: operands must stay below 2 GiB");
    return AXN_ESHAPE;
  }
  return half ? launch_shape<true, false, EPI_PAIR, false, true>(g, stream)
              : launch_shape<true, false, EPI_PAIR, false, false>(g, stream);
}

int launch_gemm_swiglu(const GemmArgs& in, bool half, hipStream_t stream) {
  GemmArgs g = in;
  const int64_t a_span = (int64_t)g.M * g.lda * 2, b_span = (int64_t)g.N * g.ldb * 2;
  if (g.M % 256 != 0 || g.N % 128 != 0 || g.Kc % 64 != 0 || a_span >= (1LL << 31) ||
      b_span >= (1LL << 31)) {
    set_error("gemm_swiglu: needs M %% 256 == 0, N %% 128 == 0, K %% 64 == 0 and operands below "
              "2 GiB (got M=%d, N=%d, K=%d)", g.M, g.N, g.Kc);
    return AXN_ESHAPE;
  }
  g.tiles_m = g.M / 256;
  g.tiles_n = g.N / 128;
  g.splits = 0;
  constexpr size_t lds = 5 * 256 * 64 * 2;
  void (*kern)(const GemmArgs) = half ? gemm_f16_swiglu_kernel : gemm_bf16_swiglu_kernel;
  {
    static std::atomic<unsigned long long> lds_allowed[2];   // bf16 and fp16 kernel
    const int rc = allow_lds((const void*)kern, lds, lds_allowed[half ? 1 : 0]);
    if (rc != AXN_OK) return rc;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)((long long)g.tiles_m * g.tiles_n)), dim3(256), lds,
                     stream, g);
  AXN_HIP_TRY(hipGetLastError());
  return AXN_OK;
}

// ---- input and weight gradient of one layer in one call ----------------------------
namespace {
// Rounds of 64-deep stages a launch of `tiles` 256 x 256 tiles over `stages` stages takes on
// 256 CUs the way launch_shape runs it (a rest of up to half a round costs about 0.7 of one).
double stages_alone(long long tiles, long long stages) {
  const long long full = tiles / 256, rest = tiles % 256;
  if (rest == 0) return (double)(full * stages);
  if (full > 0 && rest <= 128) return (full + 0.7) * stages;
  return (double)((full + 1) * stages);
}
// The same for one launch that holds both problems, longer tiles first: every CU takes the
// next tile when it is free (a heap of the CUs' busy times: a few thousand steps).
double stages_together(long long t1, long long s1, long long t2, long long s2) {
  if (s1 < s2) {
    std::swap(t1, t2);
    std::swap(s1, s2);
  }
  std::priority_queue<long long, std::vector<long long>, std::greater<long long>> cus;
  for (int c = 0; c < 256; ++c) cus.push(0);
  long long end = 0;
  auto place = [&](long long tiles, long long stages) {
    for (long long i = 0; i < tiles; ++i) {
      const long long t = cus.top() + stages;
      cus.pop();
      cus.push(t);
      end = t > end ? t : end;
    }
  };
  place(t1, s1);
  place(t2, s2);
  return (double)end;
}

template <bool HALF>
int launch_backward(const GemmArgs& gd_in, const GemmArgs& gw_in, bool dw_f32, hipStream_t stream) {
  GemmArgs gd = gd_in, gw = gw_in;
  auto whole = [](const GemmArgs& g, bool ak, bool bk) {
    const int64_t a_span = (int64_t)(ak ? g.M : g.Kc) * g.lda * 2;
    const int64_t b_span = (int64_t)(bk ? g.N : g.Kc) * g.ldb * 2;
    return g.M % 256 == 0 && g.N % 256 == 0 && g.Kc % 64 == 0 && g.Kc >= 128 && a_span < (1LL << 31) &&
           b_span < (1LL << 31);
  };
  if (whole(gd, true, false) && whole(gw, false, false)) {
    const long long td = (long long)(gd.M / 256) * (gd.N / 256), tw = (long long)(gw.M / 256) * (gw.N / 256);
    const long long sd = gd.Kc / 64, sw = gw.Kc / 64;
    // one launch when that ends at least 5 % earlier than the two launches (measured on
    // MI355X at 8192 x 5120 x 2560: 320 tiles of 80 stages and 200 of 128); the answer for
    // the last few shapes is kept, a training loop asks for the same ones again and again
    struct Planned {
      long long td, tw, sd, sw;
      bool together;
    };
    static thread_local Planned last[4] = {};
    static thread_local int next_slot = 0;
    int hit = -1;
    for (int i = 0; i < 4; ++i)
      if (last[i].td == td && last[i].tw == tw && last[i].sd == sd && last[i].sw == sw) hit = i;
    if (hit < 0) {
      hit = next_slot;
      next_slot = (next_slot + 1) % 4;
      last[hit] = {td, tw, sd, sw,
                   td + tw <= 4096 && stages_together(tw, sw, td, sd) <
                                          0.95 * (stages_alone(td, sd) + stages_alone(tw, sw))};
    }
    if (last[hit].together) {
      gw.tiles_m = gw.M / 256, gw.tiles_n = gw.N / 256, gw.wg_first = sw >= sd ? 0 : (int)td;
      gd.tiles_m = gd.M / 256, gd.tiles_n = gd.N / 256, gd.wg_first = sw >= sd ? (int)tw : 0;
      gw.splits = gd.splits = 0;
      constexpr size_t lds = 5 * 256 * 64 * 2;
      void (*kern)(const GemmArgs, const GemmArgs) =
          dw_f32 ? gemm_backward_kernel<HALF, true> : gemm_backward_kernel<HALF, false>;
      {
        static std::atomic<unsigned long long> lds_allowed[2];   // per output type of dW
        const int rc = allow_lds((const void*)kern, lds, lds_allowed[dw_f32 ? 1 : 0]);
        if (rc != AXN_OK) return rc;
      }
      hipLaunchKernelGGL(kern, dim3((unsigned)(tw + td)), dim3(256), lds, stream, gw, gd);
      AXN_HIP_TRY(hipGetLastError());
      return AXN_OK;
    }
  }
  const int rc = launch_shape<true, false, AXN_EPI_NONE, false, HALF>(gd, stream);
  if (rc != AXN_OK) return rc;
  return dw_f32 ? launch_shape<false, false, AXN_EPI_NONE, true, HALF>(gw, stream)
                : launch_shape<false, false, AXN_EPI_NONE, false, HALF>(gw, stream);
}
}  // namespace

int launch_gemm_backward(const GemmArgs& dgrad, const GemmArgs& wgrad, bool half, bool dw_f32,
                         hipStream_t stream) {
  return half ? launch_backward<true>(dgrad, wgrad, dw_f32, stream)
              : launch_backward<false>(dgrad, wgrad, dw_f32, stream);
}

int launch_gemm_bf16(GemmLayout layout, const GemmArgs& g, int epilogue,
                     bool out_f32, hipStream_t stream) {
  return launch_layout<false>(layout, g, epilogue, out_f32, stream);
}

int launch_gemm_f16(GemmLayout layout, const GemmArgs& g, int epilogue, bool out_f32,
                    hipStream_t stream) {
  return launch_layout<true>(layout, g, epilogue, out_f32, stream);
}

// Few output tiles leave most CUs without work: the contraction is cut into 2, 4 or 8 parts, each
// at least 512 deep, on 128 x 128 tiles (up to two workgroups per CU) or 256 x 128 tiles (one).
// Whether, into how many parts and on which tile to split the contraction of a problem with
// few output tiles: the choice with the smallest estimated time.  The estimate (microseconds
// on MI355X, operands coming from HBM) of a launch of w workgroups that each walk `stages`
// 64-deep stages:
//   main loop   stages x 0.77 (128 x 128 tiles, at most one workgroup per CU), x 1.33 (two
//               per CU), x 0.93 (256 x 128 tiles: twice the output per stage), times the
//               rounds of workgroups the launch takes;
//   operands    never faster than their bytes at 6 TB/s, and at 47 % of that plus the rest in
//               proportion to the CUs that have a workgroup;
//   parts       2.1 + parts x 2.5 x (millions of output elements)^0.74 for writing the fp32
//               partial products and for the pass that adds them.
// The eight constants were fitted to the choices' measured times over 165 forward and
// input-gradient problems of 128 to 1024 tokens and 2560 to 14336 features (every choice
// timed on cold operands): the rule's pick is within 0.6 % of the fastest choice on average
// and 13 % at worst; the rule it replaced (as many parts as fill the CUs, 256 x 128 tiles
// first) was 4.4 % off on average and 44 % at worst.
int gemm_splits(GemmLayout layout, const GemmArgs& g, bool* wide_tiles) {
  if (wide_tiles != nullptr) *wide_tiles = false;
  if (g.M % 128 || g.N % 128 || g.Kc % 64) return 1;
  const bool ak = layout != GEMM_TN, bkm = layout == GEMM_NT;
  const int64_t a_span = (int64_t)(ak ? g.M : g.Kc) * g.lda * 2;
  const int64_t b_span = (int64_t)(bkm ? g.N : g.Kc) * g.ldb * 2;
  if (a_span >= (1LL << 31) || b_span >= (1LL << 31)) return 1;
  const long long tiles = (long long)(g.M / 128) * (g.N / 128);
  const long long wide = g.M % 256 == 0 ? (long long)(g.M / 256) * (g.N / 128) : -1;
  // beyond 128 tiles of either kind an unsplit launch already has a workgroup on half of the CUs
  if (!(tiles <= 128 || (wide > 0 && wide <= 128))) return 1;
  const double out_m = (double)g.M * g.N * 1e-6;
  const double operand_mb = ((double)g.M + g.N) * g.Kc * 2e-6;
  const double part_cost = 2.529 * std::pow(out_m, 0.736);
  auto estimate = [&](int parts, bool wide_kind) {
    const double stages = (double)g.Kc / 64 / parts;
    const long long w = (wide_kind ? wide : tiles) * parts;
    const double loop = wide_kind ? stages * 0.928 * (double)((w + 255) / 256)
                                  : stages * (w <= 256 ? 0.771 : 1.332) * (double)((w + 511) / 512);
    const double occupied = w >= 256 ? 1.0 : (double)w / 256;
    const double stream = operand_mb / (5.998 * (0.465 + 0.535 * occupied));
    return (loop > stream ? loop : stream) + (parts > 1 ? 2.143 + parts * part_cost : 0.0);
  };
  double best = estimate(1, false);
  int best_parts = 1;
  bool best_wide = false;
  for (int parts = 2; parts <= 8; parts *= 2) {
    if (g.Kc % (64 * parts) != 0 || g.Kc / parts < 512) continue;
    for (int kind = 0; kind < 2; ++kind) {
      if (kind == 0 ? tiles * parts > 512 : (wide <= 0 || wide * parts > 256)) continue;
      const double t = estimate(parts, kind == 1);
      if (t < best) {
        best = t;
        best_parts = parts;
        best_wide = kind == 1;
      }
    }
  }
  if (wide_tiles != nullptr) *wide_tiles = best_wide;
  return best_parts;
}

int launch_gemm_splitk(GemmLayout layout, const GemmArgs& in, bool half, int out_dtype,
                       int splits, bool wide_tiles, float* ws, hipStream_t stream) {
  GemmArgs g = in;
  g.C = ws;
  g.ldc = g.N;
  g.beta = 0;
  g.bias = nullptr;
  g.Z = nullptr;
  g.splits = splits;
  g.k_split = g.Kc / splits;
  int rc;
  switch (layout) {
    case GEMM_NT:
      rc = half ? launch_split<true, true, true>(g, wide_tiles, stream)
                : launch_split<true, true, false>(g, wide_tiles, stream);
      break;
    case GEMM_NN:
      rc = half ? launch_split<true, false, true>(g, wide_tiles, stream)
                : launch_split<true, false, false>(g, wide_tiles, stream);
      break;
    default:
      rc = half ? launch_split<false, false, true>(g, wide_tiles, stream)
                : launch_split<false, false, false>(g, wide_tiles, stream);
  }
  if (rc) return rc;
  const int64_t lanes = (int64_t)in.M * (in.N / 8);
  const dim3 grid((unsigned)((lanes + 255) / 256)), block(256);
  if (out_dtype == AXN_F32)
    hipLaunchKernelGGL(splitk_reduce_kernel<float>, grid, block, 0, stream, ws, (float*)in.C,
                       (int64_t)in.M, (int64_t)in.N, in.ldc, splits, in.beta);
  else if (out_dtype == AXN_F16)
    hipLaunchKernelGGL(splitk_reduce_kernel<_Float16>, grid, block, 0, stream, ws, (_Float16*)in.C,
                       (int64_t)in.M, (int64_t)in.N, in.ldc, splits, in.beta);
  else
    hipLaunchKernelGGL(splitk_reduce_kernel<__bf16>, grid, block, 0, stream, ws, (__bf16*)in.C,
                       (int64_t)in.M, (int64_t)in.N, in.ldc, splits, in.beta);
  AXN_HIP_TRY(hipGetLastError());
  return AXN_OK;
}

}  // namespace axn
