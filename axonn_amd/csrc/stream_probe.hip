// Streaming yardsticks for benchmarks (libaxn_probe_gfx950.so; not part of the product
// library): what the memory system of an MI355X gives a plain read, a fill and a copy,
// each in the pattern that measured fastest for it.  One 16-byte vector per lane and a
// wave that ends behind it in all three (four vectors per lane: 5.6 to 5.8 TB/s for a copy,
// resident workgroups that stride: 4.7 to 5.2); stores non-temporal and written through.
//   read  256-lane workgroups, every wave the registers allow resident: 7.1 TB/s
//   fill  256-lane workgroups, 24 waves per CU (26.5 KB of LDS reserved per workgroup):
//         7.3 TB/s (7.0 with plain non-temporal stores, 6.8 with 32 waves)
//   copy  one-wave workgroups, all resident: 6.8 TB/s (256-lane workgroups 6.5 to 6.7)
#include <hip/hip_runtime.h>

#include <cstdint>

#include "axn_probe.h"

namespace {

typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int THREADS = 256;
constexpr int FILL_LDS = 27136;

__device__ __forceinline__ void store_through(f32x4 x, f32x4* p) {
  // s_nop: the wait states a store of more than 8 bytes needs before its data registers
  // may be written again, which the compiler inserts for its own stores only
  asm volatile("global_store_dwordx4 %0, %1, off sc1 nt\n\ts_nop 1" ::"v"(p), "v"(x) : "memory");
}
__global__ void __launch_bounds__(THREADS)
    probe_read_kernel(const f32x4* __restrict__ src, int64_t nvec, float* sink) {
  const int64_t i = (int64_t)blockIdx.x * THREADS + threadIdx.x;
  if (i >= nvec) return;
  const f32x4 x = __builtin_nontemporal_load(src + i);
  // never true for finite data: keeps the load alive without a store per lane
  if (x[0] + x[1] + x[2] + x[3] == 1.2345678e38f) *sink = x[0];
}
__global__ void __launch_bounds__(THREADS) probe_fill_kernel(f32x4* __restrict__ dst, int64_t nvec) {
  const int64_t i = (int64_t)blockIdx.x * THREADS + threadIdx.x;
  if (i < nvec) store_through(f32x4{0.f, 0.f, 0.f, 0.f}, dst + i);
}
__global__ void __launch_bounds__(64) probe_copy_kernel(const f32x4* src, f32x4* dst, int64_t nvec) {
  const int64_t i = (int64_t)blockIdx.x * 64 + threadIdx.x;
  if (i < nvec) store_through(__builtin_nontemporal_load(src + i), dst + i);
}

}  // namespace

extern "C" int axn_probe_stream(int kind, const void* src, void* dst, size_t bytes, void* stream_) {
  if (kind != AXN_PROBE_READ && kind != AXN_PROBE_FILL && kind != AXN_PROBE_COPY) return -1;
  if (dst == nullptr || (kind != AXN_PROBE_FILL && src == nullptr)) return -1;
  if (((uintptr_t)src & 15u) != 0 || ((uintptr_t)dst & (kind == AXN_PROBE_READ ? 3u : 15u)) != 0)
    return -2;
  hipStream_t stream = (hipStream_t)stream_;
  const int64_t nvec = (int64_t)(bytes / 16);
  if (nvec == 0) return 0;
  const int lanes = kind == AXN_PROBE_COPY ? 64 : THREADS;
  const long long blocks = (nvec + lanes - 1) / lanes;
  if (blocks > 0x7fffffffLL) return -3;
  const dim3 grid((unsigned)blocks), block(lanes);
  switch (kind) {
    case AXN_PROBE_READ:
      hipLaunchKernelGGL(probe_read_kernel, grid, block, 0, stream, (const f32x4*)src, nvec,
                         (float*)dst);
      break;
    case AXN_PROBE_FILL:
      hipLaunchKernelGGL(probe_fill_kernel, grid, block, FILL_LDS, stream, (f32x4*)dst, nvec);
      break;
    default:
      hipLaunchKernelGGL(probe_copy_kernel, grid, block, 0, stream, (const f32x4*)src, (f32x4*)dst,
                         nvec);
      break;
  }
  return hipGetLastError() == hipSuccess ? 0 : -4;
}
