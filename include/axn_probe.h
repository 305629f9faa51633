/* axn_probe.h - C ABI of libaxn_probe_gfx950.so.
 *
 * A measurement aid for benchmarks, NOT part of the drop-in boundary (that is axn.h /
 * libaxn_gfx950.so) and without a counterpart in the reference: plain streaming kernels
 * (one 16-byte vector per lane, non-temporal accesses, each in the launch shape that
 * measured fastest for it on MI355X), so that a benchmark can put the optimizer step's
 * rate beside what the memory system of the same GPU gives a plain read, fill or copy.
 *
 *   AXN_PROBE_READ: reads `bytes` from src (dst: 4 writable bytes, never written for
 *                   finite data); AXN_PROBE_FILL: writes `bytes` of zeros to dst;
 *   AXN_PROBE_COPY: copies `bytes` from src to dst (src == dst: in place).
 * Pointers 16-byte aligned; bytes is rounded down to a multiple of 16.  Asynchronous on
 * `stream` (a hipStream_t).  Returns 0, or -1 (bad argument), -2 (misaligned pointer),
 * -3 (more than 2^31 - 1 workgroups), -4 (the launch failed).
 */
#ifndef AXN_PROBE_H_
#define AXN_PROBE_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#if defined(__GNUC__)
#define AXN_PROBE_API __attribute__((visibility("default")))
#else
#define AXN_PROBE_API
#endif

typedef enum axn_probe_kind { AXN_PROBE_READ = 0, AXN_PROBE_FILL = 1, AXN_PROBE_COPY = 2 } axn_probe_kind;
AXN_PROBE_API int axn_probe_stream(int kind, const void* src, void* dst, size_t bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* AXN_PROBE_H_ */
