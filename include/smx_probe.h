/*
 * smx_probe -- bandwidth probes for the benchmark (libsmx_probe.so).  Measurement only: not part of the
 * drop-in C ABI of smore_amd.h and not needed by any caller of the scoring path.
 */
#ifndef SMX_PROBE_H
#define SMX_PROBE_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* No counterpart in the reference.  One launch of a kernel that does nothing but move memory in one of
 * the access shapes of this path, for bench.py to time: what the box sustains, next to the nominal peak.
 *   READ_NT / READ   stream `bytes` of a (non-temporal / plain loads)
 *   COPY             a -> b          UPDATE  a = 2 a in place          FILL  a = constant
 *   ROWS / ROWS_NT   n_reads rows of row_bytes (16..1024, multiple of 16) at pseudo-random positions of a
 * sink: one device float the read probes may write (keeps their loads alive); never meaningful. */
#define SMX_PROBE_READ_NT 0
#define SMX_PROBE_READ 1
#define SMX_PROBE_COPY 2
#define SMX_PROBE_UPDATE 3
#define SMX_PROBE_FILL 4
#define SMX_PROBE_ROWS 5
#define SMX_PROBE_ROWS_NT 6
int smx_probe_bandwidth(int kind, void* stream, void* a, void* b, size_t bytes, size_t row_bytes,
                        size_t n_reads, float* sink);

const char* smx_probe_last_error(void);

#ifdef __cplusplus
}
#endif
#endif /* SMX_PROBE_H */
