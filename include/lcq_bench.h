/* lcq_bench.h — entry points of liblcq.so that serve the benchmark only (no counterpart in the reference, not part
 * of the drop-in boundary declared in lcq.h).  Same conventions as lcq.h. */
#ifndef LCQ_BENCH_H
#define LCQ_BENCH_H
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Streams `bytes` (a multiple of 16, both pointers 16-byte aligned) from src and writes bytes / reads_per_write to dst (the xor of every reads_per_write
 * consecutive 16-byte chunks of a thread's share); reads_per_write in {1, 2, 4, 8}, or 0 for a read-only pass.
 * dst_bytes is the room behind dst: less than bytes / reads_per_write (4 KiB for a read-only pass) is refused.  The
 * rate is the ceiling of a quantizer kernel with the same mix of reads and writes. */
int lcq_stream_probe(const void* src, void* dst, int64_t bytes, int64_t dst_bytes, int reads_per_write, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* LCQ_BENCH_H */
