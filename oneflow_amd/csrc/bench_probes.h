/*
 * Measurement probes for bench.py: libofq_bench_probes.so, a library of its own.  They are not
 * part of the C ABI a OneFlow maintainer binds (include/ofq.h) and nothing in the product calls
 * them; they exist so that the ceilings a benchmark line is read against (the cost of a launch,
 * the time of a kernel that only reads the same bytes, the bandwidth of a plain copy) are
 * measured by the benchmark itself, in the same harness as the kernels, on the box it runs on.
 * Return: 0, or an ofq_status value.
 */
#ifndef OFQ_BENCH_PROBES_H_
#define OFQ_BENCH_PROBES_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* reads `bytes` (rounded down to 16) from buf once, one 16-byte request per lane, one round of
 * blocks, nothing computed; buf 16-byte aligned; sink: 4 writable bytes (untouched in practice) */
int ofq_bench_probe_read(void* stream, const void* buf, size_t bytes, void* sink);
/* a kernel of 256 blocks that does nothing: the fixed cost of a launch */
int ofq_bench_empty_launch(void* stream, void* sink);
/* dst[i] = src[i] over `bytes` (a multiple of 16, both 16-byte aligned): 16 bytes per lane, one
 * round of blocks, `bytes` read and `bytes` written */
int ofq_bench_copy(void* stream, void* dst, const void* src, size_t bytes);

#ifdef __cplusplus
}
#endif
#endif /* OFQ_BENCH_PROBES_H_ */
