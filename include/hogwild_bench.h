/*
 * hogwild_bench.h — calibration kernels of the measurement harness (libhogwild_bench.so).  Not part of the product
 * ABI in hogwild_hip.h and not linked into libhogwild_hip.so: nothing here has a counterpart in the reference.
 * Same status convention: 0, a negative hw_status, or a positive hipError_t.
 */
#ifndef HOGWILD_BENCH_H
#define HOGWILD_BENCH_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Streaming read of `bytes` bytes (multiple of 16) from `src`, xor-reduced into sink[0..255]: the plain
   bandwidth calibration the attention kernel is compared with. */
int hw_stream_read(const void* src, size_t bytes, uint32_t* sink, void* stream);
/* The same read with a given number of 256-thread workgroups (hw_stream_read launches 2048): the control for counter
   passes on a kernel that runs one workgroup per compute unit. */
int hw_stream_read_shaped(const void* src, size_t bytes, uint32_t* sink, int workgroups, void* stream);
/* Plain copy kernel of known size, used to scale the FETCH_SIZE / WRITE_SIZE hardware counters. */
int hw_stream_copy(void* dst, const void* src, size_t bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* HOGWILD_BENCH_H */
