/*
 * breccia_kv_bench.h -- what the tests, the benchmark and the C++ host mirror need around the
 * paged-KV library and a Breccia integration does not: device allocation, copies, streams, events
 * and graph capture for hosts without HIP bindings of their own, and the bandwidth probes the
 * benchmark prices the kernels against.  Built into a library of its own
 * (libbreccia_kv_bench.so); libbreccia_kv.so -- the product, include/breccia_kv.h -- has none of
 * it.  No reference counterpart: the reference's tests get the same services from its Vulkan
 * context crate (crates/breccia-vk).
 *
 * Every entry point returns a bkv_status; on failure bkv_bench_last_error() holds a thread-local
 * message.  `stream` is a hipStream_t passed as void* (NULL = the default stream).
 */
#ifndef BRECCIA_KV_BENCH_H
#define BRECCIA_KV_BENCH_H

#include "breccia_kv.h"

#ifdef __cplusplus
extern "C" {
#endif

const char *bkv_bench_last_error(void);

/* ---- device plumbing ----------------------------------------------------------- */
bkv_status bkv_dev_alloc(uint64_t bytes, void **dev_out);
bkv_status bkv_dev_free(void *dev);
bkv_status bkv_memcpy_h2d(void *dev, const void *host, uint64_t bytes, void *stream);
bkv_status bkv_memcpy_d2h(void *host, const void *dev, uint64_t bytes, void *stream);
bkv_status bkv_stream_create(void **stream_out);
/* Stream capture into a graph (hipStreamBeginCapture / EndCapture + hipGraphInstantiate, thread-local
 * capture mode) and its replay; `stream` must not be NULL. */
bkv_status bkv_graph_begin_capture(void *stream);
bkv_status bkv_graph_end_capture(void *stream, void **graph_exec_out);
bkv_status bkv_graph_launch(void *graph_exec, void *stream);
bkv_status bkv_graph_destroy(void *graph_exec);
bkv_status bkv_stream_destroy(void *stream);
bkv_status bkv_stream_sync(void *stream);
bkv_status bkv_device_sync(void);
bkv_status bkv_event_create(void **event_out);
bkv_status bkv_event_destroy(void *event);
bkv_status bkv_event_record(void *event, void *stream);
bkv_status bkv_event_sync(void *event);
bkv_status bkv_event_elapsed_ms(void *start, void *stop, float *ms_out);
/* name (<= 255 chars), compute units, total device memory */
bkv_status bkv_device_info(char *name_out, int32_t name_cap, int32_t *cu_out,
                           uint64_t *mem_bytes_out);
/* free and total device memory (hipMemGetInfo) */
bkv_status bkv_device_mem_info(uint64_t *free_out, uint64_t *total_out);
/* Reference bandwidth probe: a plain 16-byte-vector device copy of `bytes` bytes
 * (used to scale profiler byte counters and to report the copy ceiling). */
bkv_status bkv_copy_probe(void *dst_dev, const void *src_dev, uint64_t bytes, void *stream);
/* Read-only bandwidth probe: reads `bytes` (a power-of-two number of 8 KiB chunks -- the size of
 * one (page, kv head) run of an f16 pool) once, 8 KiB per wave at a time, in address order
 * (scattered = 0), in a fixed pseudo-random order of chunks (1), as the attention kernels see a
 * shuffled pool, or in that order with every chunk fetched by global->LDS loads instead of loads
 * into registers (2: the slower of the two ways a row can reach LDS on this chip, kept so that the
 * comparison behind the quantised kernels' data path can be repeated); nothing is written
 * except, never in practice, one word at sink_dev.  The rate it reaches is the ceiling a
 * read-only kernel can be held against on a given box. */
bkv_status bkv_read_probe(const void *src_dev, uint64_t bytes, int32_t scattered, void *sink_dev,
                          void *stream);

#ifdef __cplusplus
}
#endif
#endif /* BRECCIA_KV_BENCH_H */
