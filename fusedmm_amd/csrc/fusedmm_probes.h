/*
 * fusedmm_probes.h -- measuring aids of the benchmark (libfusedmm_amd_probes.so): a copy of
 * known size, a read-only stream and a read-only gather of whole rows.  Not part of the
 * product: nothing in libfusedmm_amd_*.so uses them, and a consumer of fusedMM_csr never
 * needs them.  Plain C ABI; every pointer is device memory; calls are asynchronous on
 * `stream` (a hipStream_t, NULL for the default stream) and return 0 or 1.
 */
#ifndef FUSEDMM_PROBES_H
#define FUSEDMM_PROBES_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Copy `bytes` (a multiple of 16, 16-byte aligned) with a plain grid-stride kernel.
 * Hardware traffic counters of the product's kernels are scaled by what they read for
 * this copy of known size. */
int fusedMM_amd_copy_probe(void *dst, const void *src, int64_t bytes, void *stream);

/* Read `bytes` (a multiple of 16, 16-byte aligned) with a grid of blocks_per_cu
 * workgroups per compute unit, each thread keeping `in_flight` (2, 4, 8 or 16)
 * independent 16-byte loads outstanding, non-temporal or not; nothing is written
 * (`sink`, 4 bytes, only keeps the loads alive).  What the memory system delivers to
 * reads alone. */
int fusedMM_amd_read_probe(const void *src, int64_t bytes, int blocks_per_cu, int in_flight, int nontemporal,
                           void *sink, void *stream);

/* Gather `n_ids` whole rows of `row_bytes` bytes (a power of two, 16..2048) from `src`
 * at the row numbers ids[0..n_ids) (the caller keeps them inside `src`), in that order,
 * with blocks_per_cu workgroups per compute unit and `in_flight` (4, 8 or 16; 4 or 8 for
 * 2048-byte rows) rows outstanding per group of lanes that shares a row; nothing else is
 * computed and nothing is written.  What the memory system delivers to gathers of rows
 * of the size a benchmark gathers. */
int fusedMM_amd_gather_probe(const void *src, int row_bytes, const unsigned int *ids, int64_t n_ids, int blocks_per_cu,
                             int in_flight, int nontemporal, void *sink, void *stream);

#ifdef __cplusplus
}
#endif

#endif /* FUSEDMM_PROBES_H */
