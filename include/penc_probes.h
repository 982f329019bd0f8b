/*
 * penc_probes.h -- C ABI of libpenc_probes.so: memory-system probes for gfx950.
 *
 * Measurement aids, not part of the encoding: the benchmark uses them to measure, on the same GPU
 * and in the same run, the rates the encoding's memory traffic is priced against.  They have no
 * counterpart in the reference and are kept out of libpenc_hip.so.  Conventions as in penc.h
 * (device pointers, a hipStream_t as void*, PENC_OK or a PENC_ERR_* code).
 *   copy   : dst[i] = src[i] for n_float4 16-byte elements (streaming bandwidth, and the known-size
 *            kernel that hardware byte counters are scaled by)
 *   read   : reads n_float4 16-byte elements and writes at most one float per workgroup (`out` needs 16384 floats):
 *            the streaming rate of a kernel that only reads, which a copy (half reads, half writes) does not reach
 *   gather : every thread sums `per_thread` (1..9) independent 8-byte loads table[idx[k][thread]] and
 *            writes one 8-byte result; idx holds per_thread * n_threads slots.  Fed with the slots a
 *            workload really uses (penc_simplex_debug), level by level, it measures what the gathers of
 *            that level cost on this memory system.
 *   gather_variant : the same gathers with the knobs a kernel author could turn: `points_per_thread`
 *            (1, 2 or 4: per_thread * points_per_thread loads are in flight per lane; per_thread is 4, 5 or 9),
 *            `block_threads` (a multiple of 64 up to 1024) and `load_kind` (0 ordinary global load, 1 the
 *            compiler's non-temporal load, 2 + bits a raw buffer load with cache-policy bits: 1 = sc0, 2 = nt,
 *            16 = sc1; accepted: 2, 3, 4, 18, 19).  n_threads must be a multiple of points_per_thread.  The
 *            benchmark sweeps them and prices the encoding's gathers at the fastest setting found.
 *   scatter: every thread issues `per_thread` pairs of fp32 atomic adds at table[idx[k][thread]]
 */
#ifndef PENC_PROBES_H_
#define PENC_PROBES_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

int penc_probe_copy(const float* src, float* dst, int64_t n_float4, void* stream);
int penc_probe_read(const float* src, int64_t n_float4, float* out, void* stream);
int penc_probe_gather(const float* table, const int* idx, int64_t n_threads, int per_thread,
                      float* out, void* stream);
int penc_probe_gather_variant(const float* table, int64_t table_slots, const int* idx, int64_t n_threads,
                              int per_thread, int points_per_thread, int block_threads, int load_kind,
                              float* out, void* stream);
int penc_probe_scatter(float* table, const int* idx, int64_t n_threads, int per_thread, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* PENC_PROBES_H_ */
