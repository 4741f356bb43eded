/* spfa_probe.h - measurement aid for benchmarks, exported by libspfa_probe.so.
 *
 * Not part of the drop-in boundary (spfa_hip.h, libspfa_hip.so) and without a counterpart in the
 * reference: nothing the six attention extensions do goes through this library. */
#ifndef SPFA_PROBE_H_
#define SPFA_PROBE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* The gather of the explicit-mask kernels with the arithmetic taken out: for each of the n_idx
 * entries of `idx` one row of `row_bytes` (64, 128, 256 or 512) bytes is loaded from `k` and one
 * from `v` (both of n_rows rows, n_rows < 2^31; an entry at or beyond n_rows - which includes
 * every entry with the top bit set - is skipped), 16 bytes per lane, `in_flight` (4, 8, 16 or 32)
 * rows of each per lane group issued back to back, by a persistent grid of wg_per_cu (1..8)
 * four-wavefront workgroups per compute unit whose wavefronts pull runs of `chunk` (>= 64) entries
 * off an atomic cursor (`cursor`: 4 bytes of device memory), or, with wg_per_cu = 0, by an ordinary
 * grid of one wavefront per run of `chunk` entries.  Nothing is computed or written.
 * When ev_start and ev_stop (hipEvent_t passed as void*) are both non-NULL they are attached to
 * the gather's own dispatch, so hipEventElapsedTime gives its duration without launch overhead.
 * The rate it reaches is what the memory system sustains for this access pattern at a given
 * working-set size: the ceiling a gather-bound kernel is priced against.  Returns the status
 * codes of spfa_hip.h (0: ok). */
int spfa_probe_gather(const void* k, const void* v, int64_t n_rows, int64_t row_bytes,
                      const uint32_t* idx, int64_t n_idx, int64_t chunk, int wg_per_cu, int in_flight,
                      void* cursor, void* ev_start, void* ev_stop, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* SPFA_PROBE_H_ */
