/*
 * sgemm_debug.h - profiling aids of libsgemm.so.  Not part of the drop-in interface of sgemm.h: nothing here has a
 * counterpart in the reference, and a caller of the library never needs it.  bench.py uses both to produce the
 * time-stamp tables and the read-only ceiling under profiles/.
 */
#ifndef SGEMM_DEBUG_H
#define SGEMM_DEBUG_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Profiling aid, no counterpart in the reference.  While a buffer is set, every launch of the LDS-ring GEMM
 * kernels (per-tile and persistent), of the mid-batch GEMM kernel and of the 2:4 kernels takes the next grid * 8 words of it and each workgroup leaves eight 64-bit
 * words there when it is done: [0] kernel entry, [1] prologue DMAs issued, [2] first stage landed, [3] last stage
 * consumed, [4] outputs stored and acknowledged - 10 ns ticks of the device's constant 100 MHz clock -
 * [5], [6] shader clock at entry and end, [7] XCC_ID << 32 | HW_ID.  Launches that no longer fit leave nothing.
 * A launch recorded into a HIP graph keeps its slice on every replay.  Process-wide; set it from one thread while
 * no other thread launches.  sg_debug_stamps(NULL, 0) switches the stamps off again. */
int sg_debug_stamps(unsigned long long* device_buffer, size_t n_words);

/* Profiling aid, no counterpart in the reference: reads the n x k weight matrix B (row stride b_stride, k % 1024 == 0)
 * the way the persistent LDS-ring GEMM streams it - one workgroup per CU walking row tiles, eight waves sharing K,
 * direct-to-LDS loads with the streaming hint, two 4 KB slots per wave - and does nothing with it.  Its duration is the
 * ceiling of that access pattern on the device: what a GEMM's streaming phase is measured against.  segment_bytes is
 * what one load instruction takes contiguously from one row: 256 (4 rows per instruction - the GEMM's own pattern),
 * 512 (2 rows) or 1024 (1 row). */
int sg_debug_read_stream(const uint8_t* B, int n, int k, int b_stride, int segment_bytes, void* stream);

/* Profiling aid, no counterpart in the reference: what a CU takes in through direct-to-LDS loads when part of its
 * stream misses the XCD's L2 and part of it hits.  `workgroups` workgroups of `waves` waves (1, 2, 4, 8 or 16) issue
 * 1 KB loads (8 rows x 128 B, rows 8 KB apart - the mid-batch GEMM's pattern) with `depth` (4, 8 or 16, at most
 * 128 / waves) instructions in flight per wave for `ticks` x 10 ns and count them: counts[0] += loads of the cold
 * stream (a region of its own per wave out of `cold`, streaming hint), counts[1] += loads of the hot stream (one window
 * per XCD out of `hot`, walked by all its workgroups; make hot_bytes / 8 fit an L2).  cold_waves >= 0: waves below it
 * stream cold, the others hot; cold_waves < 0: every wave alternates hot_per_cold hot loads with one cold one.
 * The caller zeroes counts (two 64-bit words in device memory) and reads them after the stream has finished. */
int sg_debug_cu_ingest(const uint8_t* cold, size_t cold_bytes, const uint8_t* hot, size_t hot_bytes, int workgroups, int waves,
                       int cold_waves, int hot_per_cold, int depth, int ticks, unsigned long long* counts, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* SGEMM_DEBUG_H */
