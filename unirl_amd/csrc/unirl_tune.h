/*
 * unirl_tune.h -- extra entry points of the MEASUREMENT build (libunirl_hip_tune.so,
 * `python -m unirl_amd.build --tune`).  They exist for the benchmark only: yardstick
 * kernels and the device-side timeline.  The shipped libunirl_hip.so exports none of
 * them and include/unirl_hip.h does not declare them.
 */
#ifndef UNIRL_TUNE_H_
#define UNIRL_TUNE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* A plain streaming copy of
 * `bytes` (a multiple of 16, both pointers 16-byte aligned).  Hardware byte
 * counters read for this kernel calibrate the ones read for the kernels below. */
int unirl_calib_copy(const void* src, void* dst, size_t bytes, void* stream);

/* The launch floor of a
 * streaming kernel.  One kernel reads `read_bytes` from src and writes
 * `write_bytes` to dst (multiples of 16, 16-byte aligned; the two streams are
 * independent and no arithmetic is done), followed, when tail_launch != 0, by
 * a one-wavefront kernel -- the shape of a fused kernel plus its finalize
 * launch.  Timing it for the byte counts of a fused kernel gives the time no
 * kernel of that traffic can beat on the device.  sink: 16 writable bytes. */
int unirl_calib_stream(const void* src, size_t read_bytes, void* dst, size_t write_bytes,
                       int tail_launch, void* sink, void* stream);

/* What finishing a grid-wide reduction costs.
 * Sums the `read_bytes / 4` floats at src (a multiple of 16 bytes, 16-byte aligned) over
 * n_workgroups workgroups of 256 threads and finishes in one of three ways:
 *   mode 0  the streaming kernel only (per-workgroup partials stored, *out untouched);
 *   mode 1  plus a dependent second launch that adds the partials -- the scheme of every
 *           reducing entry point of this library;
 *   mode 2  a single launch: the partials are published as self-validating tagged 8-byte units
 *           (relaxed device-scope atomics) and polled by the last workgroup, bounded by a
 *           one-second clock budget (*out is NaN if it ever runs out).
 * scratch: at least 16 + 16 * n_workgroups bytes, zero-filled ONCE before its first use with
 * mode 2 (its first word carries the call tag from call to call) and used by one call at a
 * time.  Modes 1 and 2 return the same bits in *out. */
int unirl_calib_reduce(const void* src, size_t read_bytes, int mode, unsigned int n_workgroups,
                       void* scratch, size_t scratch_bytes, double* out, void* stream);

/* Device timeline: register a device buffer the traced kernels stamp {start, mark, mark, end}
 * clock readings into (NULL stops tracing); every launch made while a buffer is registered takes
 * the next slice and is logged.  unirl_trace_entry returns the i-th launch's kernel name, its
 * workgroup count and the offset of its slice in 8-byte words. */
int unirl_trace_begin(void* buf, size_t bytes);
int unirl_trace_count(void);
const char* unirl_trace_entry(int i, unsigned int* nblocks, size_t* offset_words);

#ifdef __cplusplus
}
#endif

#endif /* UNIRL_TUNE_H_ */
