/*
 * tq_probe.h - measurement probes for the benchmark (libtq_probe.so), separate from the codec's C ABI.
 *
 * No counterpart in the reference: plain streaming and back-to-back MFMA launches whose sustained rates a
 * benchmark can set beside the published peaks.  The caller times them.
 */
#ifndef TQ_PROBE_H
#define TQ_PROBE_H
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

#define TQ_PROBE_ERR_ARG (-1)
#define TQ_PROBE_ERR_HIP (-4)
#define TQ_PROBE_MAX_ITERS 1000000

/* One launch that reads `bytes` from src (mode 0; dst may be NULL), writes `bytes` to dst (mode 1; src
 * ignored) or copies src to dst (mode 2); modes 3, 4, 5 are write, read and copy with the non-temporal hint on
 * every access.  chunked = 0: the lanes of the whole grid stride over the buffer;
 * 1: every workgroup takes one contiguous slice (reads and writes favour different orders on this part).
 * bytes: a multiple of 16; pointers 16-byte aligned.  stream: hipStream_t.  Returns 0 or a negative code. */
int tq_probe_stream(int mode, int chunked, const void *src, void *dst, int64_t bytes, void *stream);

/* One launch of `units` short-lived workgroups in dispatch order: workgroup u reads the 16 KB unit u of src
 * (src == NULL: reads nothing) and writes write_64ths / 64 of 16 KB (0 .. 64; 0: writes nothing) at
 * dst + u * 256 * write_64ths bytes: a read, a write, or a kernel's mix of the two (13: 3-bit K+V codes from
 * fp16 rows, 17: 4-bit) as one compact window moving through memory.  nontemporal != 0: the hint on every access.
 * src: units * 16 KB; dst: units * 256 * write_64ths bytes (16 bytes when write_64ths == 0); 16-byte aligned. */
int tq_probe_flat(const void *src, void *dst, int64_t units, int write_64ths, int nontemporal, void *stream);

/* One launch of `iters` (1 .. TQ_PROBE_MAX_ITERS) rounds of eight independent v_mfma_f32_32x32x16_f16 per
 * wavefront on every SIMD of the chip.  Returns the floating-point operations launched (> 0) or an error code
 * (< 0).  sink: 4 bytes of device memory (never written for valid inputs). */
int64_t tq_probe_mfma_f16(int64_t iters, float *sink, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* TQ_PROBE_H */
