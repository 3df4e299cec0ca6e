/* Measurement probes of libwoq: what the hardware allows, measured with the same harness as the kernels
 * (`python bench.py --mode ceilings`).  Not part of the drop-in boundary (include/woq.h lists what a
 * reference-side binding calls); no counterpart in the reference. */
#ifndef WOQ_PROBES_H_
#define WOQ_PROBES_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* woq_probe_read: a plain streaming read of `bytes` of device memory (every wavefront reads
 * kib_per_wave contiguous KiB, loads_in_flight of 1, 2, 4 or 8 16-byte loads per lane outstanding; nontemporal
 * != 0: loads with the non-temporal hint, as the streaming kernels read their weights); `sink` is 4 KiB of
 * device memory.  woq_probe_empty: a kernel that does nothing.  woq_probe_mfma:
 * nothing but matrix instructions (kind 0: v_mfma_f32_16x16x32_bf16, 1: v_mfma_f32_16x16x128_f8f6f4
 * on e4m3, 2: v_mfma_f32_32x32x16_bf16) on `workgroups` x 4 wavefronts, multiplying the same operand
 * registers every time (random_operands 0: least switching activity) or four pseudo-random operand pairs
 * in turn (1: what the power management sustains under real data); returns the floating-point
 * operations of the launch (negative on a bad argument).  Kinds 0 and 1 also leave two 32-bit counts at
 * sink + 4080: shader-clock cycles and ticks of the constant 100 MHz counter that the first wavefront spent
 * in its loop (their ratio x 100 = the MHz that wavefront ran at). */
int woq_probe_read(const void* src, size_t bytes, int kib_per_wave, int loads_in_flight, int nontemporal, void* sink,
    void* stream);
int woq_probe_empty(void* sink, void* stream);
double woq_probe_mfma(int kind, int random_operands, int iters, int workgroups, void* sink, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* WOQ_PROBES_H_ */
