/*
 * Measurement probes of libbitlinear_hip.so.  Not part of the drop-in interface
 * (the reference has no counterpart): bench.py uses them to measure, in the same
 * run and launch style as its headline, what a kernel launch costs on this
 * machine when the kernel does nothing, when it only requests a matrix's bytes,
 * what the matrix pipe sustains on the operand values of this workload, and what handing a flag from one
 * workgroup to another costs.  Same conventions as include/bitlinear_hip.h: device pointers owned by
 * the caller, no allocation, no synchronisation, launches on the given stream.
 */
#ifndef BITLINEAR_PROBES_H
#define BITLINEAR_PROBES_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* One launch of a kernel with an empty body: `blocks` workgroups of `threads`
 * threads (1..1024).  Returns 0, 3 (launch failed) or 4 (bad argument). */
int bitlinear_probe_empty(int blocks, int threads, void* stream);

/*
 * One launch that requests every byte of `count` (1..48) packed weights of
 * shape [N, K/4] (host array of device pointers) with the streaming product
 * kernel's own grid, access pattern and software pipeline, and does nothing
 * with them beyond an exclusive-or that keeps the requests alive: no
 * activation operand, no decode, no MFMA, no output.  sink: one device word
 * that is practically never written (may be NULL).  Returns a BITLINEAR_* code.
 */
int bitlinear_probe_weight_stream(const int8_t* const* packed, int count, int N, int K,
                                  uint32_t* sink, void* stream);

/*
 * One launch of a register-only loop of v_mfma_i32_32x32x32_i8 that fills every
 * SIMD of the device with three waves (four accumulators per wave, 32 MFMAs
 * per iteration, no memory traffic): what the matrix pipe sustains for given
 * operand values.  mode 0: all operands zero; mode 1: random int8 activations
 * x random codes 1..3 (the products this library computes), the operands
 * changing with every MFMA.  The two differ, because switching activity
 * decides the power the pipe draws and the clock it is given.  iters:
 * 1..2^20.  *ops (host, may be NULL) receives the integer operations of the
 * launch (2 per multiply-add).  sink: one device word that is practically
 * never written (may be NULL).  Returns 0, 3 or 4 as above.
 */
int bitlinear_probe_mfma_i8(int mode, int iters, uint32_t* sink, long long* ops, void* stream);

/*
 * One launch in which workgroups wg_a and wg_b (indices within the launch,
 * 0..4095, different) hand a counter back and forth `rounds` (1..2^20) times
 * through two words of `flags` (device memory, at least 128 uint32, zeroed by
 * the caller before every call) with relaxed device-scope stores and loads:
 * launch duration / rounds is the round trip of a flag between two workgroups,
 * i.e. twice what one hand-over inside a launch costs.  Workgroups go to the
 * XCDs round-robin by index, so wg_b = wg_a + 8 lands on the same XCD and
 * wg_b = wg_a + 1 on the next.  Every wait is bounded; *gave_up (device int,
 * zeroed by the caller) becomes 1 if one ran out.  Returns a BITLINEAR_* code.
 */
int bitlinear_probe_flag_roundtrip(uint32_t* flags, int wg_a, int wg_b, int rounds, int* gave_up, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* BITLINEAR_PROBES_H */
