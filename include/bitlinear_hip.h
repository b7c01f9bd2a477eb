/*
 * libbitlinear_hip.so -- C ABI of the MI355X (gfx950) ternary BitLinear library.
 *
 * Plain C: pointers and sizes only.  Every pointer is a DEVICE pointer owned
 * by the caller; the library neither allocates nor frees device memory in any
 * entry point below, never synchronises, and launches only on the stream it is
 * given (a hipStream_t passed as void*; NULL = the default stream).  All entry
 * points are therefore legal on a stream that is being captured into a graph.
 *
 * bf16 values are passed as raw 16-bit patterns (uint16_t).
 *
 * Weight operand ("packed"): int8 [N, K/4] exactly as the reference packer
 * writes it (gpu/pack_weight.py:76-98): stored 2-bit code = w + 2, 16x32 tiles
 * of 128 bytes, 16 codes interleaved per little-endian int32.  It is consumed
 * in place; no repack is needed.
 */
#ifndef BITLINEAR_HIP_H
#define BITLINEAR_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* status codes, returned by the int entry points and kept per host thread */
#define BITLINEAR_OK 0
#define BITLINEAR_ERR_SHAPE 1   /* N % 16 != 0, K % 64 != 0, or a size <= 0 */
#define BITLINEAR_ERR_NULL 2    /* a required pointer is NULL               */
#define BITLINEAR_ERR_LAUNCH 3  /* the HIP runtime refused the launch       */
#define BITLINEAR_ERR_ARG 4     /* bad mode / segment list / tuning value, or
                                   an operand not 16-byte aligned           */
#define BITLINEAR_ERR_SCRATCH 5 /* bitlinear_forward_bf16_static: the
                                   activation block exceeds the static scratch */
#define BITLINEAR_ERR_CAPTURE 6 /* bitlinear_forward_bf16_static: first call on a
                                   device made under a stream capture        */

/*
 * Drop-in replacement for the reference's only exported symbol
 *   extern "C" void bitlinear_int8xint2(int8_t*, int8_t*, __nv_bfloat16*,
 *        __nv_bfloat16*, __nv_bfloat16*, int, int, int, cudaStream_t)
 * (gpu/bitnet_kernels/bitnet_kernels.cu:3), bound by ctypes in
 * gpu/model.py:18-37 and gpu/test.py:13-29.
 *
 *   input0  int8 [M, K] row-major activations
 *   input1  packed ternary weight [N, K/4]
 *   output0 bf16 [M, N]; every element is written
 *   s       bf16 [M] activation scales (127/absmax); row m uses s[m]
 *   ws      bf16 weight scales, at least ws_num(N, K) entries
 * out[m, n] = bf16( float(acc[m, n]) / float(s[m]) * float(ws[n / (N / ws_num)]) )
 * with acc the exact int32 dot product (bitnet_kernels.h:79-82).  ws_num is
 * looked up from (N, K) with the reference's table (bitnet_kernels.cu:4-33)
 * and is 1 for shapes the reference has no instance for.  Unlike the
 * reference, any M >= 1, N % 16 == 0, K % 64 == 0 is computed; an unsupported
 * shape prints the reference's "required ladder gemm kernel" line, launches
 * nothing and sets the thread's status to BITLINEAR_ERR_SHAPE.
 */
void bitlinear_int8xint2(int8_t* input0, int8_t* input1, uint16_t* output0,
                         uint16_t* s, uint16_t* ws, int M, int N, int K,
                         void* stream);

/* Status of the calling host thread's most recent library call (the
 * reference's entry point returns void and reports nothing,
 * bitnet_kernels.cu:34-36). */
int bitlinear_last_status(void);
const char* bitlinear_status_string(int status);

/* The (N, K) -> ws_num table of bitnet_kernels.cu:4-33; 1 for other shapes. */
int bitlinear_ws_num(int N, int K);

/*
 * Same computation, also storing the raw int32 accumulators
 * (in_thread_C_local after the reduction, bitnet_kernels.h:74-78) to
 * acc_out [M, N].  output0 may be NULL (then s and ws may be NULL too).
 * Exists so tests can prove the accumulators bit-exact.
 */
int bitlinear_int8xint2_acc_i32(const int8_t* input0, const int8_t* input1,
                                int32_t* acc_out, uint16_t* output0,
                                const uint16_t* s, const uint16_t* ws,
                                int M, int N, int K, void* stream);

/*
 * Name of the product kernel that the calling host thread's most recent call
 * launched ("none" before the first).  M <= 16 takes the same kernel whether
 * or not acc_out is asked for, so a parity test of the accumulators reads what
 * the drop-in entry computes; tests and the smoke check report the name.  The
 * reference has one kernel and nothing to report (bitnet_kernels.cu:3-37).
 */
const char* bitlinear_last_kernel(void);

/*
 * Several products in one call.  Each element is one bitlinear_int8xint2 call
 * (same operands, same meaning, same results bit for bit); consecutive
 * elements of equal (M, N, K) with M <= 4 are executed by ONE kernel launch
 * whose waves walk the row blocks of all of them as one list (up to 48
 * problems per launch; longer runs take several), other elements are launched
 * one by one.  The problems of a call must be independent of each other: no
 * output0 may be an input of another element.  The reference has no such
 * entry: it launches one kernel per BitLinear (gpu/model.py:128, 160, 193,
 * 196), each far smaller than what MI355X must have in flight to use its HBM.
 * `problems` is a host array, read during the call only.
 */
typedef struct bitlinear_problem {
    const int8_t* input0;   /* int8 [M, K] */
    const int8_t* input1;   /* packed ternary weight [N, K/4] */
    uint16_t* output0;      /* bf16 [M, N] */
    const uint16_t* s;      /* bf16 [M] */
    const uint16_t* ws;     /* bf16, at least bitlinear_ws_num(N, K) entries */
    int M, N, K;
} bitlinear_problem;
int bitlinear_int8xint2_grouped(const bitlinear_problem* problems, int count, void* stream);

/*
 * Variant with explicit weight-scale segments: row n uses ws[j] for the first
 * j with n < seg_ends[j]  (seg_ends ascending, seg_ends[nseg-1] == N,
 * 1 <= nseg <= 8, host array).  This is the scale layout
 * gpu/convert_checkpoint.py:42-77 writes for fused tensors (q/k/v rows
 * 2560/640/640), which the reference kernel's equal-slot indexing
 * (bitnet_kernels.h:80) does not follow for wqkv.
 */
int bitlinear_int8xint2_seg(const int8_t* input0, const int8_t* input1,
                            uint16_t* output0, const uint16_t* s,
                            const uint16_t* ws, const int* seg_ends, int nseg,
                            int M, int N, int K, void* stream);

/*
 * Per-token absmax activation quantizer, BitLinearKernel.quant_input
 * (gpu/model.py:68-71):  s = 127 / max|x|.clamp(min=1e-5),
 * q = round_half_even(x * s).clamp(-128, 127).
 *   x bf16 [M, K] row-major, K % 8 == 0;  q int8 [M, K];  s bf16 [M].
 * torch evaluates 127 / t as t.reciprocal() * 127, and so do both modes:
 *   mode 0: r = 1/amax and r*127 in fp32, s = bf16(r*127), q from the exact
 *           fp32 product x * s (bit-identical to what torch.compile's
 *           Inductor CPU backend makes of the expression)
 *   mode 1: amax, r, s and the product x * s are each rounded to bf16
 *           (bit-identical to torch eager on bf16 tensors)
 */
int bitlinear_quant_absmax(const uint16_t* x, int8_t* q, uint16_t* s,
                           int M, int K, int mode, void* stream);

/*
 * The same quantizer, also storing rowsum[m] = sum_k q[m, k] (int32 [M]).  The
 * stored weight codes are w + 2 (gpu/pack_weight.py:80), so a product over the
 * codes is sum(w * q) + 2 * rowsum: a caller that multiplies codes itself needs
 * this sum; the library's own product kernels take it on the way.
 */
int bitlinear_quant_absmax_rowsum(const uint16_t* x, int8_t* q, uint16_t* s,
                                  int32_t* rowsum, int M, int K, int mode,
                                  void* stream);

/*
 * The load-time weight converter.  The kernels consume the layout the
 * reference packer writes (gpu/pack_weight.py:76-98) in place -- one packed
 * word is already the MFMA row operand of 16 consecutive k of one row -- so
 * the converted form IS the reference form: bitlinear_repacked_size returns
 * N * K / 4 bytes (0 for a shape the library does not take) and
 * bitlinear_repack copies (device to device, on the stream; a no-op when
 * source and destination are the same buffer).  They exist so that a loader
 * written against "convert at load time" keeps working if a later version of
 * the library prefers another layout.
 */
size_t bitlinear_repacked_size(int N, int K);
int bitlinear_repack(const int8_t* packed_ref, void* packed_out, int N, int K,
                     void* stream);

/*
 * BitLinearKernel.forward (gpu/model.py:73-75) in one call: quantizer (mode
 * as above), product and epilogue.  While the activation block is small
 * (M * K <= 16384 elements) this is ONE kernel: every workgroup (or every wave
 * its own slice of k) quantizes x itself, keeps the int8 rows in LDS and never
 * reads s from memory; five to eight tokens on rows of up to 3200 values
 * (mode 0, at most 256 workgroups) are one kernel too: every lane quantizes
 * for its own token, in registers.  Larger
 * blocks run the quantizer once, in a kernel of its own, and then the product
 * kernel (M <= 16: int8 rows staged in LDS per workgroup; M > 16: MFMA GEMM).
 *   q_ws (int8 [M, K], 16-byte aligned) and s_ws (bf16 [M]) receive the
 *   quantized activations and scales.  They may be NULL when M <= 16 and
 *   M * (K + 64) <= 60 KiB: the call then stays one kernel whatever M * K is
 *   (slower for large blocks); otherwise they are required.  Results equal
 *   bitlinear_quant_absmax followed by bitlinear_int8xint2 bit for bit.
 */
int bitlinear_forward_bf16(const uint16_t* x, const int8_t* packed,
                           uint16_t* output0, const uint16_t* ws,
                           int8_t* q_ws, uint16_t* s_ws,
                           int M, int N, int K, int mode, void* stream);

/*
 * bitlinear_forward_bf16 without workspace arguments, for callers that cannot
 * allocate device memory at all (code under graph capture that owns no
 * buffers of its own, tight serving loops, harnesses that forbid hipMalloc).
 * It has no counterpart in the reference, whose host shim allocates per call
 * (gpu/model.py:33).  The quantized rows and their scales, which
 * bitlinear_forward_bf16 keeps in q_ws / s_ws, live in a 16 MiB array inside
 * the library's device image (one copy per GPU, held until the process ends).
 * Limits: M <= 16384 tokens and M * K <= 16744448 activation elements (the
 * largest prompt block of the 2B shapes, 2048 x 6912, fits); beyond them the
 * call launches nothing and returns BITLINEAR_ERR_SCRATCH.  The array costs its
 * 16 MiB of device memory in every process that loads the library, on every GPU
 * it uses, whether or not this entry is ever called.  Same kernels and
 * the same bits as bitlinear_forward_bf16.  Allocates nothing and frees
 * nothing; the first call on a device looks the array's address up (a host
 * call, not stream work, which a stream capture in progress may refuse: made
 * under a capture, that first call launches nothing and returns
 * BITLINEAR_ERR_CAPTURE; every later call may be captured).  All calls on one GPU share the array: two of them
 * must not overlap in time (same stream, or ordered by events), or they race
 * on the quantized rows.  Nothing in the array needs clearing between calls:
 * every element the product reads was written by the same call's quantizer.
 */
int bitlinear_forward_bf16_static(const uint16_t* x, const int8_t* packed,
                                  uint16_t* output0, const uint16_t* ws,
                                  int M, int N, int K, int mode, void* stream);

/*
 * bitlinear_forward_bf16 that also stores the int32 accumulators of the product
 * (bitnet_kernels.h:74-78) to acc_out [M, N]: the same kernels, launch shapes
 * and results.  Exists so tests can prove the accumulators of the one-kernel
 * forward bit-exact.
 */
int bitlinear_forward_bf16_acc_i32(const uint16_t* x, const int8_t* packed,
                                   int32_t* acc_out, uint16_t* output0,
                                   const uint16_t* ws, int8_t* q_ws, uint16_t* s_ws,
                                   int M, int N, int K, int mode, void* stream);

/*
 * bitlinear_forward_bf16 with the operations that surround a BitLinear in the
 * reference's decoder folded in.  One kernel under the one-kernel conditions of
 * bitlinear_forward_bf16; otherwise a gate / norm / quantizer kernel (one
 * workgroup per token row, K <= 32768) followed by the product kernel, which
 * needs q_ws / s_ws as above; every product kernel has the residual epilogue:
 *   in front  y = RMSNorm(h) = bf16(h * rsqrt(mean(h^2) + eps) * norm_weight)
 *             (attention_norm / ffn_norm / attn_sub_norm / ffn_sub_norm,
 *             gpu/model.py:159, 195, 228-229); the sum of squares is taken in fp64,
 *             rounded to fp32 and divided by K in fp32; the two multiplies are fp32, one rounding to
 *             bf16.  With glu != 0, x is [M, 2K] = (x1 | x3) and
 *             h = bf16(bf16(relu(x1)^2) * x3) (gpu/model.py:164-166, 195);
 *             otherwise h = x, [M, K].
 *   behind    if residual != NULL: out = bf16(residual + bf16(result))
 *             (gpu/model.py:237-243), residual bf16 [M, N].
 *   norm_weight bf16 [K].  The reference uses xformers' RMSNorm, which is not
 *   part of its tree: the rounding points above are this library's definition.
 */
int bitlinear_norm_forward_bf16(const uint16_t* x, const uint16_t* norm_weight,
                                float eps, int glu, const int8_t* packed,
                                const uint16_t* ws, const uint16_t* residual,
                                uint16_t* output0, int8_t* q_ws, uint16_t* s_ws,
                                int M, int N, int K, int mode, void* stream);

/*
 * bitlinear_forward_bf16 and bitlinear_norm_forward_bf16 with the weight
 * scales assigned by explicit output-row segments, as bitlinear_int8xint2_seg
 * does for the plain product: rows [seg_ends[j-1], seg_ends[j]) use ws[j]
 * (seg_ends host array, strictly increasing, seg_ends[nseg-1] == N,
 * 1 <= nseg <= 8, every boundary a multiple of 16).  This is how
 * gpu/convert_checkpoint.py:42-50 lays the scales of a fused matrix out: wqkv
 * stores [s_q, s_k, s_v, 0] for segments of 2560 / 640 / 640 rows, which the
 * reference kernel's equal-thirds rule (bitnet_kernels.h:80) does not follow.
 * Opt-in: the plain entries keep the reference's rule bit for bit.  Same
 * kernels, launch shapes and arithmetic as the plain entries.
 */
int bitlinear_forward_bf16_seg(const uint16_t* x, const int8_t* packed,
                               uint16_t* output0, const uint16_t* ws,
                               const int* seg_ends, int nseg,
                               int8_t* q_ws, uint16_t* s_ws,
                               int M, int N, int K, int mode, void* stream);
int bitlinear_norm_forward_bf16_seg(const uint16_t* x, const uint16_t* norm_weight,
                                    float eps, int glu, const int8_t* packed,
                                    const uint16_t* ws, const int* seg_ends, int nseg,
                                    const uint16_t* residual, uint16_t* output0,
                                    int8_t* q_ws, uint16_t* s_ws,
                                    int M, int N, int K, int mode, void* stream);

/*
 * What the library would launch for a call, without launching it (host only:
 * works without a GPU).  Runs the dispatch code of the entry point itself --
 * entry 0: bitlinear_int8xint2, 1: bitlinear_forward_bf16 (mode 0, with
 * workspaces), 2: bitlinear_norm_forward_bf16 (norm), 3: the same with a
 * residual, 4: with gate and residual -- and writes into buf, for every kernel
 * of the call in launch order and joined by " + ", the kernel with its template
 * arguments, the grid, the workgroup size and the dynamic LDS bytes, e.g.
 * "bitlinear_solo_kernel<5, 1, 1, true, 0, false, 1> grid=(160,1,1) block=512
 * lds=0".  Returns the status the call itself would return for the shape.
 * The current bitlinear_set_tuning overrides apply.  No counterpart in the
 * reference, whose dispatch is a table of ten shapes (bitnet_kernels.cu:4-33).
 */
int bitlinear_plan_name(int entry, int M, int N, int K, char* buf, int buflen);

/*
 * Kernel / launch-shape override for tuning runs and tests.  Process-wide;
 * results never depend on it.
 *   kernel 0: built-in choice (other arguments ignored)
 *   kernel 2: split-K kernel always, a (1..16) waves per workgroup each
 *             keeping one to two rounds of b (1, 2, 4 or 8) 64-wide k-steps in flight
 *             (a = b = 0: the library's own launch shape)
 *   kernel 3: fused forward kernel with a (1..4) 16-row blocks per workgroup,
 *             b waves splitting K for each (a*b <= 16), c (4, 5, 8, 10 or 16)
 *             k-steps in flight per wave
 *   kernel 4: bitlinear_forward_bf16 always as two kernels
 *   kernel 5: prefill GEMM (M > 16) with output tile a per workgroup:
 *             0 = 64 x 128, 1 = 128 x 256, 2 = 64 x 256, 3 = 64 x 512, 4 = 32 x 128 (tokens
 *             x columns), 5 = 64 x 256 through the kernel that brings the activation
 *             chunks straight into LDS (the built-in choice for that tile when
 *             K % 128 == 0; a = 2 forces the other kernel), 6 = 32 x 256 and
 *             7 = 128 x 256 through that kernel (without K % 128 == 0: 32 x 128 and
 *             128 x 256 through the other), 8 = whole rounds of 64 x 256 tiles over
 *             the first columns and 32 x 128 tiles behind them in one launch (the
 *             built-in choice when those are at most about 1.4 per CU; needs
 *             K % 128 == 0); b = row tiles per band of the tile order (0 = the
 *             library's choice, up to 64); c = groups of four waves that split a
 *             tile's K between them (0 = the library's choice, 1, 2 (tiles 0 and 4)
 *             or 4 (tile 4))
 *   kernel 6: product of int8 rows (M <= 16) through the kernel that stages
 *             them in LDS: a = 0 built-in choice (M > 4 and N >= 6912), 1 whenever it
 *             fits, 2 never.  Independent of kernels 1..5; kernel 0 resets it.
 *   kernel 7: product of int8 rows (M <= 4) through the streaming kernel (one
 *             wave per 16-row block, no staging): a = 0 built-in choice, 1
 *             whenever it applies, 2 never (also in grouped calls); b = loads in
 *             flight per lane (0 = built-in choice, or 4, 5, 6, 7, 8, 10); c = waves
 *             per CU the launch is sized for (0 = built-in choice, up to 32).
 *             Applies with kernel 0 only; kernel 0 resets it.
 *   kernel 8: bitlinear_forward_bf16 (mode 0, M <= 4) through the kernel whose
 *             waves take the row maximum and quantize their own slice of k
 *             themselves (no workgroup-wide step in front of the products):
 *             a = 0 built-in choice (one token; two to four where measured faster), a = 1..4 always, with a
 *             16-row blocks per workgroup, b waves per row block and c (4, 5, 7 or
 *             8) k-steps per wave (a * b <= 16; b * c * 64 must cover K, else the
 *             built-in kernel runs), a = 5 never.  Applies with kernel 0 only;
 *             kernel 0 resets it.
 *   kernel 9: how that kernel takes the row maximum: a = 0 built-in choice, 1 =
 *             slice maxima exchanged between the waves of a workgroup (one
 *             barrier), 2 = every wave scans the whole rows (no barrier; one
 *             token up to K = 8192, two up to 4096, more up to 2560);
 *             b = 16-row blocks a wave multiplies its slice with: 0 built-in
 *             choice, 1..4 (more than one: one token, 5 or 8 k-steps per wave,
 *             at most as many as waves per row block; otherwise one).
 *             bitlinear_norm_forward_bf16 takes the same kernel (always
 *             exchanging) under the kernel 8 settings.  Kernel 0 resets it.
 *   kernel 10: the product of int8 rows (M <= 16) through the kernel that reads
 *             its activation operands straight from the caller's rows (no
 *             staging, one barrier): a = 0 built-in choice (many row blocks, or
 *             more than four tokens), a = 1 always, with b waves per row block
 *             and c (4, 5, 7 or 8) k-steps per wave (b * c * 64 must cover K,
 *             else the built-in kernels run; row blocks per wave from kernel 9's
 *             b), a = 2 never.  Applies with kernel 0 only; kernel 0 resets it.
 *   kernel 11: bitlinear_forward_bf16 (mode 0, M <= 8) in one launch through the
 *             kernel whose lanes quantize for their own token: a = 0 built-in
 *             choice (5 to 8 tokens, K <= 3200, at most 256 workgroups), 1 wherever
 *             its launch shape exists (waves of five k-steps cover K, one or four
 *             row blocks per wave; the kernel 8 setting a = 5
 *             keeps the one-to-four-token kernel out of the way), 2 never.
 *             Applies with kernel 0 only; kernel 0 resets it.
 */
int bitlinear_set_tuning(int kernel, int a, int b, int c);

#ifdef __cplusplus
}
#endif
#endif /* BITLINEAR_HIP_H */
