/* sq_probes.h -- C ABI of libsq_probes.so: diagnostic kernels for MI355X (gfx950).
 *
 * None of these has a counterpart in the reference and none is part of the product library
 * (libsq_w4a16.so, include/sq_w4a16.h): the benchmark uses them to put its figures in context
 * (what the memory system charges for a weight stream, what the matrix pipes sustain under the
 * power limit, which clock the chip holds under a kernel's load).  Same conventions as the product
 * ABI: plain device pointers, a hipStream_t as void*, no allocation, no synchronisation; returns 0
 * or an SQP_ERR_* code, in which case nothing was launched.
 */
#ifndef SQ_PROBES_H
#define SQ_PROBES_H

#ifdef __cplusplus
extern "C" {
#endif

#define SQP_OK 0
#define SQP_ERR_NULL_POINTER 1
#define SQP_ERR_BAD_SHAPE 2
#define SQP_ERR_MISALIGNED 6
#define SQP_ERR_LAUNCH 7

/* reads an L1 weight and its zeros_scales exactly as the
 * single-token GEMV does (same grid, lane -> address mapping and loads in flight) and does nothing
 * else; its duration is what the memory system charges for the weight stream of one launch.  out:
 * at least ceil(N / 8) uint32 (practically never written).  Used by bench.py to report the read-only
 * floor of the decode step beside the measured figure. */
int sq_read_probe(const void* w, const void* zs, void* out, int N, int K, int group_size, void* stream);

/* `workgroups` workgroups of four waves (one per SIMD)
 * issue nothing but independent v_mfma_f32_32x32x16_f16, 16 * iters each, on operands taken from
 * data (5120 fp16 values, 16-byte aligned: the power drawn and so the sustained clock depend on
 * the operand bits).  out receives one uint64 per workgroup (shader-clock ticks spent in the loop)
 * followed by 4 scratch bytes, i.e. workgroups * 8 + 4 bytes.  Timed by the caller it gives the
 * fp16 matrix throughput the part sustains under its power limit (used by bench.py beside the
 * prefill figures). */
int sq_mfma_probe(const void* data, void* out, int workgroups, int iters, void* stream);

/* a single wave spins for `spins`
 * (1 .. 2^26) dependent multiply-adds and writes three uint64 to out: shader-clock
 * ticks elapsed, ticks of the constant 100 MHz counter elapsed, and a dummy.  Run on
 * a second stream beside a kernel it gives the clock the chip sustains under that
 * kernel's load (matrix-heavy kernels run power-limited, well below the nominal
 * clock that published peak rates assume). */
int sq_clock_probe(void* out, int spins, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* SQ_PROBES_H */
