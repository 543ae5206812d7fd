/* sq_w4a16.h -- C ABI of libsq_w4a16.so: W4A16 quantized linear on MI355X (gfx950).
 *
 * Every entry point takes plain device pointers and sizes, launches on the
 * given HIP stream (a hipStream_t passed as void*; NULL = the null stream),
 * never allocates or frees device memory, never synchronises, never throws.
 * The return value is 0 on success or one of the SQ_ERR_* codes; on any error
 * nothing has been launched.  All matrices are dense and row-major.
 *
 * Weight layouts
 *   SQ_LAYOUT_L1  weight  uint8 [N, K/2] == uint32 [N, K/8]; the nibbles of a
 *                 word, least significant first, hold k0,k2,k4,k6,k1,k3,k5,k7
 *                 of 8 consecutive k.  zeros_scales fp16 [N, 2K/g]: pairs
 *                 (zero + 64, scale) per (row, group).
 *                 (reference: test/muxi/utils/quant_funcs.py:75-83,116-127,142-174)
 *   SQ_LAYOUT_L2  weight  int32 [K, N/8] in the tensor-core tile order produced
 *                 by convert_ours_to_awq + convert_awq_to_lmdeploy;
 *                 zeros_scales fp16 [K/g, 2N]: pairs (zero + 64, scale) per
 *                 (group, column).  Group size must be 128.
 *                 (reference: test/nvidia/utils/quant_dequant_nvidia.py:5-32)
 */
#ifndef SQ_W4A16_H
#define SQ_W4A16_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SQ_OK 0
#define SQ_ERR_NULL_POINTER 1    /* a required pointer is NULL */
#define SQ_ERR_BAD_SHAPE 2       /* M/N/K out of range or not a supported multiple */
#define SQ_ERR_BAD_GROUP 3       /* unsupported group size */
#define SQ_ERR_BAD_LAYOUT 4      /* unknown layout id */
#define SQ_ERR_BAD_ALGO 5        /* unknown or inapplicable kernel id */
#define SQ_ERR_MISALIGNED 6      /* pointer not 16-byte aligned */
#define SQ_ERR_LAUNCH 7          /* the HIP runtime rejected the launch */
#define SQ_ERR_WORKSPACE 8       /* workspace missing or too small */
#define SQ_ERR_STATIC_WS 9       /* sq_w4a16_gemm_static_ws: the shape needs more than SQ_STATIC_WS_BYTES */
#define SQ_ERR_SEQ_TIMEOUT 10    /* sq_w4a16_gemv_sequence_status: a one-launch sequence gave up a wait */

#define SQ_LAYOUT_L1 1
#define SQ_LAYOUT_L2 2

/* Kernel selection for sq_w4a16_gemm_ex (SQ_ALGO_AUTO is what sq_w4a16_gemm uses). */
#define SQ_ALGO_AUTO 0
#define SQ_ALGO_GEMV 1           /* M <= 8: lane-private rows on 4x4x4 MFMA, exact W_hat */
#define SQ_ALGO_GEMV_FIXUP 2     /* M <= 8: same, zero/scale applied per group in fp32 */
#define SQ_ALGO_SKINNY 3         /* M <= 64: 16-column MFMA tiles, weights straight from registers */
#define SQ_ALGO_GEMM 4           /* any M: LDS-tiled MFMA GEMM */
#define SQ_ALGO_SKINNY_WS 5      /* M <= 32: 64-row tiles, K split over workgroups through a workspace
                                    (sq_w4a16_gemm_ws only) */
#define SQ_ALGO_STREAM 6         /* M <= 16 at group size 128 or 64, M <= 32 at group size 128: weight loads a fixed
                                  * distance ahead of the arithmetic, activations staged in LDS first; K beyond 4096
                                  * is split through the workspace */

/* Library version (major*10000 + minor*100 + patch). */
int sq_version(void);

/* Static, human-readable text for an SQ_ERR_* code. */
const char* sq_strerror(int code);

/* Y[M,N] (fp16) = X[M,K] (fp16) * W_hat^T, W_hat[n,k] = (q - z) * s, fp32
 * accumulation.  Replaces the body of gemm_awq_ut / Gemm_awq_pure
 * (reference: quantization/muxi/backend/gemm_quant.cu:12-59,84-109;
 * quantization/nvidia/kernel/gemm_quant.cu:13-40,98-123).
 * Requirements: N % 8 == 0; K % 32 == 0; K % g == 0; g in {32,64,128}; x, w, zs,
 * y 16-byte aligned.  M == 0 is accepted and launches nothing.  The kernels
 * consume layout L1; for SQ_LAYOUT_L2 the call returns SQ_ERR_BAD_LAYOUT: convert
 * the weight once with sq_repack_l2_to_l1 (the `quant` extension does this behind
 * gemm_awq_ut and caches the result for the life of the source tensor). */
int sq_w4a16_gemm(const void* x, const void* w, const void* zs, void* y,
                  int M, int N, int K, int group_size, int layout, void* stream);

/* Same with an explicit kernel choice (tests and benchmarks). */
int sq_w4a16_gemm_ex(const void* x, const void* w, const void* zs, void* y,
                     int M, int N, int K, int group_size, int layout, int algo,
                     void* stream);

/* Same product with a caller-owned device workspace, which lets the kernels split K
 * over workgroups where a single pass cannot fill the chip (fp32 partial tiles, summed
 * in a fixed order by the workgroup that finishes last, so results are
 * bit-reproducible).  No counterpart in the reference.  The workspace must hold at
 * least sq_w4a16_workspace_bytes(M, N, K) bytes, be 16-byte aligned, and have its
 * first 64 KiB zeroed before the first call (every call leaves them zero); calls that
 * share a workspace must not overlap in time.  With SQ_ALGO_AUTO the split is taken
 * where it is the fastest: the streaming decode kernel for 3..16 tokens at group size
 * 128 when K exceeds 4096 (a shorter K needs no split and no workspace), the split-K
 * decode kernel for 5..32 tokens otherwise on weights of 2^25 elements or more or with
 * K > 8192 and for 17..32 tokens on any weight, the same kernel in two blocks for 33..48
 * tokens on such weights, and a K split of the tiled GEMM for larger M whose grid would
 * leave most CUs idle and for 17..32 tokens on weights of 2^25 elements or more that the
 * two-tile streaming kernel would serve in part-empty rounds of workgroups (K a multiple
 * of 256; at group size 64 and 32, N >= 8192).  A workspace that is NULL, misaligned or too small is ignored under
 * SQ_ALGO_AUTO (the workspace-free kernels run); an explicit SQ_ALGO_SKINNY_WS then
 * returns SQ_ERR_WORKSPACE. */
int sq_w4a16_gemm_ws(const void* x, const void* w, const void* zs, void* y,
                     int M, int N, int K, int group_size, int layout, int algo,
                     void* workspace, size_t workspace_bytes, void* stream);

/* Measured kernel choice.  In the role of TurboMind's measuring mode, which times its 17 tile
 * configurations on the shape at hand and keeps the fastest (reference:
 * quantization/nvidia/kernel/gemm_s4_f16/gemm_s4_f16.cu:92-197, gemm_s4_f16_kernel.h:83-134);
 * SQ_ALGO_AUTO's built-in rules are constants from sweeps of the OPT-6.7B / Llama-2-7B shapes.
 * sq_w4a16_autotune runs the product x * W_hat^T with every kernel family and tuning that can
 * serve (M, N, K, group_size) -- the decode GEMV's workgroup shapes, the streaming kernel's row
 * blocks and K splits, the split-K kernel's splits, the tiled GEMM's tile heights, K splits and
 * staging variants -- `reps` launches each between two HIP events on `stream`, and records the
 * fastest in a process-wide table that SQ_ALGO_AUTO consults first from then on, for exactly
 * this (M, N, K, group_size) and workspace situation (a workspace of at least
 * sq_w4a16_workspace_bytes(M, N, K) bytes present or not).  This is the one GEMM entry point
 * that SYNCHRONISES (once per candidate) and creates host-side event objects; it allocates no
 * device memory.  y is written by every candidate and holds the chosen kernel's result at the end.
 *   copies, w_stride, zs_stride  copies > 1: candidate launch i reads the weight at
 *             w + (i % copies) * w_stride and its zeros/scales at zs + (i % copies) * zs_stride
 *             (bytes, multiples of 16), so that a pool larger than the 256 MB last-level cache is
 *             timed from HBM, as a decode step meets its weights; copies = 1 times one weight,
 *             which stays in that cache when it is smaller.
 *   best_algo  (may be NULL) the chosen kernel word for sq_w4a16_gemm_ex / _ws, 0 when the built-in
 *             choice was not beaten (then nothing is recorded); best_us, auto_us (may be NULL) the
 *             average launch time of the chosen and of the built-in choice.
 * sq_w4a16_autotune_clear forgets every recorded choice and returns how many there were.  The table
 * is append-only (1024 recordings per process; later ones are measured but not kept). */
int sq_w4a16_autotune(const void* x, const void* w, const void* zs, void* y, int M, int N, int K,
                      int group_size, int layout, void* workspace, size_t workspace_bytes, int copies,
                      size_t w_stride, size_t zs_stride, int reps, void* stream, int* best_algo,
                      float* best_us, float* auto_us);
int sq_w4a16_autotune_clear(void);

/* sq_w4a16_gemm_ws for callers that cannot allocate device memory: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the
 * reference.  Same product, same kernels and the same automatic kernel choice, bit-identical
 * results; the workspace is a buffer of SQ_STATIC_WS_BYTES (16 MiB + 64 KiB) that lives inside
 * the library's device code, one copy per GPU for the life of the process, so the call
 * allocates and frees nothing.  The caller still passes inputs and the output.
 * Limit: a call whose kernels would take more than SQ_STATIC_WS_BYTES from a workspace is rejected
 * with SQ_ERR_STATIC_WS and nothing is launched: the split-K decode kernels at 3..32 tokens (every
 * such batch with N <= 16384 fits) and the K splits of the tiled GEMM beyond 16 tokens.  One or two
 * tokens, and a GEMM whose grid fills the chip without a K split, use no workspace and are never
 * rejected, whatever N is.
 * The first call on a device looks the buffer's address up (hipGetSymbolAddress); nothing is
 * cleared, the array is zero when the library is loaded and every kernel leaves its counters zero.
 * Every call on a GPU shares that GPU's buffer: calls that overlap in time on one GPU (two
 * streams, two threads) race; calls on one stream are ordered and safe.  The buffer keeps the
 * last call's partial sums; the kernels overwrite what they read and leave the counters zero. */
#define SQ_STATIC_WS_BYTES (16 * 1024 * 1024 + 64 * 1024)
int sq_w4a16_gemm_static_ws(const void* x, const void* w, const void* zs, void* y,
                            int M, int N, int K, int group_size, int layout, int algo,
                            void* stream);

/* Workspace hygiene (no counterpart in the reference).  Every workspace-taking entry point above
 * and below relies on one invariant: the counter region at the start of its workspace (64 KiB for
 * sq_w4a16_gemm_ws / _fused, 1 KiB for sq_decode_attention, all 256 bytes for
 * sq_w4a16_gemv_sequence) is zero when a call starts, every call leaves it zero, and calls that
 * share a workspace do not overlap in time.  Inside the kernels, partial results are exchanged
 * between workgroups with stores and loads at the device-coherent cache level (sc1) followed by a
 * wait for the stores and a relaxed agent-scope counter; no device-wide release / acquire fence is
 * used, so correctness rests on that cache-policy behaviour of gfx950.  A launch that dies midway,
 * or two streams sharing a workspace, can leave counters non-zero; later calls on that workspace
 * would then never find a last arriver and leave their output unwritten.
 *   sq_workspace_reset  clears `bytes` (a multiple of 4, workspace 16-byte aligned) with a small
 *                       fill kernel on `stream` (not a memset node: safe under HIP-graph capture);
 *                       use it at workspace creation and on error paths.
 *   sq_workspace_check  debugging aid, the one entry point that SYNCHRONISES: copies the first
 *                       min(bytes, 64 KiB) back on `stream`, waits, and returns SQ_ERR_WORKSPACE if
 *                       any word is non-zero (a previous call did not complete, or calls raced). */
int sq_workspace_reset(void* workspace, size_t bytes, void* stream);
int sq_workspace_check(const void* workspace, size_t bytes, void* stream);

/* Bytes sq_w4a16_gemm_ws / sq_w4a16_gemm_fused can use for this shape (8.06 MiB for
 * every decode batch with N <= 16384; up to tens of MiB for the GEMM split). */
size_t sq_w4a16_workspace_bytes(int M, int N, int K);

/* The same product with the element-wise tail of the linear folded into the kernel's
 * store: Y = act(X * W_hat^T + bias) + residual, computed on the fp32 accumulator and
 * rounded to fp16 once.  bias fp16 [N] or NULL; residual fp16 [M, N] or NULL (must not
 * overlap y); act SQ_ACT_NONE, SQ_ACT_RELU or SQ_ACT_SILU (v / (1 + exp(-v))).  workspace may be NULL (then the
 * workspace-free kernels are used); otherwise as for sq_w4a16_gemm_ws.  Replaces the
 * separate `out + bias` of WALinear.forward (reference:
 * test/nvidia/module/qlinear/qlinear.py:69-70), the ReLU after fc1 and the residual
 * adds of the decoder layer (reference:
 * test/nvidia/module/opt/modeling_opt_ours.py:590,608-609,614), in the role of the
 * fused gemm_awq_residual_ut family the reference scripts import from a package that
 * is not part of it (quantization/nvidia/script/gemm_awq_test.py). */
#define SQ_ACT_NONE 0
#define SQ_ACT_RELU 1
#define SQ_ACT_SILU 2
int sq_w4a16_gemm_fused(const void* x, const void* w, const void* zs, const void* bias,
                        const void* residual, void* y, int M, int N, int K, int group_size,
                        int layout, int act, int algo, void* workspace, size_t workspace_bytes,
                        void* stream);

/* Front half of a gated MLP: Y = silu(X * W_gate_hat^T) .* (X * W_up_hat^T), two launches: the up
 * projection into up_scratch (fp16 [M, N], caller-allocated, must not overlap y; holds the up
 * projection afterwards), then the gate projection, whose store applies SiLU to the fp32
 * accumulator and multiplies by up_scratch before the one rounding of Y.  Both weights are [N, K]
 * with their own zeros/scales; for a packed weight cat(W_gate, W_up) in layout L1 pass the two
 * row slices (w_up = w + N * K / 2 bytes, zs_up = zs + N * (K / g) * 4 bytes).  workspace as for
 * sq_w4a16_gemm_ws (may be NULL).  In the role of gemm_awq_silu_dot_ut, which the reference's
 * kernel test imports from a package that is not part of it; the expected value and tolerance
 * are that test's: silu(x W1^T) * (x W2^T) within atol = rtol = 2e-2 (reference:
 * quantization/nvidia/script/gemm_awq_test.py:50-56,66-72,105). */
int sq_w4a16_gemm_silu_dot(const void* x, const void* w_gate, const void* zs_gate, const void* w_up,
                           const void* zs_up, void* y, void* up_scratch, int M, int N, int K,
                           int group_size, int layout, void* workspace, size_t workspace_bytes,
                           void* stream);

/* Up to SQ_SEQUENCE_MAX decode linears (1..4 tokens) with one call:
 *     for l in 0 .. count-1:  y_l = act_l(x_l * W_hat_l^T + bias_l) + residual_l
 * executed in order.  No counterpart in the reference, which launches its GEMV once per linear
 * (quantization/muxi/backend/w4a16_gemm.cuh:14-326 under test/muxi/module/qlinear/qlinear.py:61-70);
 * at one token every such launch spends about as long getting started as streaming its weights.
 * Consecutive linears that do not depend on each other and share K and the group size (q, k and v
 * of a decoder layer, kept as three weights) are served by ONE launch whose grid is the
 * concatenation of their row blocks (the decode GEMV up to 4 tokens; the split-K decode kernel for
 * 5..32 tokens when a workspace is given); a linear that depends on an earlier one starts a new
 * launch.
 *   depends  set it on linear l when x_l or residual_l (or any buffer it reads) is written by an
 *            earlier linear of the same call.  Linears without it may run ahead of earlier ones.
 *            A buffer written by linear i may be read or overwritten by linear j > i only if j, or
 *            a linear between them, has depends set; y_l must not alias x_l or residual_l.
 *   mode     SQ_SEQ_AUTO: as above;
 *            SQ_SEQ_ONE_LAUNCH: everything in one persistent launch (one workgroup per CU stays
 *            resident and the weight stream runs on across the linears).  There is no grid
 *            barrier: an output that a later linear of the call reads (x_j or residual_j is exactly
 *            the buffer y_i, same address and extent) is also written to the workspace as 8-byte
 *            words {two fp16, launch tag}, and the reader repeats its load until the tags are the
 *            launch's, so a dependency costs one store and one load; meanwhile the waiting
 *            workgroup keeps fetching the next weights into LDS.  Needs 1..4 tokens, one group size
 *            for all linears, bias and residual 4-byte aligned, activations of a linear within LDS
 *            (M * K * 2 bytes up to about 64 KiB), a data flow it can see (depends set only where a
 *            pointer matches an earlier y; no output that aliases a buffer an unordered linear
 *            still reads) and every workgroup resident at once (one per CU: the GPU otherwise idle;
 *            other work delays it, and a workgroup that never becomes resident makes the others'
 *            waits run out).  Whatever does not fit is launched as under SQ_SEQ_AUTO.
 *   workspace  NULL, or sq_w4a16_gemv_sequence_workspace_bytes(linears, count, M) bytes, 16-byte
 *            aligned, ALL of it zero before the first call; calls that share it must be ordered and
 *            must describe the same list.  Its first part is the split-K workspace of
 *            sq_w4a16_gemm_ws (64 KiB of counters, every call leaves them zero, and with 3..32
 *            tokens the partial tiles of the linears that may share a launch); behind it lies the
 *            region of SQ_SEQ_ONE_LAUNCH (launch number, sticky error word, exit counter, exchange
 *            words), which only that mode touches.
 * sq_w4a16_gemv_sequence_status (the one call here that SYNCHRONISES) reads that region back:
 * SQ_OK, SQ_ERR_SEQ_TIMEOUT if a wait for another workgroup's output ever ran out of polls since
 * the word was last cleared (the results of that call are undefined; `clear` != 0 resets the word
 * with a fill kernel on `stream`), SQ_ERR_WORKSPACE if a launch did not finish.
 * sq_w4a16_gemv_sequence_tune sets, process-wide, the number of polls a wait may take (default
 * 65536, each a round trip to memory) and the loads a streaming wave keeps in flight (0 = default,
 * at most 16); tests use a poll limit of 0 to drive the give-up path from the host.
 * Shapes as for sq_w4a16_gemm (all linears share M).  A lone linear, M > 32, and whatever does not
 * fit the rules above is launched linear by linear on the stream (the automatic dispatch of
 * sq_w4a16_gemm_ws): same results. */
#define SQ_SEQ_AUTO 0
#define SQ_SEQ_ONE_LAUNCH 1
#define SQ_SEQUENCE_MAX 8
typedef struct sq_linear_desc {
    const void* x;         /* fp16 [M, K] */
    const void* w;         /* layout L1 */
    const void* zs;
    const void* bias;      /* fp16 [N] or NULL */
    const void* residual;  /* fp16 [M, N] or NULL */
    void* y;               /* fp16 [M, N] */
    int N, K, group_size;
    int act;               /* SQ_ACT_NONE or SQ_ACT_RELU */
    int depends;           /* see above */
} sq_linear_desc;
int sq_w4a16_gemv_sequence(const sq_linear_desc* linears, int count, int M, int layout, int mode,
                           void* workspace, size_t workspace_bytes, void* stream);
size_t sq_w4a16_gemv_sequence_workspace_bytes(const sq_linear_desc* linears, int count, int M);
int sq_w4a16_gemv_sequence_status(const sq_linear_desc* linears, int count, int M, void* workspace,
                                  size_t workspace_bytes, int clear, void* stream);
int sq_w4a16_gemv_sequence_tune(unsigned spin_limit, int loads_in_flight);

/* out[N,K] (fp16) = W_hat in natural k order, bit-identical to fp16
 * (q_fp16 - z_fp16) * s_fp16.  Replaces dequant
 * (reference: quantization/tianshu/backend/gemm_quant.cu:153-164 and
 * quantization/tianshu/backend/w4a16_gemm.cuh:1060-1154). */
int sq_w4a16_dequant(const void* w, const void* zs, void* out, int N, int K,
                     int group_size, int layout, void* stream);

/* zeros, scales fp16 [N, K/g] (zeros without the +64) -> zs fp16 [K/g, 2N]
 * = pairs (zero + 64, scale).  Replaces transpose_merge_zeros_scales
 * (reference: quantization/nvidia/kernel/gemm_s4_f16/format.cu:206-239). */
int sq_transpose_merge_zeros_scales(const void* zeros, const void* scales, void* zs,
                                    int in_features, int out_features, int group_size,
                                    void* stream);

/* src uint8 [N, K/2] (even k in the high nibble) -> dst uint32 [K, N/8], word
 * (k,c) holding columns 8c + {0,2,4,6,1,3,5,7}.  Replaces convert_ours_to_awq
 * (reference: quantization/nvidia/kernel/gemm_s4_f16/format.cu:151-201). */
int sq_convert_ours_to_awq(const void* src, void* dst, int in_features, int out_features,
                           void* stream);

/* src uint32 [K, N/8] (AWQ order) -> dst int32 [K, N/8] storage in layout L2.
 * Replaces convert_awq_to_lmdeploy
 * (reference: quantization/nvidia/kernel/gemm_s4_f16/format.cu:24-57,66-71,135-149).
 * Needs K % 32 == 0 and N % 32 == 0; src and dst must not overlap. */
int sq_convert_awq_to_lmdeploy(const void* src, void* dst, int in_features, int out_features,
                               void* stream);

/* Layout L2 -> layout L1 (weight and zeros_scales), so that an L2 checkpoint
 * can be served by the L1 kernels.  No counterpart in the reference (its
 * back-ends each accept one layout only). */
int sq_repack_l2_to_l1(const void* w_l2, const void* zs_l2, void* w_l1, void* zs_l1,
                       int N, int K, int group_size, void* stream);

/* 2-bit packed weight uint8 [N, K/4] -> 4-bit packed uint8 [N, K/2] (layout
 * L1 nibbles).  Replaces WALinear.convert_2bit_to_4bit
 * (reference: test/muxi/module/qlinear/qlinear.py:93-103). */
int sq_convert_2bit_to_4bit(const void* src, void* dst, int N, int K, void* stream);

/* Layout L2 with 2-bit storage: int32 [K, N/8] (4-bit words) -> int32 [K, N/16] and back, with
 * the arithmetic the reference's Python performs.  Shifts bind tighter than `&` in its
 * expressions, so a pair of words (a, b) is stored as (a & 0xFFFF0000) + (b & 0x0000FFFF) and a
 * stored word w expands to (w & 0x33333333, w & 0x33333333): the two are not inverses, and the
 * library reproduces them bit for bit so that a 2-bit layer computes what it computes there.
 * Replace convert_4bit_to_2bit / convert_2bit_to_4bit
 * (reference: test/nvidia/utils/quant_dequant_nvidia.py:34-43 and :45-54; called from
 * test/nvidia/module/qlinear/qlinear.py:58-62).  N must be a multiple of 16. */
int sq_l2_convert_4bit_to_2bit(const void* src, void* dst, int K, int N, void* stream);
int sq_l2_convert_2bit_to_4bit(const void* src, void* dst, int K, int N, void* stream);

/* LUT block-sparse attention, prefill: out[z,h,m,:] = softmax over the keys of the
 * blocks lut[h][m/64][0..nnz) of (q k^T * sm_scale) (optionally causal) times v.
 * q, k, v, out fp16 [Z, H, S, D] contiguous, D in {64, 128}; lut int32 or int64
 * (lut_elem_bytes 4 or 8) [H, ceil(S/64), nnz], key-block indices of 64 keys; an
 * entry equal to its predecessor in the row is padding (a block named again after a
 * different one is attended, and weighted, again); at most ceil(S/64) entries of a row
 * are visited; entries outside [0, ceil(S/64)) select nothing.  A query row without any
 * visible key gives NaN, as in the reference.  Replaces sparse_attention_prefill (reference:
 * sparse-attention/nvidia/playground/kernels/block_sparse_attention_lut.py:22-243;
 * sparse-attention/muxi/playground/kernels/csrc/src/block_sparse_attention_lut.cu:49-55). */
int sq_lut_attention_fwd(const void* q, const void* k, const void* v, void* out, const void* lut,
                         int lut_elem_bytes, int Z, int H, int S, int D, int nnz, float sm_scale, int causal,
                         void* stream);

/* Dense decode attention, one query token per sequence (q_len == 1 < kv_len):
 *   out[b,h,:] = sum_j P[j] v[b,h,j,:],  P = softmax_j(q[b,h,:] . k[b,h,j,:] * sm_scale + mask[b,j])
 * over the first L rows of an fp16 key/value cache, softmax and accumulation in fp32 (one
 * streaming pass with an online softmax; the reference's rounding of P to fp16 is not
 * reproduced, the result is within that rounding of it).  Replaces the decode branch of
 * sparse_attention (reference: sparse-attention/nvidia/playground/kernels/
 * block_sparse_attention_lut.py:272-300), which runs two torch.matmul and a softmax.
 *   q          fp16, element (b,h,d) at q[b*q_bstride + h*q_hstride + d]
 *   k_cache, v_cache  fp16, row j of (b,h) at cache[b*cache_bstride + h*cache_hstride + j*D],
 *              room for Lmax rows per (b,h) (cache_hstride >= Lmax*D)
 *   k_new, v_new  both NULL, or the step's new key/value rows, element (b,h,d) at
 *              new[b*new_bstride + h*new_hstride + d]: they are stored to cache row
 *              cache_len and take part in the attention (L = cache_len + 1); without them
 *              L = cache_len.  (Extension over the reference, which appends with torch.cat
 *              before the call; it saves two copy launches per layer.)
 *   mask       NULL or fp16 additive mask, element (b,j) at mask[b*mask_bstride + j], j < L
 *              (the reference's attention_mask [bsz,1,1,kv_len])
 *   out        fp16 [B, H, D] contiguous (= [B, 1, H*D], the layout the output projection reads)
 *   cache_len  rows already valid; cache_len_dev, if not NULL, points to that number on the
 *              device (int64) and overrides cache_len -- read by the kernel, so a captured HIP
 *              graph follows a growing cache; the kernel clamps it to the cache size.
 *   workspace  NULL, or sq_decode_attention_workspace_bytes(B, H, D) bytes, 16-byte aligned, its
 *              first 1024 bytes (256 counters, a fixed region whatever B*H is) zero before the first call
 *              (every call leaves them zero), so one workspace serves calls with different B*H.  The kernel
 *              runs one workgroup per (batch, head); with fewer than 256 of them and a workspace
 *              the cache rows of a head are shared among up to 16 workgroups whose partial
 *              softmax states meet in the workspace (batch 1, 32 heads, 640 rows: 4 workgroups
 *              per head).  Calls that share a workspace must be ordered (same stream).
 * D in {64, 128}; all strides in elements and multiples of 8; pointers 16-byte aligned.  A fully
 * masked row gives NaN, as in the reference. */
int sq_decode_attention(const void* q, const void* k_new, const void* v_new, void* k_cache, void* v_cache,
                        const void* mask, void* out, int B, int H, int D, int Lmax, long q_bstride, long q_hstride,
                        long new_bstride, long new_hstride, long cache_bstride, long cache_hstride, long mask_bstride,
                        int cache_len, const long long* cache_len_dev, float sm_scale, void* workspace,
                        size_t workspace_bytes, void* stream);
size_t sq_decode_attention_workspace_bytes(int B, int H, int D);

/* LayerNorm over the last dimension: y[r,:] = (x[r,:] - mean) * rsqrt(var + eps) * gamma + beta,
 * biased variance, statistics and arithmetic in fp32, x and y fp16 [rows, cols] contiguous (y may
 * be x), gamma / beta fp16 [cols] or NULL; cols a multiple of 8, at most 16384.  Feeds the q/k/v and
 * fc1 linears of a decoder layer, where torch's nn.LayerNorm costs as much as a decode GEMV
 * (reference: test/nvidia/module/opt/modeling_opt_ours.py:500-507,561-562,603-604). */
int sq_layernorm(const void* x, const void* gamma, const void* beta, void* y, int rows, int cols, float eps,
                 void* stream);

/* LayerNorm followed by the fused linear, y = act(LN(x) W_hat^T + bias) + residual, as ONE entry point: what a
 * pre-LN decoder layer does in front of q/k/v and fc1 (reference: test/nvidia/module/opt/modeling_opt_ours.py:
 * 561-562 with 505-506, and 603-604 with 608; nn.LayerNorm and the linear are separate modules there).
 * Where sq_w4a16_ln_fusable() says 1 (layout L1, group size 128, up to 8 tokens, 2048 < K <= 4096) the
 * normalisation happens inside the linear's kernel: every workgroup of the streaming decode kernel stages the
 * whole activation rows in LDS anyway, computes mean and variance there while its first weights are in flight,
 * and no LayerNorm launch, no normalised copy in memory and no second read of it exist; x_norm is then not
 * touched and may be NULL.  Otherwise sq_layernorm writes x_norm [M, K] (fp16, caller-allocated, must not be NULL)
 * and the linear runs on it through the automatic dispatch (workspace as for sq_w4a16_gemm_fused, may be NULL).
 * Inside the kernel the statistics are fp32 (mean first, then the variance around it) and the normalisation
 * runs on fp16 pairs: the deviations are taken around the fp16-rounded mean with the remainder carried exactly,
 * 1 / sigma enters as the sum of two fp16 numbers, gamma and beta are applied in fp16; the normalised row can
 * differ from sq_layernorm's (one rounding from fp32) by an fp16 ulp or two per element.  ln_gamma / ln_beta
 * fp16 [K] or NULL. */
int sq_w4a16_ln_fusable(int M, int N, int K, int group_size, int layout);
int sq_w4a16_gemm_ln_fused(const void* x, const void* ln_gamma, const void* ln_beta, float ln_eps, void* x_norm,
                           const void* w, const void* zs, const void* bias, const void* residual, void* y, int M, int N,
                           int K, int group_size, int layout, int act, void* workspace, size_t workspace_bytes,
                           void* stream);

/* The ends of a greedy decode step around the quantised layers, for the end-to-end configuration (random-init
 * OPT-6.7B, batch 8): what the reference runs as torch modules and ops -- embed_tokens + embed_positions
 * (test/nvidia/module/opt/modeling_opt_ours.py:900-913), the fp16 lm_head (:1097, :1229), the argmax of greedy
 * generation and the bookkeeping between two steps -- as three launches that a HIP graph can hold whole.
 *
 * sq_embed_rows:      out[r, :] = embed[tok[r], :] + pos_table[*pos + pos_offset, :], fp16 [rows, hidden],
 *                     hidden % 8 == 0; tok int64 [rows], pos int64 [1] on the device; indices are clamped to
 *                     [0, vocab) and [0, positions).  The sum is rounded once, as torch's fp16 add.
 * sq_f16_gemv:        y[M, N] = x[M, K] w[N, K]^T, fp16 in and out, fp32 sums; M <= 8, K % 512 == 0, K <= 8192.
 *                     part_val (float) / part_idx (int32), both or neither, [8][sq_f16_gemv_parts(N)]: per token the
 *                     largest stored value and its row for every workgroup of the kernel's fixed grid (two per
 *                     CU; the lowest row among equals).
 * sq_greedy_feedback: tok[m] = the row of the best candidate of token m (lowest row among equals: torch.argmax's
 *                     rule; NaN never wins); if history and step are given and *step < history_rows,
 *                     history[*step, m] = tok[m]; then *pos += 1 and *step += 1 where given (int64 on the device). */
int sq_embed_rows(const void* embed, const void* pos_table, const void* tok, const void* pos, long long pos_offset,
                  void* out, int rows, int hidden, long long vocab, long long positions, void* stream);
int sq_f16_gemv_parts(int N);
int sq_f16_gemv(const void* x, const void* w, void* y, void* part_val, void* part_idx, int M, int N, int K, void* stream);
int sq_greedy_feedback(const void* part_val, const void* part_idx, int parts, int M, void* tok, void* pos, void* history,
                       void* step, long long history_rows, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* SQ_W4A16_H */
