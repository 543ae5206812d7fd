// Internal launch interface between the C ABI (sq_api.hip) and the kernel files.
// Every launcher assumes its arguments were validated by the caller, enqueues on
// `st` and returns the hipError_t of the launch.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "sq_common.h"

namespace sq {

// sq_dequant.hip
hipError_t launch_dequant_l1(const void* w, const void* zs, void* out, int N, int K, int g, hipStream_t st);
hipError_t launch_dequant_l2(const void* w, const void* zs, void* out, int N, int K, int g, hipStream_t st);

// sq_repack.hip
hipError_t launch_transpose_merge_zeros_scales(const void* zeros, const void* scales, void* zs, int K, int N,
                                               int g, hipStream_t st);
hipError_t launch_ours_to_awq(const void* src, void* dst, int K, int N, hipStream_t st);
hipError_t launch_awq_to_lmdeploy(const void* src, void* dst, int K, int N, hipStream_t st);
hipError_t launch_l2_to_l1(const void* w_l2, const void* zs_l2, void* w_l1, void* zs_l1, int N, int K, int g,
                           hipStream_t st);
hipError_t launch_2bit_to_4bit(const void* src, void* dst, int N, int K, hipStream_t st);
hipError_t launch_l2_4bit_to_2bit(const void* src, void* dst, int K, int N, hipStream_t st);
hipError_t launch_l2_2bit_to_4bit(const void* src, void* dst, int K, int N, hipStream_t st);

// The *_tuned launchers take a kernel-specific tuning word (0 = built-in heuristic).
// sq_gemv2.hip: M <= 8, streaming formulation.  tune = waves per workgroup (1,2,4,8).
hipError_t launch_gemv2_tuned(const void* x, const void* w, const void* zs, void* y, int M, int N, int K, int g,
                              bool fixup, int tune, Epilogue epi, hipStream_t st);
// sq_gemv_seq.hip: up to SEQ_MAX_LINEARS decode linears (M <= 4) in one persistent launch.
constexpr int SEQ_MAX_LINEARS = 8;
constexpr size_t SEQ_LDS_LIMIT = 156 * 1024;
struct SeqProblem {
    const void* x;
    const void* w;
    const void* zs;
    const void* bias;
    const void* residual;
    void* y;
    int N, K, group_size, act, depends;
};
// sq_gemv2.hip: 2..GEMV_GROUP_MAX independent decode linears with equal K (<= 8192) and group size, M <= 4, as one
// launch of the single-linear GEMV (the grid is the concatenation of their row blocks).  hipErrorInvalidValue
// when the group does not qualify.
constexpr int GEMV_GROUP_MAX = 4;
hipError_t launch_gemv2_group(const SeqProblem* probs, int count, int M, hipStream_t st);
// sq_skinny2.hip: the same for 5 <= M <= 32 (group size 128) with the split-K decode kernel; ws as for
// sq_w4a16_gemm_ws, at least skinny2_group_workspace_bytes().
size_t skinny2_group_workspace_bytes(const SeqProblem* probs, int count, int M);
hipError_t launch_skinny2_group(const SeqProblem* probs, int count, int M, void* ws, size_t ws_bytes, hipStream_t st);
// sq_gemv_seq.hip: up to SEQ_MAX_LINEARS decode linears (M <= 4) in one persistent launch; outputs that later
// linears of the list read travel between workgroups as tagged words in the workspace.
// gemv_seq_workspace_bytes: a control block of 256 bytes ([0] launch number, [1] sticky error word, [2] exit
// counter) + the exchange words; a region of its own, 256-byte aligned, that no other kernel writes.
size_t gemv_seq_workspace_bytes(const SeqProblem* probs, int count, int M);
// 0: launched; 1: the sequence does not fit this kernel (the caller launches the linears one by one);
// 2: the HIP runtime rejected the launch.  The workspace's control block and exchange words are zero before the
// first launch.  spin_limit bounds the polls for another workgroup's output; lim = loads a streaming wave keeps
// in flight (0: default).
int launch_gemv_seq(const SeqProblem* probs, int count, int M, void* workspace, size_t workspace_bytes,
                    unsigned spin_limit, int lim, hipStream_t st);

// sq_skinny.hip: M <= 64.  tune = waves | mode << 8 (mode 1 = exact, 2 = fixup).
hipError_t launch_skinny_tuned(const void* x, const void* w, const void* zs, void* y, int M, int N, int K, int g,
                               int tune, Epilogue epi, hipStream_t st);
// sq_skinny2.hip: 5 <= M <= 32 with a workspace (counters + fp32 partial tiles).
// tune = ksplit (1,2,4,8) | mode << 8 (1 = exact, 2 = fixup).
size_t skinny2_workspace_bytes(int M, int N, int K);
hipError_t launch_skinny2_tuned(const void* x, const void* w, const void* zs, void* y, void* ws, int M, int N, int K,
                                int g, int tune, Epilogue epi, hipStream_t st);
// sq_skinny3.hip: M <= 16, group size 128 or 64, K % 128 == 0: the streaming decode kernel.  ws may be null when
// K <= 4096 (no K split).  tune = rows per workgroup (1: 16, 3: 48, 4: 64) | ksplit << 4, 0 = heuristic.
// hipErrorInvalidValue when the shape does not fit.
// ln (may be null): LayerNorm of the activations inside the kernel (2048 < K <= 4096, at most 8 tokens).
hipError_t launch_skinny3_tuned(const void* x, const void* w, const void* zs, void* y, void* ws, int M, int N, int K,
                                int g, int tune, Epilogue epi, const LnPre* ln, hipStream_t st);
hipError_t launch_skinny3_group(const SeqProblem* probs, int count, int M, void* ws, size_t ws_bytes, hipStream_t st);
// The same kernel family for 17..32 tokens (two token tiles, activations staged in two halves); group size 128 only.
hipError_t launch_skinny3_wide(const void* x, const void* w, const void* zs, void* y, void* ws, int M, int N, int K,
                               Epilogue epi, hipStream_t st);
bool skinny3_wide_applies(int N, int K, bool have_ws);
bool skinny3_wide_shape(int N, int K, bool have_ws, long* workgroups, int* slots_in_use);
hipError_t launch_skinny3_wide_group(const SeqProblem* probs, int count, int M, void* ws, size_t ws_bytes,
                                     hipStream_t st);
// sq_gemm.hip: any M.  tune = 32-row tiles per workgroup (1,2,4) | ksplit << 8; ws may be null.
size_t gemm_workspace_bytes(int M, int N, int K);
hipError_t launch_gemm_tuned(const void* x, const void* w, const void* zs, void* y, void* ws, size_t ws_bytes, int M,
                             int N, int K, int g, int tune, Epilogue epi, hipStream_t st);

// sq_gemm2.hip: software-pipelined 128 x 256 tile variant for M > 64.
hipError_t launch_gemm_pipe(const void* x, const void* w, const void* zs, void* y, int M, int N, int K, int g,
                            int variant, Epilogue epi, hipStream_t st);

// sq_attn.hip: LUT block-sparse attention, prefill.  D in {64, 128}; lut int32 or int64 [H, ceil(S/64), nnz].
hipError_t launch_lut_attention(const void* q, const void* k, const void* v, void* o, const void* lut,
                                int lut_elem_bytes, int Z, int H, int S, int D, int nnz, float sm_scale, int causal,
                                hipStream_t st);

// sq_decode_attn.hip: dense decode attention over an fp16 KV cache (one query row per sequence),
// optionally appending the new key/value row.  Strides in elements.
hipError_t launch_decode_attention(const void* q, const void* k_new, const void* v_new, void* k_cache, void* v_cache,
                                   const void* mask, void* out, int B, int H, int D, int Lmax, long q_bs, long q_hs,
                                   long n_bs, long n_hs, long c_bs, long c_hs, long m_bs, int cache_len,
                                   const long long* cache_len_dev, float sm_scale, void* workspace,
                                   size_t workspace_bytes, hipStream_t st);
constexpr int DECODE_ATTN_MAX_SPLIT = 16;
size_t decode_attention_workspace_bytes(int B, int H, int D);

// sq_lm_head.hip: the ends of a greedy decode step around the W4A16 layers (the end-to-end harness).
// out[r, :] = embed[tok[r], :] + pos_table[*pos + pos_offset, :] (fp16; indices clamped to their tables).
hipError_t launch_embed_rows(const void* embed, const void* pos_table, const void* tok, const void* pos, long long pos_offset,
                             void* out, int rows, int hidden, long long vocab, long long positions, hipStream_t st);
// y[M, N] = x[M, K] w[N, K]^T in fp16 with fp32 sums, M <= 8, K % 512 == 0, K <= 8192; part_val / part_idx (both or
// neither): per token the best value and row of every workgroup, [8][f16_gemv_parts(N)].
int f16_gemv_parts(int N);
hipError_t launch_f16_gemv(const void* x, const void* w, void* y, float* part_val, int* part_idx, int M, int N, int K,
                           hipStream_t st);
// tok[m] = the row of the best candidate of token m (lowest row among equals); history[*step, m] = tok[m] when both
// are given and *step < history_rows; then *pos += 1 and *step += 1 (each where given).
hipError_t launch_greedy_feedback(const float* part_val, const int* part_idx, int parts, int M, void* tok, void* pos,
                                  void* history, void* step, long long history_rows, hipStream_t st);

// sq_layernorm.hip: LayerNorm over the last dimension, fp16 in/out, fp32 statistics; cols % 8 == 0,
// cols <= 16384.
hipError_t launch_layernorm(const void* x, const void* gamma, const void* beta, void* y, int rows, int cols, float eps,
                            hipStream_t st);

}  // namespace sq
