// The ends of a greedy decode step of the end-to-end harness, around the W4A16 layers: the token and position
// embeddings in front, and behind them the fp16 lm_head with the argmax and the feedback of the chosen token.
// The reference runs these as torch ops (test/nvidia/module/opt/modeling_opt_ours.py:900-913 embeddings, 1097 and
// 1229 the fp16 lm_head; generation picks the argmax); as library calls they took 13 launches and 160 us of a 1.85 ms step at
// batch 8 (the fp16 product alone 90 us for 412 MB), here three launches:
//
//   embed_rows      x[b, :] = embed[tok[b], :] + pos_table[*pos + offset, :]                (one launch for four)
//   f16_gemv        logits[M, N] = x[M, K] . W[N, K]^T, fp16 in and out, fp32 sums, M <= 8; the decode GEMV's
//                   mapping (v_mfma_f32_4x4x4_16B_f16: a lane owns one weight row and sixteen of its k) without the
//                   unpacking; beside the logits every workgroup leaves the maximum of its rows per token
//   greedy_feedback the maxima of the workgroups -> the argmax per token (the first index among equals, as torch
//                   defines it), written where the next step reads its token, appended to a history, and the
//                   position and step counters advanced -- the five small launches between two steps in one.
#include "sq_common.h"
#include "sq_kernels.h"

namespace sq {

namespace {

constexpr int LMH_WAVES = 8;
constexpr int LMH_S = 8;                 // 128-wide k-steps a wave has in flight

__global__ __launch_bounds__(256) void embed_rows_kernel(const half_t* __restrict__ embed, const half_t* __restrict__ pos_table,
                                                         const long long* __restrict__ tok, const long long* __restrict__ pos,
                                                         long long pos_offset, half_t* __restrict__ out, int hidden, long long vocab,
                                                         long long positions) {
    const int b = blockIdx.x;
    long long t = tok[b];
    t = t < 0 ? 0 : (t >= vocab ? vocab - 1 : t);
    long long p = *pos + pos_offset;
    p = p < 0 ? 0 : (p >= positions ? positions - 1 : p);
    const half_t* e = embed + t * hidden;
    const half_t* q = pos_table + p * hidden;
    for (int c = threadIdx.x * 8; c < hidden; c += 256 * 8) {
        const half8_t a = *(const half8_t*)(e + c), d = *(const half8_t*)(q + c);
        half8_t o;
#pragma unroll
        for (int i = 0; i < 8; i++) o[i] = (half_t)((float)a[i] + (float)d[i]);
        *(half8_t*)(out + (long)b * hidden + c) = o;
    }
}

// MT token tiles of four.  A fixed grid of workgroups (two per CU where the activations leave room) stages the
// activations once -- LDS [k-step][token][128 k]: the 64 lanes of an operand read fall on 64 different 16-byte
// slots -- and then walks over the weight in rounds: eight waves = two groups of four rows x the four quarters of
// K, group q of round t being rows 4 (wg + G (2 t + q)) .. + 3.  Many short workgroups would each have to stage the
// activations again (64 KiB at 8 tokens against the 32 KiB of weights of four rows), few long ones leave the last
// round of the grid a third empty; this way every CU streams the same number of row groups to within one.  The
// quarter sums wait in LDS until the end: one barrier for the whole walk.
template <int MT>
__global__ __launch_bounds__(64 * LMH_WAVES) void f16_gemv_kernel(const half_t* __restrict__ W, const half_t* __restrict__ X,
                                                                 half_t* __restrict__ Y, float* __restrict__ part_val,
                                                                 int* __restrict__ part_idx, int M, int N, int K, int iters) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lmh_lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int i = lane & 3, b = lane >> 2;
    const int sel = wave >> 2, part = wave & 3;
    const int G = gridDim.x;
    const int steps = K >> 9;  // 128-wide k-steps of a quarter of K
    const int xbytes = (K >> 7) * (4 * MT) * 256;
    const int cbytes = (4 * MT) * iters * 8 * 4;
    float* red = (float*)(lmh_lds + (xbytes > cbytes ? xbytes : cbytes));  // [iters][2 groups][4 quarters][4 MT tokens][4 rows]

    auto rows_of = [&](int it) { return 4 * (blockIdx.x + G * (2 * it + sel)); };
    auto request = [&](u32x4_t (&w)[LMH_S], int it, int rnd) {
        const int row = imin(rows_of(it) + i, N - 1);
        const half_t* wrow = W + (long)row * K + part * (K >> 2) + 8 * b;
#pragma unroll
        for (int s = 0; s < LMH_S; s++)
            w[s] = __builtin_nontemporal_load((const u32x4_t*)(wrow + (long)imin(rnd * LMH_S + s, steps - 1) * 128));
    };
    const int rounds = (steps + LMH_S - 1) / LMH_S;  // per row group
    const int total = iters * rounds;
    u32x4_t wq[2][LMH_S];
    request(wq[0], 0, 0);  // ahead of the activations
    // activations -> LDS (tokens past M: zeros)
    const int vec_per_row = K >> 3;
    for (int v = tid; v < 4 * MT * vec_per_row; v += 64 * LMH_WAVES) {
        const int m = v / vec_per_row, c = v - m * vec_per_row;
        u32x4_t x = {0u, 0u, 0u, 0u};
        if (m < M) x = *(const u32x4_t*)(X + (long)m * K + 8 * c);
        *(u32x4_t*)(lmh_lds + (c >> 4) * (4 * MT * 256) + m * 256 + (c & 15) * 16) = x;
    }
    __syncthreads();

    float4_t acc[MT];
    auto consume = [&](const u32x4_t (&w)[LMH_S], int it, int rnd) {
        if (rnd == 0) {
#pragma unroll
            for (int mt = 0; mt < MT; mt++) acc[mt] = (float4_t){0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int s = 0; s < LMH_S; s++) {
            const int st = rnd * LMH_S + s;
            half8_t wv = bit_cast<half8_t>(w[s]);
            if (st >= steps) wv = (half8_t){0, 0, 0, 0, 0, 0, 0, 0};  // a step past the quarter re-read its last one
            const int kstep = part * steps + imin(st, steps - 1);
#pragma unroll
            for (int mt = 0; mt < MT; mt++) {
                const half8_t xa = *(const half8_t*)(lmh_lds + kstep * (4 * MT * 256) + (4 * mt + i) * 256 + 16 * b);
                acc[mt] = __builtin_amdgcn_mfma_f32_4x4x4f16(xa.lo, wv.lo, acc[mt], 0, 0, 0);
                acc[mt] = __builtin_amdgcn_mfma_f32_4x4x4f16(xa.hi, wv.hi, acc[mt], 0, 0, 0);
            }
        }
        if (rnd == rounds - 1) {
            // fold the sixteen k blocks of a row; lanes 0..3 hold rows 0..3 of the group
#pragma unroll
            for (int mt = 0; mt < MT; mt++)
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    float v = row_sum_stride4(acc[mt][j]);
                    v += __shfl_xor(v, 16);
                    v += __shfl_xor(v, 32);
                    if (lane < 4) red[(((it * 2 + sel) * 4 + part) * (4 * MT) + 4 * mt + j) * 4 + i] = v;
                }
        }
    };
    // two register sets take turns; the request past the last round re-reads and is not consumed
    for (int u = 0; u < total; u += 2) {
        request(wq[1], (u + 1) / rounds, (u + 1) % rounds);
        consume(wq[0], u / rounds, u % rounds);
        if (u + 1 < total) {
            request(wq[0], (u + 2) / rounds, (u + 2) % rounds);
            consume(wq[1], (u + 1) / rounds, (u + 1) % rounds);
        }
    }
    __syncthreads();

    // the four quarters of every output; the candidates of the workgroup per token
    float* cval = (float*)lmh_lds;  // [4 MT][iters * 8] stored values of the workgroup's rows, where the activations were
    const int nout = iters * 2 * (4 * MT) * 4;
    for (int o = tid; o < nout; o += 64 * LMH_WAVES) {
        const int r = o & 3, m = (o >> 2) % (4 * MT), grp = o / (16 * MT);  // grp = it * 2 + sel
        float v = 0.f;
#pragma unroll
        for (int q = 0; q < 4; q++) v += red[((grp * 4 + q) * (4 * MT) + m) * 4 + r];
        const int row = 4 * (blockIdx.x + G * grp) + r;
        const half_t h = (half_t)v;
        const bool ok = row < N && m < M;
        if (ok) Y[(long)m * N + row] = h;
        if (part_val) cval[m * (iters * 8) + grp * 4 + r] = ok ? (float)h : -INFINITY;
    }
    if (part_val) {
        __syncthreads();
        if (wave < 4 * MT && wave < M) {
            // wave m: the best of token m's values, lowest row among equals
            float best = -INFINITY;
            int arg = 0x7fffffff;
            for (int c = lane; c < iters * 8; c += 64) {
                const float v = cval[wave * (iters * 8) + c];
                const int row = 4 * (blockIdx.x + G * (c >> 2)) + (c & 3);
                if (v > best || (v == best && row < arg)) best = v, arg = row;
            }
#pragma unroll
            for (int o = 1; o < 64; o <<= 1) {
                const float ob = __shfl_xor(best, o);
                const int oa = __shfl_xor(arg, o);
                if (ob > best || (ob == best && oa < arg)) best = ob, arg = oa;
            }
            if (lane == 0) {
                part_val[(long)wave * G + blockIdx.x] = best;
                part_idx[(long)wave * G + blockIdx.x] = arg;
            }
        }
    }
}

// One workgroup: wave m finds the best of token m's `parts` candidates; then the feedback writes.
__global__ __launch_bounds__(512) void greedy_feedback_kernel(const float* __restrict__ part_val, const int* __restrict__ part_idx,
                                                              int parts, int M, long long* __restrict__ tok,
                                                              long long* __restrict__ pos, long long* __restrict__ history,
                                                              long long* __restrict__ step, long long history_rows) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (wave < M) {
        float best = -INFINITY;
        int arg = 0x7fffffff;
        for (int p = lane; p < parts; p += 64) {
            const float v = part_val[(long)wave * parts + p];
            const int a = part_idx[(long)wave * parts + p];
            if (v > best || (v == best && a < arg)) best = v, arg = a;
        }
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const float ob = __shfl_xor(best, o);
            const int oa = __shfl_xor(arg, o);
            if (ob > best || (ob == best && oa < arg)) best = ob, arg = oa;
        }
        if (lane == 0) {
            if (arg == 0x7fffffff) arg = 0;  // a row without a finite candidate
            tok[wave] = arg;
            if (history && step) {
                const long long s = *step;
                if (s >= 0 && s < history_rows) history[s * M + wave] = arg;
            }
        }
    }
    __syncthreads();  // every wave has read *step before it moves
    if (tid == 0) {
        if (pos) *pos += 1;
        if (step) *step += 1;
    }
}

}  // namespace

hipError_t launch_embed_rows(const void* embed, const void* pos_table, const void* tok, const void* pos, long long pos_offset,
                             void* out, int rows, int hidden, long long vocab, long long positions, hipStream_t st) {
    hipLaunchKernelGGL(embed_rows_kernel, dim3(rows), dim3(256), 0, st, (const half_t*)embed, (const half_t*)pos_table,
                       (const long long*)tok, (const long long*)pos, pos_offset, (half_t*)out, hidden, vocab, positions);
    return hipGetLastError();
}

// Workgroups of the fixed grid (= candidates per token): two per CU of the device, fewer for a weight that has
// fewer groups of eight rows.
int f16_gemv_parts(int N) {
    static int cus[64] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
    if (cus[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cus[dev] = n;
    }
    const int pairs = ((N + 3) / 4 + 1) / 2;
    const int g = 2 * cus[dev];
    return pairs < g ? pairs : g;
}

// M <= 8, K % 512 == 0, K <= 8192.  part_val / part_idx: null, or [8][f16_gemv_parts(N)] each.
hipError_t launch_f16_gemv(const void* x, const void* w, void* y, float* part_val, int* part_idx, int M, int N, int K,
                           hipStream_t st) {
    if (M < 1 || M > 8 || K < 512 || K % 512 != 0 || K > 8192 || N < 1) return hipErrorInvalidValue;
    const int G = f16_gemv_parts(N);
    if (G <= 0) return hipErrorInvalidDevice;
    const int quads = (N + 3) / 4;
    const int iters = (quads + 2 * G - 1) / (2 * G);
    const int mt4 = M <= 4 ? 4 : 8;
    // activations + quarter sums (two workgroups per CU fit while this stays under 80 KiB: 77 KiB for the
    // OPT-6.7B lm_head at 8 tokens)
    const int xb = (K >> 7) * mt4 * 256, cb = mt4 * iters * 8 * 4;  // the stored values reuse the activations' space
    const int lds = (xb > cb ? xb : cb) + iters * 2 * 4 * mt4 * 4 * 4;
    if (lds > 160 * 1024) return hipErrorInvalidValue;
    static bool allowed[2][64] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return hipErrorInvalidDevice;
    if (M <= 4) {
        if (lds > 64 * 1024 && !allowed[0][dev]) {
            const hipError_t e = hipFuncSetAttribute((const void*)f16_gemv_kernel<1>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            if (e != hipSuccess) return e;
            allowed[0][dev] = true;
        }
        hipLaunchKernelGGL((f16_gemv_kernel<1>), dim3(G), dim3(64 * LMH_WAVES), lds, st, (const half_t*)w, (const half_t*)x,
                           (half_t*)y, part_val, part_idx, M, N, K, iters);
    } else {
        if (lds > 64 * 1024 && !allowed[1][dev]) {
            const hipError_t e = hipFuncSetAttribute((const void*)f16_gemv_kernel<2>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            if (e != hipSuccess) return e;
            allowed[1][dev] = true;
        }
        hipLaunchKernelGGL((f16_gemv_kernel<2>), dim3(G), dim3(64 * LMH_WAVES), lds, st, (const half_t*)w, (const half_t*)x,
                           (half_t*)y, part_val, part_idx, M, N, K, iters);
    }
    return hipGetLastError();
}

hipError_t launch_greedy_feedback(const float* part_val, const int* part_idx, int parts, int M, void* tok, void* pos,
                                  void* history, void* step, long long history_rows, hipStream_t st) {
    if (M < 1 || M > 8 || parts < 1) return hipErrorInvalidValue;
    hipLaunchKernelGGL(greedy_feedback_kernel, dim3(1), dim3(512), 0, st, part_val, part_idx, parts, M, (long long*)tok,
                       (long long*)pos, (long long*)history, (long long*)step, history_rows);
    return hipGetLastError();
}

}  // namespace sq
