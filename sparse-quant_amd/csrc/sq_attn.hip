// LUT block-sparse attention, prefill (fp16 in/out, fp32 softmax and accumulation).
// For query block i of head h only the key blocks lut[h][i][0..nnz) are visited
// (64 x 64 blocks; a LUT entry equal to its predecessor is padding and is skipped);
// inside a block an optional causal mask and the sequence-length mask apply.
// (replaces _sparse_attention_prefill_fwd_kernel, reference:
// sparse-attention/nvidia/playground/kernels/block_sparse_attention_lut.py:22-172, and
// sparse_attention_prefill_fwd_p, sparse-attention/muxi/playground/kernels/csrc/include/
// block_sparse_attention_lut.cuh:30-236)
//
// Mapping.  A workgroup (4 waves) owns one 64-row query block of one (batch, head);
// wave w owns queries 16w .. 16w+15.  Both products are computed transposed with
// v_mfma_f32_16x16x32_f16 so that a lane always owns ONE query (column l%16):
//   S^T = K Q^T : A = K tile (row = key, from LDS), B = Q^T (registers, pre-scaled by
//                 sm_scale*log2(e) and rounded to fp16 like the reference);
//                 D: lane (query l%16) holds keys 16t + 4*(l/16) + v of key tile t.
//   softmax     : over a lane's 16 values and the 4 lanes {l, l^16, l^32, l^48}; the
//                 reference maximum of a query lives in its lanes and moves lazily (only when
//                 a score exceeds it by more than 2^8), the row sum stays split over the four
//                 lanes until the end: in the common case nothing is exchanged or rescaled.
//   O^T = V^T P^T: B = P^T is exactly what the lane already holds: for the k-step
//                 covering keys 32s .. 32s+31 lane group g supplies keys 32s+4g+{0..3}
//                 and 32s+16+4g+{0..3}; A = V^T rows read from an LDS copy of the V
//                 tile that was transposed while staging (two 64-bit reads);
//                 D: lane (query l%16) holds head-dim rows 16*dt + 4*(l/16) + v.
// K and V tiles are staged once per block for the four waves (global -> registers one
// visited block ahead -> LDS); V is transposed on the way in (each thread packs two
// adjacent keys into 32-bit LDS writes).
#include "sq_common.h"
#include "sq_kernels.h"

namespace sq {

#ifndef SQ_ATTN_KPAD
#define SQ_ATTN_KPAD 16
#endif
#ifndef SQ_ATTN_VPAD
#define SQ_ATTN_VPAD 12
#endif

// QT = 16-query tiles per wave: the workgroup has 4 / QT waves, and every K / V operand read
// from LDS feeds QT matrix instructions.  QT = 2 was measured (3 % slower at D = 64, 30 %
// slower at D = 128, where it needs more than 256 registers); QT = 1 is what is launched.
template <int D, int QT>
__global__ __launch_bounds__(256 / QT) void lut_attn_kernel(const half_t* __restrict__ Q, const half_t* __restrict__ Kp,
                                                            const half_t* __restrict__ V, half_t* __restrict__ O,
                                                            const void* __restrict__ lut, int lut_is_64, int H, int S,
                                                            int nblk_q, int nnz, int nvisit, float qk_scale,
                                                            int causal, int total_wg) {
    constexpr int NT = 256 / QT;                 // threads per workgroup
    constexpr int KP = D + SQ_ATTN_KPAD;         // halves per row of the K tile in LDS
    constexpr int VP = 64 + SQ_ATTN_VPAD;        // halves per row of the transposed V tile in LDS
    constexpr int DK = D / 32;                   // k-steps of S^T
    constexpr int DT = D / 16;                   // row tiles of O^T
    constexpr int KPASS = (64 * D / 8) / NT;     // 16-byte words of the K tile per thread
    constexpr int VPASS = (32 * D / 8) / NT;     // key pairs x 8 head-dim values of the V tile per thread
    __shared__ __attribute__((aligned(16))) half_t ks[64 * KP];
    __shared__ __attribute__((aligned(16))) half_t vt[D * VP];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int lq = lane & 15;
    const int g = lane >> 4;
    // Workgroups are handed to the eight XCDs round-robin by their linear id, and every XCD has its own L2.
    // The id is therefore re-read as (XCD, slot): XCD x works through the x-th eighth of the (head, query block)
    // list, so that all query blocks of a head, which visit the same K and V rows, share one L2
    // instead of pulling those rows into all eight.
    const int per_xcd = (total_wg + 7) >> 3;
    const int work = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if (work >= total_wg) return;
    const int qb = work % nblk_q;
    const int zh = work / nblk_q;
    const int h = zh % H;
    const long base = (long)zh * S * D;
    int m[QT];  // this lane's queries
#pragma unroll
    for (int qt = 0; qt < QT; qt++) m[qt] = qb * 64 + 16 * (QT * wave + qt) + lq;

    // Q^T operands: q * (sm_scale * log2 e), rounded to fp16.
    half8_t qf[QT][DK];
#pragma unroll
    for (int qt = 0; qt < QT; qt++)
#pragma unroll
        for (int s = 0; s < DK; s++) {
            const half8_t raw = *(const half8_t*)(Q + base + (long)imin(m[qt], S - 1) * D + 32 * s + 8 * g);
#pragma unroll
            for (int e = 0; e < 8; e++) qf[qt][s][e] = (half_t)((float)raw[e] * qk_scale);
        }

    float m_i[QT], l_i[QT];
    float4_t acc[QT][DT];
#pragma unroll
    for (int qt = 0; qt < QT; qt++) {
        m_i[qt] = -INFINITY;
        l_i[qt] = 0.f;
#pragma unroll
        for (int dt = 0; dt < DT; dt++) acc[qt][dt] = (float4_t){0.f, 0.f, 0.f, 0.f};
    }

    const long lut_row = ((long)h * nblk_q + qb) * nnz;
    // Tiles travel global -> registers -> LDS; the registers of the next visited block are
    // requested before the current block is consumed, so their latency hides behind it.
    u32x4_t kreg[KPASS];
    half8_t v0reg[VPASS], v1reg[VPASS];
    auto fetch = [&](int n0) {
        // K tile: 64 keys x D halves, 16 bytes per thread per pass.
#pragma unroll
        for (int p = 0; p < KPASS; p++) {
            const int idx = tid + NT * p;
            const int key = idx / (D / 8);
            const int c8 = idx % (D / 8);
            kreg[p] = *(const u32x4_t*)(Kp + base + (long)imin(n0 + key, S - 1) * D + 8 * c8);
        }
        // V tile: a thread takes keys 2kp, 2kp+1 and 8 head-dim values.
#pragma unroll
        for (int p = 0; p < VPASS; p++) {
            const int idx = tid + NT * p;
            const int kp = idx & 31;
            const int c8 = idx >> 5;
            v0reg[p] = *(const half8_t*)(V + base + (long)imin(n0 + 2 * kp, S - 1) * D + 8 * c8);
            v1reg[p] = *(const half8_t*)(V + base + (long)imin(n0 + 2 * kp + 1, S - 1) * D + 8 * c8);
        }
    };
    auto stash = [&]() {
#pragma unroll
        for (int p = 0; p < KPASS; p++) {
            const int idx = tid + NT * p;
            const int key = idx / (D / 8);
            const int c8 = idx % (D / 8);
            *(u32x4_t*)(&ks[key * KP + 8 * c8]) = kreg[p];
        }
        // V transposed: 8 packed pairs vt[d][2kp .. 2kp+1] per pass.
#pragma unroll
        for (int p = 0; p < VPASS; p++) {
            const int idx = tid + NT * p;
            const int kp = idx & 31;
            const int c8 = idx >> 5;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const half2_t pr = {v0reg[p][e], v1reg[p][e]};
                *(half2_t*)(&vt[(8 * c8 + e) * VP + 2 * kp]) = pr;
            }
        }
    };
    // Next visited block (first key index) or -1; a LUT entry equal to its predecessor is
    // padding.  Uniform over the workgroup.
    int jn = 0, last = -1;
    auto advance = [&]() {
        while (jn < nvisit) {
            const int blk = lut_is_64 ? (int)((const long long*)lut)[lut_row + jn] : ((const int*)lut)[lut_row + jn];
            jn++;
            const bool skip = (blk == last) || blk < 0 || (long)blk * 64 >= S;
            last = blk;
            if (!skip) return blk * 64;
        }
        return -1;
    };

    int n0 = advance();
    if (n0 >= 0) fetch(n0);
    while (n0 >= 0) {
        __syncthreads();  // the previous tiles are no longer read
        stash();
        __syncthreads();
        const int n1 = advance();
        if (n1 >= 0) fetch(n1);

        // S^T = K Q^T for the four 16-key tiles; a K operand serves all QT query tiles.  The accumulators
        // start at -m_ref of the lane's query, so the matrix core delivers the scores already shifted by
        // the reference maximum and the softmax needs no subtraction.
        float4_t st[QT][4];
#pragma unroll
        for (int t = 0; t < 4; t++) {
#pragma unroll
            for (int qt = 0; qt < QT; qt++) {
                const float c = (m_i[qt] == -INFINITY) ? 0.f : -m_i[qt];
                st[qt][t] = (float4_t){c, c, c, c};
            }
#pragma unroll
            for (int s = 0; s < DK; s++) {
                const half8_t a = *(const half8_t*)(&ks[(16 * t + lq) * KP + 32 * s + 8 * g]);
#pragma unroll
                for (int qt = 0; qt < QT; qt++)
                    st[qt][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, qf[qt][s], st[qt][t], 0, 0, 0);
            }
        }
        // Masks (only where the block touches the end of the sequence or the causal diagonal;
        // the test is uniform over the workgroup).
        const bool need_mask = (n0 + 64 > S) || (causal && n0 + 63 > qb * 64);
        half8_t pk[QT][2];
#pragma unroll
        for (int qt = 0; qt < QT; qt++) {
            if (need_mask) {
#pragma unroll
                for (int t = 0; t < 4; t++)
#pragma unroll
                    for (int v = 0; v < 4; v++) {
                        const int n = n0 + 16 * t + 4 * g + v;
                        const bool keep = (n < S) && (!causal || n <= m[qt]);
                        st[qt][t][v] = keep ? st[qt][t][v] : -INFINITY;
                    }
            }
            // Largest shifted score of this lane.  The reference maximum m_ref of a query moves only when a
            // score exceeds it by more than 2^LAZY (or when it is still unset): until then p = exp2(s - m_ref)
            // stays below 2^LAZY, well inside fp16, the final O = acc / l does not depend on the reference,
            // and neither the accumulators nor the scores need rescaling.  The test is made per lane and
            // voted over the wave; the maximum over a query's four lanes is formed only when it is needed.
            constexpr float LAZY = 8.f;
            float mx = -INFINITY;
#pragma unroll
            for (int t = 0; t < 4; t++)
#pragma unroll
                for (int v = 0; v < 4; v++) mx = fmaxf(mx, st[qt][t][v]);
            const bool unset = (m_i[qt] == -INFINITY);
            if (__builtin_amdgcn_ballot_w64(mx > LAZY || (unset && mx > -INFINITY)) != 0) {
                float mq = fmaxf(mx, __shfl_xor(mx, 16));
                mq = fmaxf(mq, __shfl_xor(mq, 32));
                const bool upd = mq > LAZY || (unset && mq > -INFINITY);
                const float delta = upd ? mq : 0.f;
                // a query without a reference so far has l = 0 and acc = 0: nothing to rescale
                const float alpha = (upd && !unset) ? __builtin_amdgcn_exp2f(-delta) : 1.f;
                m_i[qt] = upd ? (unset ? delta : m_i[qt] + delta) : m_i[qt];
                l_i[qt] *= alpha;
#pragma unroll
                for (int t = 0; t < 4; t++)
#pragma unroll
                    for (int v = 0; v < 4; v++) st[qt][t][v] -= delta;
#pragma unroll
                for (int dt = 0; dt < DT; dt++) acc[qt][dt] *= alpha;
            }
            // p = exp2(shifted score) (bare v_exp_f32: exp2(-inf) = 0 for masked entries), rounded to fp16
            // for the second product like the reference; the lane's share of the row sum is taken from the
            // rounded pairs with one dot instruction per pair and stays in the lane until the end.
            float rs = 0.f;
#pragma unroll
            for (int t = 0; t < 4; t++)
#pragma unroll
                for (int v = 0; v < 4; v += 2) {
                    const half2_t pp = {(half_t)__builtin_amdgcn_exp2f(st[qt][t][v]),
                                        (half_t)__builtin_amdgcn_exp2f(st[qt][t][v + 1])};
                    rs = __builtin_amdgcn_fdot2(pp, (half2_t){(half_t)1.f, (half_t)1.f}, rs, false);
                    pk[qt][t >> 1][4 * (t & 1) + v] = pp.x;
                    pk[qt][t >> 1][4 * (t & 1) + v + 1] = pp.y;
                }
            l_i[qt] += rs;
        }

        // O^T += V^T P^T; a V operand serves all QT query tiles.
#pragma unroll
        for (int dt = 0; dt < DT; dt++) {
#pragma unroll
            for (int s = 0; s < 2; s++) {
                const half_t* vp = &vt[(16 * dt + lq) * VP + 32 * s + 4 * g];
                const u32x2_t lo = *(const u32x2_t*)(vp);
                const u32x2_t hi = *(const u32x2_t*)(vp + 16);
                const u32x4_t a = {lo.x, lo.y, hi.x, hi.y};
#pragma unroll
                for (int qt = 0; qt < QT; qt++)
                    acc[qt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(bit_cast<half8_t>(a), pk[qt][s], acc[qt][dt],
                                                                         0, 0, 0);
            }
        }
        n0 = n1;
    }

    // O[m][16*dt + 4g + v] = acc / l.
#pragma unroll
    for (int qt = 0; qt < QT; qt++) {
        // the row sum of a query is spread over its four lanes
        float l = l_i[qt] + __shfl_xor(l_i[qt], 16);
        l += __shfl_xor(l, 32);
        if (m[qt] < S) {
            // A query row without any visible key has l = 0 and acc = 0: 0 * inf = NaN, which is
            // also what the reference's running sums produce for such a row.
            const float inv = 1.f / l;
#pragma unroll
            for (int dt = 0; dt < DT; dt++) {
                half4_t o;
#pragma unroll
                for (int v = 0; v < 4; v++) o[v] = (half_t)(acc[qt][dt][v] * inv);
                *(half4_t*)(O + base + (long)m[qt] * D + 16 * dt + 4 * g) = o;
            }
        }
    }
}

hipError_t launch_lut_attention(const void* q, const void* k, const void* v, void* o, const void* lut,
                                int lut_elem_bytes, int Z, int H, int S, int D, int nnz, float sm_scale, int causal,
                                hipStream_t st) {
    const int nblk = (S + 63) / 64;
    const int total_wg = nblk * Z * H;
    const dim3 grid(((total_wg + 7) / 8) * 8);
    const float qk_scale = sm_scale * 1.44269504f;
    const int use_nnz = nnz < nblk ? nnz : nblk;  // the reference clamps NNZ to ceil(S / 64) as well
    // (the LUT row pitch stays nnz even when fewer entries are visited)
#define SQ_ATTN_LAUNCH(D_, QT_)                                                                                   \
    hipLaunchKernelGGL((lut_attn_kernel<D_, QT_>), grid, dim3(256 / QT_), 0, st, (const half_t*)q, (const half_t*)k, \
                       (const half_t*)v, (half_t*)o, lut, lut_elem_bytes == 8, H, S, nblk, nnz, use_nnz, qk_scale,   \
                       causal, total_wg)
    if (D == 64)
        SQ_ATTN_LAUNCH(64, 1);
    else
        SQ_ATTN_LAUNCH(128, 1);
#undef SQ_ATTN_LAUNCH
    return hipGetLastError();
}

}  // namespace sq
