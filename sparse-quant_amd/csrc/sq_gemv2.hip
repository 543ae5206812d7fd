// Decode GEMV / very skinny GEMM (M <= 8) for layout L1, streaming formulation.
// HBM-bandwidth bound: algorithmic bytes = N*K/2 + (K/g)*N*4 + M*K*2 + M*N*2.
//
// Mapping.  v_mfma_f32_4x4x4_16B_f16 multiplies 16 independent 4x4x4 blocks; in
// block b lane 4b+i supplies row i of A (4 k) and column i of B (4 k) and receives
// D[0..3][i].  With A = activations (row = token) and B = weights (column = output
// row) every lane accumulates its own output row over its own k for up to 4
// tokens, and the matrix core does every multiply-add; the VALU only unpacks.
//
// A workgroup is NR x KS waves: wave (r, q) owns the 4 output rows r0 + 4r .. +3
// and the q-th of KS contiguous ranges of 512-wide k-steps.  In k-step s lane
// 4b+i loads the 128-bit word with k = 512*s + 32*b .. +31 of its row, so one
// wave-wide load covers 4 rows x 256 contiguous bytes, and all (up to S) loads of
// a round are issued back to back before anything is consumed.  The activations
// of the round (and, for the fixup mode, their sums over each run of 32 k) are
// staged once per workgroup in LDS with row pitch 1 KiB * S + 16 bytes, which
// puts the 64 lanes of a 128-bit read on 64 distinct 16-byte slots.  A lane's sum
// over its 16 blocks is folded with DPP row rotations and two cross-row shuffles;
// the KS partial sums of a row meet in LDS once, at the end.
//
// Arithmetic modes (both accumulate in fp32):
//   exact : B = fp16((q - z) * s), bit-identical to the reference's W_hat.
//   fixup : B = bias + q (bit pattern only); per run of 32 k the lane adds
//           s * (sum x*(bias+q) - sum x*bias - z * sum x): zero and scale are applied once
//           per run in fp32 instead of once per weight in fp16.  Up to 4 tokens: the unpack
//           without shifts (bias 1024 on four of every eight positions, 64 on the others,
//           5 operations per word instead of 7); the bias terms come from two sums staged
//           beside the activations or, with more than 4 tokens, from a second matrix
//           instruction whose B operand is -(bias + z).
// (replaces w4a16_bs1_kernel / w4a16_bs2_kernel, reference:
// quantization/muxi/backend/w4a16_gemm.cuh:14-151,153-326)
#include "sq_common.h"
#include "sq_kernels.h"

namespace sq {

template <int MROWS, int NR, int KS, int S, bool FIXUP>
struct Gemv2Lds {
    static constexpr int PITCH = 1024 * S + 16;
    static constexpr bool SUMS = FIXUP && MROWS <= 4;
    static constexpr int XSUM_OFF = KS * MROWS * PITCH;
    static constexpr int RED_OFF = XSUM_OFF + (SUMS ? KS * S * 16 * MROWS * 2 * 4 : 0);
    static constexpr int BYTES = RED_OFF + KS * NR * MROWS * 4 * 4;
};

// Launch with Gemv2Lds::BYTES of dynamic LDS; instantiations beyond 64 KiB need the attribute first.
template <typename Kern>
static hipError_t gemv2_allow_lds(Kern kern, int bytes, bool* done) {
    if (bytes <= 64 * 1024) return hipSuccess;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return hipErrorInvalidDevice;
    if (!done[dev]) {
        const hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
        if (e != hipSuccess) return e;
        done[dev] = true;
    }
    return hipSuccess;
}

template <int MROWS, int NR, int KS, int S, bool FIXUP>
__device__ __forceinline__ void gemv2_body(const uint8_t* __restrict__ W, const half2_t* __restrict__ ZS,
                                           const half_t* __restrict__ X, half_t* __restrict__ Y, int M, int N, int K,
                                           int gshift, const Epilogue& epi, int blk) {
    constexpr int MT = (MROWS + 3) / 4;
    // Fixup mode, where the zero point is applied: with up to 4 tokens through per-run activation
    // sums staged beside the activations; with more, where that vector arithmetic starts to
    // bound the kernel, by a second matrix instruction with B = -(64 + z).
    constexpr bool ZMFMA = MROWS > 4;
    constexpr int PITCH = 1024 * S + 16;                 // bytes per staged activation row
    constexpr int NT = 64 * NR * KS;
    constexpr int STAGE_TOTAL = KS * MROWS * S * 64;     // 128-bit words staged per round
    constexpr int STAGE_PER_THREAD = (STAGE_TOTAL + NT - 1) / NT;

    // Dynamic LDS (Gemv2Lds gives the layout to the launcher): staged activations; per run of 32 k and token
    // {sum of x, 960 * sum of x over the positions unpacked with bias 1024} (only where the zero point is
    // applied through them); the partial sums of the k ranges.
    using Lds = Gemv2Lds<MROWS, NR, KS, S, FIXUP>;
    extern __shared__ __attribute__((aligned(16))) uint8_t gemv2_lds[];
    uint8_t(*xbuf)[MROWS * PITCH] = reinterpret_cast<uint8_t(*)[MROWS * PITCH]>(gemv2_lds);
    float(*xsum)[S * 16][MROWS][2] = reinterpret_cast<float(*)[S * 16][MROWS][2]>(gemv2_lds + Lds::XSUM_OFF);
    float(*red)[NR][MROWS][4] = reinterpret_cast<float(*)[NR][MROWS][4]>(gemv2_lds + Lds::RED_OFF);

    const NibbleMasks nm = nibble_masks();
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wr = wave % NR;   // row group of this wave
    const int wq_ = wave / NR;  // k range of this wave
    const int i = lane & 3;
    const int b = lane >> 2;
    const int out_row = blk * (4 * NR) + 4 * wr + i;
    const int row = imin(out_row, N - 1);
    const int groups = K >> gshift;
    const int nsteps = (K + 511) >> 9;
    const int spw = (nsteps + KS - 1) / KS;  // k-steps per wave
    const int rounds = (spw + S - 1) / S;
    const uint8_t* wrow = W + (long)row * (K >> 1);
    const half2_t* zrow = ZS + (long)row * groups;

    float4_t acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; mt++) acc[mt] = (float4_t){0.f, 0.f, 0.f, 0.f};

    for (int rnd = 0; rnd < rounds; rnd++) {
        // Stage the activations of this round for all KS ranges: word idx covers
        // range q = idx / (MROWS*S*64), token m, k-step j = (idx / 64) % S.
        u32x4_t xr[STAGE_PER_THREAD];
#pragma unroll
        for (int p = 0; p < STAGE_PER_THREAD; p++) {
            const int idx = tid + p * NT;
            const int q = idx / (MROWS * S * 64);
            const int m = (idx / (S * 64)) % MROWS;
            const int w8 = idx % (S * 64);  // 128-bit word inside the staged row
            const int j = rnd * S + (w8 >> 6);
            const int k = (q * spw + j) * 512 + (w8 & 63) * 8;
            const bool ok = (idx < STAGE_TOTAL) && (m < M) && (j < spw) && (k < K);
            const u32x4_t v = *(const u32x4_t*)(X + (ok ? (long)m * K + k : 0));
            xr[p] = ok ? v : (u32x4_t){0u, 0u, 0u, 0u};
        }
        // The weight stream of this round; a k-step outside the wave's range or
        // past K reads a valid address and meets zero activations (the host picks S and
        // KS so that this is rare).
        u32x4_t wq[S];
        half2_t zq[S];
#pragma unroll
        for (int s = 0; s < S; s++) {
            const int j = rnd * S + s;
            const int kk = (wq_ * spw + j) * 512 + 32 * b;
            const int kc = (j < spw && kk < K) ? kk : 0;
            wq[s] = __builtin_nontemporal_load((const u32x4_t*)(wrow + (kc >> 1)));
            zq[s] = zrow[kc >> gshift];
        }
        if (rnd > 0) __syncthreads();  // everyone is done reading the previous round
#pragma unroll
        for (int p = 0; p < STAGE_PER_THREAD; p++) {
            const int idx = tid + p * NT;
            const int q = idx / (MROWS * S * 64);
            const int m = (idx / (S * 64)) % MROWS;
            const int w8 = idx % (S * 64);
            if (idx < STAGE_TOTAL) *(u32x4_t*)(&xbuf[q][m * PITCH + w8 * 16]) = xr[p];
            if (FIXUP && !ZMFMA) {
                const half8_t h = bit_cast<half8_t>(xr[p]);
                float lo = ((float)h[0] + (float)h[1]) + ((float)h[4] + (float)h[5]);
                float sum = lo + (((float)h[2] + (float)h[3]) + ((float)h[6] + (float)h[7]));
                sum = quad_sum(sum);
                lo = quad_sum(lo);
                if ((tid & 3) == 0 && idx < STAGE_TOTAL) {
                    xsum[q][w8 >> 2][m][0] = sum;
                    xsum[q][w8 >> 2][m][1] = 960.f * lo;
                }
            }
        }
        __syncthreads();

#pragma unroll
        for (int s = 0; s < S; s++) {
            half8_t xa[MT][4];
#pragma unroll
            for (int mt = 0; mt < MT; mt++) {
                const int m = (4 * mt + i) & (MROWS - 1);
                const uint8_t* xp = &xbuf[wq_][m * PITCH + (512 * s + 32 * b) * 2];
#pragma unroll
                for (int t = 0; t < 4; t++) xa[mt][t] = *(const half8_t*)(xp + 16 * t);
            }
            const half2_t p = zq[s];
            if (!FIXUP) {
                const half2_t z64 = {p.x, p.x};
                const half2_t sc = {p.y, p.y};
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    const half8_t wv = dequant8(wq[s][t], z64, sc, nm);
#pragma unroll
                    for (int mt = 0; mt < MT; mt++) {
                        acc[mt] = __builtin_amdgcn_mfma_f32_4x4x4f16(xa[mt][t].lo, wv.lo, acc[mt], 0, 0, 0);
                        acc[mt] = __builtin_amdgcn_mfma_f32_4x4x4f16(xa[mt][t].hi, wv.hi, acc[mt], 0, 0, 0);
                    }
                }
            } else {
                // Two accumulators per token tile (words 0, 1 and words 2, 3): with one wave per SIMD a single
                // chain of dependent matrix instructions would leave their latency exposed.
                float4_t tmp[MT], tmp2[MT];
#pragma unroll
                for (int mt = 0; mt < MT; mt++) tmp[mt] = tmp2[mt] = (float4_t){0.f, 0.f, 0.f, 0.f};
                // zero-point operand for the mixed-bias unpack: -(1024 + z) where the weight carries
                // bias 1024 (positions 0, 1 of each four), -(64 + z) elsewhere; both exact in fp16
                const half_t nz = -p.x;
                const half_t nz1024 = nz - (half_t)960.f;
                const half4_t nzb = {nz1024, nz1024, nz, nz};
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    const half8_t wv = unpack8_mixed(wq[s][t], nm);
#pragma unroll
                    for (int mt = 0; mt < MT; mt++) {
                        float4_t& tq = (t < 2) ? tmp[mt] : tmp2[mt];
                        tq = __builtin_amdgcn_mfma_f32_4x4x4f16(xa[mt][t].lo, wv.lo, tq, 0, 0, 0);
                        tq = __builtin_amdgcn_mfma_f32_4x4x4f16(xa[mt][t].hi, wv.hi, tq, 0, 0, 0);
                        if (ZMFMA) {
                            tq = __builtin_amdgcn_mfma_f32_4x4x4f16(xa[mt][t].lo, nzb, tq, 0, 0, 0);
                            tq = __builtin_amdgcn_mfma_f32_4x4x4f16(xa[mt][t].hi, nzb, tq, 0, 0, 0);
                        }
                    }
                }
#pragma unroll
                for (int mt = 0; mt < MT; mt++) tmp[mt] += tmp2[mt];
                const float zf = (float)p.x;
                const float sf = (float)p.y;
                const float* xs = &xsum[wq_][16 * s + b][0][0];
#pragma unroll
                for (int mt = 0; mt < MT; mt++)
#pragma unroll
                    for (int j = 0; j < 4; j++)
                        if (4 * mt + j < MROWS)
                            acc[mt][j] += ZMFMA ? sf * tmp[mt][j]
                                                : sf * ((tmp[mt][j] - xs[2 * (4 * mt + j) + 1]) - zf * xs[2 * (4 * mt + j)]);
            }
        }
    }

    // Fold the 16 blocks of the wave: DPP inside each 16-lane row, shuffles across
    // rows; then the KS ranges of a row through LDS.
#pragma unroll
    for (int m = 0; m < MROWS; m++) {
        float v = row_sum_stride4(acc[m >> 2][m & 3]);
        v += __shfl_xor(v, 16);
        v += __shfl_xor(v, 32);
        if (KS == 1) {
            if (lane < 4 && out_row < N && m < M) Y[(long)m * N + out_row] = epilogue(v, m, out_row, N, epi);
        } else if (lane < 4) {
            red[wq_][wr][m][i] = v;
        }
    }
    if (KS > 1) {
        __syncthreads();
        if (tid < NR * MROWS * 4) {
            const int ri = tid & 3;
            const int m = (tid >> 2) % MROWS;
            const int r = (tid >> 2) / MROWS;
            float sum = 0.f;
#pragma unroll
            for (int q = 0; q < KS; q++) sum += red[q][r][m][ri];
            const int orow = blk * (4 * NR) + 4 * r + ri;
            if (orow < N && m < M) Y[(long)m * N + orow] = epilogue(sum, m, orow, N, epi);
        }
    }
}

template <int MROWS, int NR, int KS, int S, bool FIXUP>
__global__ __launch_bounds__(64 * NR * KS) void gemv2_kernel(const uint8_t* __restrict__ W,
                                                             const half2_t* __restrict__ ZS,
                                                             const half_t* __restrict__ X,
                                                             half_t* __restrict__ Y, int M, int N, int K,
                                                             int gshift, Epilogue epi) {
    gemv2_body<MROWS, NR, KS, S, FIXUP>(W, ZS, X, Y, M, N, K, gshift, epi, blockIdx.x);
}

// Up to four linears that do not depend on each other and share M, K and the group size (q, k and v of a
// decoder layer) in one launch: the grid is the concatenation of their row blocks, a workgroup looks its
// linear up by its block index and then runs the single-linear body unchanged.
struct Gemv2Group {
    const uint8_t* W[GEMV_GROUP_MAX];
    const half2_t* ZS[GEMV_GROUP_MAX];
    const half_t* X[GEMV_GROUP_MAX];
    half_t* Y[GEMV_GROUP_MAX];
    const half_t* bias[GEMV_GROUP_MAX];
    const half_t* residual[GEMV_GROUP_MAX];
    int N[GEMV_GROUP_MAX];
    int act[GEMV_GROUP_MAX];
    int blk_end[GEMV_GROUP_MAX];  // first block index behind linear p
    int count;
};

template <int MROWS, int NR, int KS, int S, bool FIXUP>
__global__ __launch_bounds__(64 * NR * KS) void gemv2_group_kernel(const Gemv2Group grp, int M, int K, int gshift) {
    int p = 0;
#pragma unroll
    for (int q = 0; q < GEMV_GROUP_MAX - 1; q++)
        if (q + 1 < grp.count && (int)blockIdx.x >= grp.blk_end[q]) p = q + 1;
    const int blk = blockIdx.x - (p > 0 ? grp.blk_end[p - 1] : 0);
    const Epilogue epi{grp.bias[p], grp.residual[p], grp.act[p]};
    gemv2_body<MROWS, NR, KS, S, FIXUP>(grp.W[p], grp.ZS[p], grp.X[p], grp.Y[p], M, grp.N[p], K, gshift, epi, blk);
}

template <int MROWS, int NR, int KS, int S>
static hipError_t launch_group_cfg(const SeqProblem* probs, int count, int M, int K, int gshift, hipStream_t st) {
    Gemv2Group g;
    int blocks = 0;
    for (int p = 0; p < GEMV_GROUP_MAX; p++) {
        const SeqProblem& q = probs[p < count ? p : 0];
        g.W[p] = (const uint8_t*)q.w;
        g.ZS[p] = (const half2_t*)q.zs;
        g.X[p] = (const half_t*)q.x;
        g.Y[p] = (half_t*)q.y;
        g.bias[p] = (const half_t*)q.bias;
        g.residual[p] = (const half_t*)q.residual;
        g.N[p] = q.N;
        g.act[p] = q.act;
        if (p < count) blocks += (q.N + 4 * NR - 1) / (4 * NR);
        g.blk_end[p] = blocks;
    }
    g.count = count;
    constexpr int lds = Gemv2Lds<MROWS, NR, KS, S, true>::BYTES;
    static bool allowed[64] = {};
    const hipError_t e = gemv2_allow_lds(gemv2_group_kernel<MROWS, NR, KS, S, true>, lds, allowed);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((gemv2_group_kernel<MROWS, NR, KS, S, true>), dim3(blocks), dim3(64 * NR * KS), lds, st, g, M, K,
                       gshift);
    return hipGetLastError();
}

template <int MROWS, int NR, int KS, int S>
static hipError_t launch_cfg(const void* x, const void* w, const void* zs, void* y, int M, int N, int K, int gshift,
                             bool fixup, Epilogue epi, hipStream_t st) {
    const dim3 grid((N + 4 * NR - 1) / (4 * NR));
    static bool allowed[2][64] = {};
    if (fixup) {
        constexpr int lds = Gemv2Lds<MROWS, NR, KS, S, true>::BYTES;
        const hipError_t e = gemv2_allow_lds(gemv2_kernel<MROWS, NR, KS, S, true>, lds, allowed[1]);
        if (e != hipSuccess) return e;
        hipLaunchKernelGGL((gemv2_kernel<MROWS, NR, KS, S, true>), grid, dim3(64 * NR * KS), lds, st, (const uint8_t*)w,
                           (const half2_t*)zs, (const half_t*)x, (half_t*)y, M, N, K, gshift, epi);
    } else {
        constexpr int lds = Gemv2Lds<MROWS, NR, KS, S, false>::BYTES;
        const hipError_t e = gemv2_allow_lds(gemv2_kernel<MROWS, NR, KS, S, false>, lds, allowed[0]);
        if (e != hipSuccess) return e;
        hipLaunchKernelGGL((gemv2_kernel<MROWS, NR, KS, S, false>), grid, dim3(64 * NR * KS), lds, st,
                           (const uint8_t*)w, (const half2_t*)zs, (const half_t*)x, (half_t*)y, M, N, K, gshift, epi);
    }
    return hipGetLastError();
}

// Staged activations are kept under 48 KiB of LDS: KS * MROWS * S KiB (eight tokens with all eight k-steps of
// K = 4096 in one round, 64 KiB, were measured: 6.7 us against 6.5 us in two rounds).
template <int MROWS, int S>
static hipError_t launch_steps(int nr, int ks, const void* x, const void* w, const void* zs, void* y, int M, int N,
                               int K, int gshift, bool fixup, Epilogue epi, hipStream_t st) {
    constexpr int KS_MAX = 48 / (MROWS * S) >= 4 ? 4 : (48 / (MROWS * S) >= 2 ? 2 : 1);
    if (ks > KS_MAX) ks = KS_MAX;
    while (nr * ks > 16) nr >>= 1;
#define SQ_CASE(NR_, KS_)                                                                    \
    if (nr == NR_ && ks == KS_) {                                                           \
        if constexpr (KS_ <= KS_MAX)                                                        \
            return launch_cfg<MROWS, NR_, KS_, S>(x, w, zs, y, M, N, K, gshift, fixup, epi, st); \
    }
    SQ_CASE(2, 1) SQ_CASE(4, 1) SQ_CASE(8, 1)
    SQ_CASE(2, 2) SQ_CASE(4, 2) SQ_CASE(8, 2)
    SQ_CASE(2, 4) SQ_CASE(4, 4)
#undef SQ_CASE
    return launch_cfg<MROWS, 4, 1, S>(x, w, zs, y, M, N, K, gshift, fixup, epi, st);
}

template <int MROWS>
static hipError_t launch_rows(int nr, int ks, int steps, const void* x, const void* w, const void* zs, void* y,
                              int M, int N, int K, int gshift, bool fixup, Epilogue epi, hipStream_t st) {
    constexpr int S_MAX = (MROWS >= 4) ? 4 : 8;
    if (steps >= 8 && S_MAX >= 8) return launch_steps<MROWS, S_MAX>(nr, ks, x, w, zs, y, M, N, K, gshift, fixup, epi, st);
    if (steps >= 4) return launch_steps<MROWS, 4>(nr, ks, x, w, zs, y, M, N, K, gshift, fixup, epi, st);
    return launch_steps<MROWS, 2>(nr, ks, x, w, zs, y, M, N, K, gshift, fixup, epi, st);
}

// tune = 0 for the built-in heuristic, else (row groups per workgroup: 2,4,8) |
// (k ranges per workgroup: 1,2,4) << 4.  A workgroup covers 4 * row groups rows; the
// number of k-steps a wave issues per round (2, 4 or 8) follows from K and the k ranges.
hipError_t launch_gemv2_tuned(const void* x, const void* w, const void* zs, void* y, int M, int N, int K, int g,
                              bool fixup, int tune, Epilogue epi, hipStream_t st) {
    int gshift = 0;
    while ((1 << gshift) < g) gshift++;
    int nr = tune & 0xF, ks = (tune >> 4) & 0xF;
    const int nsteps = (K + 511) / 512;
    // Measured on MI355X (cold weights, M = 1): K = 16384 wants 4 k ranges x 2 row groups,
    // 16384 x 4096 wants 2 x 4, 4096 x 4096 wants 1 x 4.
    // A wave issues its k-steps in rounds of 2, 4 or 8: the k-step slots a split into k_ ranges streams.
    const int smax = M <= 2 ? 8 : 4;
    auto slots = [&](int k_) {
        const int spw_ = (nsteps + k_ - 1) / k_;
        const int s_ = (spw_ >= 8 && smax >= 8) ? 8 : (spw_ >= 4 ? 4 : 2);
        return (spw_ + s_ - 1) / s_ * s_ * k_;
    };
    if (ks != 1 && ks != 2 && ks != 4) {
        // (two ranges from 24 M weights up: 5120 x 5120 at M = 1 7.3 -> 6.7 us; 4096 x 4096 stays at one)
        ks = nsteps > 16 ? 4 : (((long)N * K >= (3L << 23) && nsteps >= 8) ? 2 : 1);
        if (M >= 3 && M <= 4 && ks == 1 && nsteps >= 8) ks = 2;  // 4096 x 4096 with 3..4 tokens: 4.5 vs 5.6 us
        // A K whose steps do not fill the rounds of that choice (11008 = 21.5 steps: 4 ranges x 2 rounds x 4 = 32
        // slots) streams padding.  Take the split that wastes least when the first choice wastes more than an
        // eighth (4096 x 11008 at M = 1: 8.9 -> 7.9 us).
        if (slots(ks) * 8 > nsteps * 9) {
            int best = ks;
            for (int k_ : {4, 2, 1})
                if (slots(k_) < slots(best)) best = k_;
            ks = best;
        }
    }
    if (nr != 2 && nr != 4 && nr != 8) {
        // (one token on a split K >= 8192: two row groups, i.e. twice as many workgroups of half the size -- 8192 x 8192
        // 9.2 -> 8.8 us, 16384 x 8192 16.0 -> 14.7, 28672 x 8192 26.4 -> 23.9; 4096 x 16384 at M = 4 wants four:
        // 12.8 vs 13.7 us)
        nr = ((ks == 4 || (ks == 2 && nsteps >= 16)) && M <= 1) ? 2 : 4;
        // The busiest CU gets ceil(workgroups / 256) workgroups of 4 nr rows each: where halving the workgroup
        // lowers that product, halve it (5120 rows: 320 workgroups of 16 rows are two rounds for a quarter of the
        // CUs; 5120 x 13824 at M = 2: 16.0 -> 12.6 us.  1024 rows: 64 workgroups leave three CUs in four idle).
        auto busiest = [&](int r) { return ((N + 4 * r - 1) / (4 * r) + 255) / 256 * r; };
        // (with 3..4 tokens every workgroup stages that many activation rows, and halving only pays where 16-row
        // workgroups leave CUs without one: 5120 x 5120 at 4 tokens 10.3 -> 8.8 us with four row groups, 6144 x 2048
        // 5.2 -> 4.2; 2048 x 8192 5.8 with two against 6.7)
        if (nr == 4 && busiest(2) < busiest(4) && (M <= 2 || (N + 15) / 16 < 256)) nr = 2;
        // and a weight that gives the chip less than one wave per SIMD splits K further, down to two k-steps
        // per wave (M = 1: 1024 x 8192 5.0 -> 3.4 us, 768 x 3072 3.4 -> 2.8, 2048 x 2048 at 2 tokens 3.05 -> 2.7)
        if (((tune >> 4) & 0xF) == 0)
            while (ks < 4 && (long)((N + 4 * nr - 1) / (4 * nr)) * nr * ks < 1024 && nsteps > 2 * ks &&
                   slots(2 * ks) <= slots(ks))  // (not into padding: 2560 x 10240, 20 k-steps, 8.2 -> 7.3 us unsplit)
                ks *= 2;
    }
    const int spw = (nsteps + ks - 1) / ks;
    if (M <= 1) return launch_rows<1>(nr, ks, spw, x, w, zs, y, M, N, K, gshift, fixup, epi, st);
    if (M <= 2) return launch_rows<2>(nr, ks, spw, x, w, zs, y, M, N, K, gshift, fixup, epi, st);
    if (M <= 4) return launch_rows<4>(nr, ks, spw, x, w, zs, y, M, N, K, gshift, fixup, epi, st);
    return launch_rows<8>(nr, ks, spw, x, w, zs, y, M, N, K, gshift, fixup, epi, st);
}

// Grouped launch (fixup arithmetic, as the automatic dispatch uses): count in 2..GEMV_GROUP_MAX linears with
// the same K <= 8192 and group size, M <= 4.  Returns hipErrorInvalidValue when the group does not qualify.
hipError_t launch_gemv2_group(const SeqProblem* probs, int count, int M, hipStream_t st) {
    if (count < 2 || count > GEMV_GROUP_MAX || M < 1 || M > 4) return hipErrorInvalidValue;
    const int K = probs[0].K, g = probs[0].group_size;
    for (int p = 1; p < count; p++)
        if (probs[p].K != K || probs[p].group_size != g) return hipErrorInvalidValue;
    const int nsteps = (K + 511) / 512;
    if (nsteps > 16) return hipErrorInvalidValue;
    int gshift = 0;
    while ((1 << gshift) < g) gshift++;
    // the single-linear choices for a weight of this K: one k range, four row groups (two k ranges for 3..4
    // tokens on K >= 4096), all k-steps of a wave in one round
    const int ks = (M >= 3 && nsteps >= 8) ? 2 : 1;
    const int spw = (nsteps + ks - 1) / ks;
#define SQ_GROUP(MR_, KS_, S_) return launch_group_cfg<MR_, 4, KS_, S_>(probs, count, M, K, gshift, st)
    if (M <= 1) {
        if (spw >= 8) SQ_GROUP(1, 1, 8);
        if (spw >= 4) SQ_GROUP(1, 1, 4);
        SQ_GROUP(1, 1, 2);
    }
    if (M <= 2) {
        if (spw >= 8) SQ_GROUP(2, 1, 8);
        if (spw >= 4) SQ_GROUP(2, 1, 4);
        SQ_GROUP(2, 1, 2);
    }
    if (ks == 2) {
        if (spw >= 4) SQ_GROUP(4, 2, 4);
        SQ_GROUP(4, 2, 2);
    }
    if (spw >= 4) SQ_GROUP(4, 1, 4);
    SQ_GROUP(4, 1, 2);
#undef SQ_GROUP
}

}  // namespace sq
