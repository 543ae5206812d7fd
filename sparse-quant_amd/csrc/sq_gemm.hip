// Prefill GEMM (any M, tuned for M >= 128) for layout L1: a dense contraction on
// the fp16 matrix cores, bounded by MFMA throughput (2*M*N*K flops).
//
// Tile.  A workgroup of 4 waves computes BM x 256 outputs (BM = 32*MI); wave wv
// owns all BM rows and the 64 columns n0 + 64*wv .. +63, i.e. MI x 2 tiles of
// v_mfma_f32_32x32x16_f16.  Per 64-wide K step:
//   * weights: lane l loads one 128-bit word per column tile = 32 consecutive k of
//     weight row n0 + 64*wv + 32*ni + l%32, starting at k0 + 32*(l/32), and
//     dequantises it in registers to fp16 (q - z) * s (bit-identical to the
//     reference's W_hat).  Its four 32-bit words are exactly the B operands of the
//     four MFMA k-steps, so the weights never pass through LDS and no wave repeats
//     another wave's dequantisation;
//   * activations: the BM x 64 tile goes global -> registers -> LDS (double
//     buffered, row pitch 144 B so that 128-bit reads are bank-conflict free) and
//     every wave reads its A operands with ds_read_b128; lane (l%32, l/32) reads
//     x[m0 + 32*mi + l%32][k0 + 32*(l/32) + 8*t .. +7], the same k the weight
//     operand of that lane holds.
// One barrier per K step.  D[m][n]: lane = n%32 + 32*((m/4)%2), register =
// m%4 + 4*(m/8).
// (replaces w4a16_gemm_wmma_kernel, reference:
// quantization/muxi/backend/w4a16_gemm.cuh:466-600, and the role of
// turbomind::GemmS4F16, quantization/nvidia/kernel/gemm_s4_f16/gemm_template.h:358-450)
#include "sq_common.h"
#include "sq_kernels.h"

namespace sq {

constexpr int GEMM_BN = 256;
constexpr int GEMM_BK = 64;
constexpr int GEMM_PITCH = 72;  // halves per LDS row (64 + 8 padding)

template <int MI>
__global__ __launch_bounds__(256) void gemm_kernel(const uint8_t* __restrict__ W, const half2_t* __restrict__ ZS,
                                                   const half_t* __restrict__ X, half_t* __restrict__ Y, int M,
                                                   int N, int K, int gshift) {
    constexpr int BM = 32 * MI;
    __shared__ __attribute__((aligned(16))) half_t xs[2][BM * GEMM_PITCH];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int ln = lane & 31;
    const int lc = lane >> 5;
    const int m0 = blockIdx.y * BM;
    const int n0 = blockIdx.x * GEMM_BN + 64 * wave;
    const int groups = K >> gshift;
    const int nit = (K + GEMM_BK - 1) / GEMM_BK;

    // Global -> LDS staging of the activation tile: thread t moves, per pass p, the
    // 16 bytes at row 32*p + t/8, halves (t%8)*8 .. +7.
    const int xr = tid >> 3;
    const int xc = (tid & 7) * 8;
    const half_t* xsrc[MI];
    bool xrow_ok[MI];
#pragma unroll
    for (int p = 0; p < MI; p++) {
        const int m = m0 + 32 * p + xr;
        xrow_ok[p] = m < M;
        xsrc[p] = X + (long)imin(m, M - 1) * K + xc;
    }

    const uint8_t* wsrc[2];
    const half2_t* zsrc[2];
#pragma unroll
    for (int ni = 0; ni < 2; ni++) {
        const int n = imin(n0 + 32 * ni + ln, N - 1);
        wsrc[ni] = W + (long)n * (K >> 1);
        zsrc[ni] = ZS + (long)n * groups;
    }

    float16_t acc[MI][2];
#pragma unroll
    for (int mi = 0; mi < MI; mi++)
#pragma unroll
        for (int ni = 0; ni < 2; ni++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[mi][ni][v] = 0.f;

    u32x4_t xreg[MI];
    u32x4_t wq[2];
    half2_t zq[2];

    auto load_tile = [&](int it) {
        const int k0 = it * GEMM_BK;
#pragma unroll
        for (int p = 0; p < MI; p++) {
            const bool ok = xrow_ok[p] && (k0 + xc < K);
            const u32x4_t v = *(const u32x4_t*)(xsrc[p] + (ok ? k0 : 0));
            xreg[p] = ok ? v : (u32x4_t){0u, 0u, 0u, 0u};
        }
        const int kw = k0 + 32 * lc;
        const int kc = kw < K ? kw : 0;  // past-the-end k meets zero activations
#pragma unroll
        for (int ni = 0; ni < 2; ni++) {
            wq[ni] = *(const u32x4_t*)(wsrc[ni] + (kc >> 1));
            zq[ni] = zsrc[ni][kc >> gshift];
        }
    };
    auto store_tile = [&](int buf) {
#pragma unroll
        for (int p = 0; p < MI; p++) *(u32x4_t*)(&xs[buf][(32 * p + xr) * GEMM_PITCH + xc]) = xreg[p];
    };

    load_tile(0);
    store_tile(0);
    __syncthreads();

    for (int it = 0; it < nit; it++) {
        const int cur = it & 1;
        // Dequantise this step's weights into the four B operands per column tile.
        half8_t bf[2][4];
#pragma unroll
        for (int ni = 0; ni < 2; ni++) {
            const half2_t z64 = {zq[ni].x, zq[ni].x};
            const half2_t sc = {zq[ni].y, zq[ni].y};
#pragma unroll
            for (int t = 0; t < 4; t++) bf[ni][t] = dequant8(wq[ni][t], z64, sc);
        }
        // Prefetch the next step (registers only; LDS is written after the MFMAs).
        if (it + 1 < nit) load_tile(it + 1);

        const half_t* xb = &xs[cur][ln * GEMM_PITCH + 32 * lc];
#pragma unroll
        for (int t = 0; t < 4; t++) {
#pragma unroll
            for (int mi = 0; mi < MI; mi++) {
                const half8_t a = *(const half8_t*)(xb + (32 * mi) * GEMM_PITCH + 8 * t);
#pragma unroll
                for (int ni = 0; ni < 2; ni++)
                    acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, bf[ni][t], acc[mi][ni], 0, 0, 0);
            }
        }
        if (it + 1 < nit) store_tile(cur ^ 1);
        __syncthreads();
    }

    // Epilogue: fp32 -> fp16, 32 consecutive columns per half-wave.
#pragma unroll
    for (int mi = 0; mi < MI; mi++)
#pragma unroll
        for (int ni = 0; ni < 2; ni++) {
            const int n = n0 + 32 * ni + ln;
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int m = m0 + 32 * mi + 8 * (v >> 2) + 4 * lc + (v & 3);
                if (m < M && n < N) Y[(long)m * N + n] = (half_t)acc[mi][ni][v];
            }
        }
}

template <int MI>
static hipError_t launch_mi(const void* x, const void* w, const void* zs, void* y, int M, int N, int K, int gshift,
                            hipStream_t st) {
    const dim3 grid((N + GEMM_BN - 1) / GEMM_BN, (M + 32 * MI - 1) / (32 * MI));
    hipLaunchKernelGGL((gemm_kernel<MI>), grid, dim3(256), 0, st, (const uint8_t*)w, (const half2_t*)zs,
                       (const half_t*)x, (half_t*)y, M, N, K, gshift);
    return hipGetLastError();
}

// tune = 0 for the heuristic, else the number of 32-row tiles per workgroup (1, 2 or 4).
hipError_t launch_gemm_tuned(const void* x, const void* w, const void* zs, void* y, int M, int N, int K, int g,
                             int tune, hipStream_t st) {
    int gshift = 0;
    while ((1 << gshift) < g) gshift++;
    int mi = tune & 0xFF;
    if (mi != 1 && mi != 2 && mi != 4) mi = M > 64 ? 4 : (M > 32 ? 2 : 1);
    switch (mi) {
        case 1: return launch_mi<1>(x, w, zs, y, M, N, K, gshift, st);
        case 2: return launch_mi<2>(x, w, zs, y, M, N, K, gshift, st);
        default: return launch_mi<4>(x, w, zs, y, M, N, K, gshift, st);
    }
}


}  // namespace sq
