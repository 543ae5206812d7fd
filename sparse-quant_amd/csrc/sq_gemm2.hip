// Prefill GEMM for layout L1, software-pipelined variant for M > 64: the same
// 128 x 256 workgroup tile, operand mapping and arithmetic as the kernel in
// sq_gemm.hip (weights dequantised in registers as the B operand of
// v_mfma_f32_32x32x16_f16, activations through a double-buffered swizzled LDS
// tile), but every operand of a 16-wide k slice is fetched one slice ahead:
//   * while the eight matrix instructions of slice t run, the four activation
//     operands of slice t+1 are read from LDS and the two weight operands of
//     slice t+1 are dequantised, so no matrix instruction waits for an LDS read
//     or for the unpack arithmetic of its own slice;
//   * the last slice of a 64-wide K step prefetches slice 0 of the next step; the
//     one barrier of a step sits before that slice, right after the activations of
//     the next step have been stored to the other LDS buffer.
// Global loads run two K steps ahead in registers, as in the base kernel.
#include "sq_common.h"
#include "sq_kernels.h"

#include <type_traits>

namespace sq {

constexpr int G2_BN = 256;
constexpr int G2_BK = 64;

__device__ __forceinline__ int swz2(int row) { return (row & 7) ^ ((row >> 3) & 1); }

template <int MI, int OCC>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(OCC, OCC))) void gemm_pipe_kernel(
    const uint8_t* __restrict__ W, const half2_t* __restrict__ ZS, const half_t* __restrict__ X,
    half_t* __restrict__ Y, int M, int N, int K, int gshift, Epilogue epi) {
    constexpr int G2_BM = 32 * MI;
    __shared__ __attribute__((aligned(1024))) uint8_t xs[2][G2_BM * 128];

    const NibbleMasks nm = nibble_masks();
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int ln = lane & 31;
    const int lc = lane >> 5;
    const int m0 = blockIdx.y * G2_BM;
    const int n0 = blockIdx.x * G2_BN + 64 * wave;
    const int groups = K >> gshift;
    const int nit = (K + G2_BK - 1) / G2_BK;

    // Staging of the activation tile: pass p of wave w moves rows 32p + 8w .. +7; lane
    // 8r + c' fetches the 16-byte chunk that belongs at position c' of its row.
    const half_t* xsrc[MI];
    int xchunk[MI];
#pragma unroll
    for (int p = 0; p < MI; p++) {
        const int R = 32 * p + 8 * wave + (lane >> 3);
        xchunk[p] = ((lane & 7) ^ swz2(R)) * 8;
        xsrc[p] = X + (long)imin(m0 + R, M - 1) * K;
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

    struct WStage {
        u32x4_t q[2];
        half2_t zs[2];
    };
    WStage w[3];
    u32x4_t xr[3][MI];
    half8_t a[2][MI];   // activation operands of the current / next slice
    half8_t bf[2][2];   // weight operands of the current / next slice

    auto load_x = [&](int it, u32x4_t (&dst)[MI]) {
#pragma unroll
        for (int p = 0; p < MI; p++) {
            const int kx = imin(it * G2_BK + xchunk[p], K - 8);
            dst[p] = *(const u32x4_t*)(xsrc[p] + kx);
        }
    };
    auto store_x = [&](int buf, const u32x4_t (&src)[MI]) {
#pragma unroll
        for (int p = 0; p < MI; p++) *(u32x4_t*)(&xs[buf][(32 * p + 8 * wave) * 128 + lane * 16]) = src[p];
    };
    auto load_w = [&](int it, WStage& ws) {
        const int kc = imin(it * G2_BK + 32 * lc, K - 32);
#pragma unroll
        for (int ni = 0; ni < 2; ni++) {
            ws.q[ni] = *(const u32x4_t*)(wsrc[ni] + (kc >> 1));
            ws.zs[ni] = zsrc[ni][kc >> gshift];
        }
    };
    int xoff[4];
#pragma unroll
    for (int t = 0; t < 4; t++) xoff[t] = ln * 128 + (((4 * lc + t) ^ swz2(ln)) * 16);

    auto read_a = [&](int buf, int t, half8_t (&dst)[MI]) {
        const uint8_t* xp = &xs[buf][0];
#pragma unroll
        for (int mi = 0; mi < MI; mi++) dst[mi] = *(const half8_t*)(xp + (32 * mi) * 128 + xoff[t]);
    };
    // Weight operands of slice t of the step held in `ws`; a k past the end gets scale 0.
    auto dequant_slice = [&](const WStage& ws, int it, int t, half8_t (&dst)[2]) {
        const bool kin = it * G2_BK + 32 * lc < K;
#pragma unroll
        for (int ni = 0; ni < 2; ni++) {
            const half_t sv = kin ? ws.zs[ni].y : (half_t)0.f;
            const half2_t z64 = {ws.zs[ni].x, ws.zs[ni].x};
            const half2_t sc = {sv, sv};
            dst[ni] = dequant8(ws.q[ni][t], z64, sc, nm);
        }
    };

    auto step = [&](int it, auto C, auto P) {
        constexpr int c = decltype(C)::value;    // register stage of this step
        constexpr int par = decltype(P)::value;  // LDS buffer of this step
        constexpr int cf = (c + 2) % 3;          // stage receiving step it + 2
        constexpr int c1 = (c + 1) % 3;          // stage holding step it + 1
        load_x(it + 2, xr[cf]);
        load_w(it + 2, w[cf]);
#pragma unroll
        for (int t = 0; t < 4; t++) {
            const int cur = t & 1, nxt = cur ^ 1;
            if (t < 3) {
                read_a(par, t + 1, a[nxt]);
                dequant_slice(w[c], it, t + 1, bf[nxt]);
            } else {
                read_a(par ^ 1, 0, a[nxt]);
                dequant_slice(w[c1], it + 1, 0, bf[nxt]);
            }
#pragma unroll
            for (int mi = 0; mi < MI; mi++)
#pragma unroll
                for (int ni = 0; ni < 2; ni++)
                    acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[cur][mi], bf[cur][ni], acc[mi][ni], 0, 0, 0);
            // One matrix instruction, then a share of the slice's other work.
#pragma unroll
            for (int q = 0; q < MI; q++) {
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);       // one LDS read
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);       // one MFMA
                __builtin_amdgcn_sched_group_barrier(0x002, 16 / MI, 0);  // VALU
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x002, 16 / MI, 0);
            }
            if (t == 2) {
                store_x(par ^ 1, xr[c1]);
                __syncthreads();
            }
        }
    };

    load_x(0, xr[0]);
    load_w(0, w[0]);
    load_x(1, xr[1]);
    load_w(1, w[1]);
    store_x(0, xr[0]);
    __syncthreads();
    read_a(0, 0, a[0]);
    dequant_slice(w[0], 0, 0, bf[0]);

    // Six steps per trip (register stage = step % 3, LDS buffer = step % 2); the step
    // count is padded with steps whose scale is 0 everywhere and whose loads are clamped.
    const int nitp = (nit + 5) / 6 * 6;
    for (int it = 0; it < nitp; it += 6) {
        step(it, std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{});
        step(it + 1, std::integral_constant<int, 1>{}, std::integral_constant<int, 1>{});
        step(it + 2, std::integral_constant<int, 2>{}, std::integral_constant<int, 0>{});
        step(it + 3, std::integral_constant<int, 0>{}, std::integral_constant<int, 1>{});
        step(it + 4, std::integral_constant<int, 1>{}, std::integral_constant<int, 0>{});
        step(it + 5, std::integral_constant<int, 2>{}, std::integral_constant<int, 1>{});
    }

    // the two activation stages (at least 32 KiB) carry the tile on its way out
    tile_store_via_lds<MI>(acc, Y, M, N, m0, blockIdx.x * G2_BN, epi, reinterpret_cast<float*>(&xs[0][0]));
}

template <int MI, int OCC>
static hipError_t launch_pipe_cfg(const void* x, const void* w, const void* zs, void* y, int M, int N, int K, int gshift,
                                  Epilogue epi, hipStream_t st) {
    const dim3 grid((N + G2_BN - 1) / G2_BN, (M + 32 * MI - 1) / (32 * MI));
    hipLaunchKernelGGL((gemm_pipe_kernel<MI, OCC>), grid, dim3(256), 0, st, (const uint8_t*)w, (const half2_t*)zs,
                       (const half_t*)x, (half_t*)y, M, N, K, gshift, epi);
    return hipGetLastError();
}

// variant: 0 = 128-row tile, two waves per SIMD; 1 = 128-row tile, one wave per SIMD;
// 2 = 256-row tile, one wave per SIMD.
hipError_t launch_gemm_pipe(const void* x, const void* w, const void* zs, void* y, int M, int N, int K, int g,
                            int variant, Epilogue epi, hipStream_t st) {
    int gshift = 0;
    while ((1 << gshift) < g) gshift++;
    if (variant == 0) return launch_pipe_cfg<4, 2>(x, w, zs, y, M, N, K, gshift, epi, st);
    if (variant == 1) return launch_pipe_cfg<4, 1>(x, w, zs, y, M, N, K, gshift, epi, st);
    return launch_pipe_cfg<8, 1>(x, w, zs, y, M, N, K, gshift, epi, st);
}

}  // namespace sq
