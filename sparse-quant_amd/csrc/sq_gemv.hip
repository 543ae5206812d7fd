// Decode GEMV / very skinny GEMM (M <= 8) for layout L1.  HBM-bandwidth bound:
// per output row the kernel streams K/2 bytes of int4 weights and K/g half2
// (zero,scale) pairs once; algorithmic bytes = N*K/2 + (K/g)*N*4 + M*K*2 + M*N*2.
//
// Mapping.  v_mfma_f32_4x4x4_16B_f16 multiplies 16 independent 4x4x4 blocks; in
// block b lane 4b+i supplies row i of A (4 k) and column i of B (4 k) and receives
// D[0..3][i].  With A = activations (row = token m) and B = weights (column =
// output row), every lane accumulates its own output row over its own k range
// for up to 4 tokens, and the matrix core does all the multiply-adds: the VALU
// only unpacks nibbles.  Lane 4b+i of a wave owns output row r0+i and the 32
// consecutive k starting at slice*512 + 32*b, i.e. one 128-bit weight load; a
// wave-wide load therefore covers 4 rows x 256 contiguous bytes.  The waves of
// a workgroup take different 512-wide K slices of the same rows; partial sums
// are combined over the 16 blocks with DPP row rotations and over row groups /
// waves through LDS.
//
// Two arithmetic modes (both accumulate in fp32):
//   exact : B = fp16((q - z) * s), bit-identical to the reference's W_hat.
//   fixup : B = 64 + q (bit pattern only); per 32-k run the lane adds
//           s * (sum x*(64+q) - (64+z) * sum x), i.e. zero and scale are applied
//           once per run in fp32 instead of once per weight in fp16.
// (replaces w4a16_bs1_kernel / w4a16_bs2_kernel, reference:
// quantization/muxi/backend/w4a16_gemm.cuh:14-151,153-326)
#include "sq_common.h"
#include "sq_kernels.h"

namespace sq {

template <int RS, int MROWS, bool FIXUP>
__global__ __launch_bounds__(1024) void gemv_kernel(const uint8_t* __restrict__ W, const half2_t* __restrict__ ZS,
                                                    const half_t* __restrict__ X, half_t* __restrict__ Y, int M,
                                                    int N, int K, int gshift, Epilogue epi) {
    constexpr int MT = (MROWS + 3) / 4;
    extern __shared__ float red[];

    const NibbleMasks nm = nibble_masks();
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int nwaves = blockDim.x >> 6;
    const int i = lane & 3;
    const int b = lane >> 2;
    const int row0 = blockIdx.x * (4 * RS);
    const int nslices = (K + 511) >> 9;
    const int groups = K >> gshift;

    float4_t acc[RS][MT];
#pragma unroll
    for (int rs = 0; rs < RS; rs++)
#pragma unroll
        for (int mt = 0; mt < MT; mt++) acc[rs][mt] = (float4_t){0.f, 0.f, 0.f, 0.f};

    const half4_t ones = {(half_t)1.f, (half_t)1.f, (half_t)1.f, (half_t)1.f};

    for (int s = wave; s < nslices; s += nwaves) {
        const int kk = (s << 9) + 32 * b;
        const bool kvalid = kk < K;
        const int kc = kvalid ? kk : 0;

        // Weights and (zero,scale) first: they are the HBM stream.
        u32x4_t wq[RS];
        half2_t zsv[RS];
#pragma unroll
        for (int rs = 0; rs < RS; rs++) {
            const int row = imin(row0 + 4 * rs + i, N - 1);
            wq[rs] = __builtin_nontemporal_load((const u32x4_t*)(W + (long)row * (K >> 1) + (kc >> 1)));
            zsv[rs] = ZS[(long)row * groups + (kc >> gshift)];
        }
        // Activations of the 32 k of this block.
        u32x4_t xa[MT][4];
        float4_t xs[MT];
        if (MROWS == 1) {
            // One token: the four lanes of a block need the same 64 bytes.  Each
            // loads a different quarter (so the wave reads the slice's 1 KiB once,
            // fully coalesced) and the quarters are exchanged with DPP quad
            // broadcasts; every row of A then holds token 0.
            const u32x4_t own = *(const u32x4_t*)(X + kc + 8 * i);
            const u32x4_t xv = kvalid ? own : (u32x4_t){0u, 0u, 0u, 0u};
            xa[0][0] = quad_bcast<0>(xv);
            xa[0][1] = quad_bcast<1>(xv);
            xa[0][2] = quad_bcast<2>(xv);
            xa[0][3] = quad_bcast<3>(xv);
            if (FIXUP) {
                const half8_t h = bit_cast<half8_t>(xv);
                float sum = 0.f;
#pragma unroll
                for (int e = 0; e < 8; e++) sum += (float)h[e];
                sum = quad_sum(sum);
                xs[0] = (float4_t){sum, sum, sum, sum};
            }
        } else {
#pragma unroll
            for (int mt = 0; mt < MT; mt++) {
                const int m = imin(4 * mt + i, M - 1);
                const u32x4_t* xp = (const u32x4_t*)(X + (long)m * K + kc);
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    u32x4_t v = xp[t];
                    xa[mt][t] = kvalid ? v : (u32x4_t){0u, 0u, 0u, 0u};
                }
            }
            if (FIXUP) {
#pragma unroll
                for (int mt = 0; mt < MT; mt++) {
                    xs[mt] = (float4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int t = 0; t < 4; t++) {
                        const half8_t xv = bit_cast<half8_t>(xa[mt][t]);
                        xs[mt] = __builtin_amdgcn_mfma_f32_4x4x4f16(xv.lo, ones, xs[mt], 0, 0, 0);
                        xs[mt] = __builtin_amdgcn_mfma_f32_4x4x4f16(xv.hi, ones, xs[mt], 0, 0, 0);
                    }
                }
            }
        }

#pragma unroll
        for (int rs = 0; rs < RS; rs++) {
            const half2_t z64 = {zsv[rs].x, zsv[rs].x};
            const half2_t sc = {zsv[rs].y, zsv[rs].y};
            if (!FIXUP) {
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    const half8_t wv = dequant8(wq[rs][t], z64, sc, nm);
#pragma unroll
                    for (int mt = 0; mt < MT; mt++) {
                        const half8_t xv = bit_cast<half8_t>(xa[mt][t]);
                        acc[rs][mt] = __builtin_amdgcn_mfma_f32_4x4x4f16(xv.lo, wv.lo, acc[rs][mt], 0, 0, 0);
                        acc[rs][mt] = __builtin_amdgcn_mfma_f32_4x4x4f16(xv.hi, wv.hi, acc[rs][mt], 0, 0, 0);
                    }
                }
            } else {
                float4_t tmp[MT];
#pragma unroll
                for (int mt = 0; mt < MT; mt++) tmp[mt] = (float4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    const half8_t wv = unpack8_raw(wq[rs][t], nm);
#pragma unroll
                    for (int mt = 0; mt < MT; mt++) {
                        const half8_t xv = bit_cast<half8_t>(xa[mt][t]);
                        tmp[mt] = __builtin_amdgcn_mfma_f32_4x4x4f16(xv.lo, wv.lo, tmp[mt], 0, 0, 0);
                        tmp[mt] = __builtin_amdgcn_mfma_f32_4x4x4f16(xv.hi, wv.hi, tmp[mt], 0, 0, 0);
                    }
                }
                const float zf = (float)zsv[rs].x;
                const float sf = (float)zsv[rs].y;
#pragma unroll
                for (int mt = 0; mt < MT; mt++)
#pragma unroll
                    for (int j = 0; j < 4; j++)
                        if (4 * mt + j < MROWS) acc[rs][mt][j] += sf * (tmp[mt][j] - zf * xs[mt][j]);
            }
        }
    }

    // Combine the 16 blocks of a wave (DPP within each 16-lane row, LDS across
    // the 4 rows) and the waves of the workgroup.
    constexpr int VALS = RS * MROWS;
#pragma unroll
    for (int rs = 0; rs < RS; rs++)
#pragma unroll
        for (int m = 0; m < MROWS; m++) {
            const float v = row_sum_stride4(acc[rs][m >> 2][m & 3]);
            if ((lane & 12) == 0) red[((wave * 4 + (lane >> 4)) * VALS + rs * MROWS + m) * 4 + i] = v;
        }
    __syncthreads();
    const int parts = nwaves * 4;
    for (int t = threadIdx.x; t < VALS * 4; t += blockDim.x) {
        float sum = 0.f;
        for (int p = 0; p < parts; p++) sum += red[p * (VALS * 4) + t];
        const int ri = t & 3;
        const int m = (t >> 2) % MROWS;
        const int rs = (t >> 2) / MROWS;
        const int row = row0 + 4 * rs + ri;
        if (row < N && m < M) Y[(long)m * N + row] = epilogue(sum, m, row, N, epi);
    }
}

template <int RS, int MROWS>
static hipError_t launch_cfg(const void* x, const void* w, const void* zs, void* y, int M, int N, int K, int gshift,
                             bool fixup, int nwaves, Epilogue epi, hipStream_t st) {
    const int rows = 4 * RS;
    const dim3 grid((N + rows - 1) / rows);
    const dim3 block(64 * nwaves);
    const size_t lds = (size_t)nwaves * 4 * RS * MROWS * 4 * sizeof(float);
    if (fixup)
        hipLaunchKernelGGL((gemv_kernel<RS, MROWS, true>), grid, block, lds, st, (const uint8_t*)w,
                           (const half2_t*)zs, (const half_t*)x, (half_t*)y, M, N, K, gshift, epi);
    else
        hipLaunchKernelGGL((gemv_kernel<RS, MROWS, false>), grid, block, lds, st, (const uint8_t*)w,
                           (const half2_t*)zs, (const half_t*)x, (half_t*)y, M, N, K, gshift, epi);
    return hipGetLastError();
}

template <int MROWS>
static hipError_t launch_rows(int rs, const void* x, const void* w, const void* zs, void* y, int M, int N, int K,
                              int gshift, bool fixup, int nwaves, Epilogue epi, hipStream_t st) {
    switch (rs) {
        case 1: return launch_cfg<1, MROWS>(x, w, zs, y, M, N, K, gshift, fixup, nwaves, epi, st);
        case 2: return launch_cfg<2, MROWS>(x, w, zs, y, M, N, K, gshift, fixup, nwaves, epi, st);
        default: return launch_cfg<4, MROWS>(x, w, zs, y, M, N, K, gshift, fixup, nwaves, epi, st);
    }
}

// tune = 0 for the built-in heuristic, else (row steps per workgroup) | (waves << 8).
hipError_t launch_gemv_tuned(const void* x, const void* w, const void* zs, void* y, int M, int N, int K, int g,
                             bool fixup, int tune, Epilogue epi, hipStream_t st) {
    int gshift = 0;
    while ((1 << gshift) < g) gshift++;
    const int nslices = (K + 511) / 512;
    int rs = tune & 0xFF, nwaves = (tune >> 8) & 0xFF;
    if (rs != 1 && rs != 2 && rs != 4) rs = (N >= 8192) ? 4 : 2;
    if (nwaves < 1 || nwaves > 16) nwaves = nslices >= 32 ? 16 : (nslices >= 8 ? 8 : (nslices >= 4 ? 4 : nslices));
    if (M <= 1) return launch_rows<1>(rs, x, w, zs, y, M, N, K, gshift, fixup, nwaves, epi, st);
    if (M <= 2) return launch_rows<2>(rs, x, w, zs, y, M, N, K, gshift, fixup, nwaves, epi, st);
    if (M <= 4) return launch_rows<4>(rs, x, w, zs, y, M, N, K, gshift, fixup, nwaves, epi, st);
    return launch_rows<8>(rs, x, w, zs, y, M, N, K, gshift, fixup, nwaves, epi, st);
}


}  // namespace sq
