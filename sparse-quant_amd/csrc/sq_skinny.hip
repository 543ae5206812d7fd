// Skinny GEMM (8 < M <= 64) for layout L1: still HBM-bound on the weight stream,
// but wide enough in M that the 16x16x32 matrix instruction is the right shape.
//
// Mapping.  A workgroup owns 16 output rows (weight rows) and the whole K; its
// waves take interleaved 128-wide K chunks.  For v_mfma_f32_16x16x32_f16 lane l
// supplies, for both operands, index l%16 of the non-contracted dimension and 8
// contracted elements selected by l/16.  The weight operand is built directly
// in registers: lane l loads the 128-bit word holding k = 128c + 32*(l/16) ..
// +31 of row r0 + l%16 and uses one of its four 32-bit words per MFMA; the
// activation operand takes the matching 8 k from x[m = l%16].  Weights never
// touch LDS.  D[m][n] lands as lane = n + 16*(m/4), register = m%4.
//
// Arithmetic modes as in the GEMV kernel: exact (per-weight fp16 (q-z)*s) for any
// group size, and for g == 128 (one group per chunk) the fixup mode that feeds
// 64+q to the matrix core and applies s*(acc - (64+z)*sum_x) per chunk in fp32.
// (replaces w4a16_gemm_wmma_kernel<16,16,256,264,24> for small M, reference:
// quantization/muxi/backend/w4a16_gemm.cuh:466-600)
#include "sq_common.h"
#include "sq_kernels.h"

namespace sq {

template <int MT, bool FIXUP>
__global__ __launch_bounds__(512) void skinny_kernel(const uint8_t* __restrict__ W, const half2_t* __restrict__ ZS,
                                                     const half_t* __restrict__ X, half_t* __restrict__ Y, int M,
                                                     int N, int K, int gshift, Epilogue epi) {
    extern __shared__ float red[];
    const NibbleMasks nm = nibble_masks();
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int nwaves = blockDim.x >> 6;
    const int li = lane & 15;
    const int lj = lane >> 4;
    const int row0 = blockIdx.x * 16;
    const int row = imin(row0 + li, N - 1);
    const int nchunks = (K + 127) >> 7;
    const int groups = K >> gshift;

    float4_t acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; mt++) acc[mt] = (float4_t){0.f, 0.f, 0.f, 0.f};
    const half8_t ones = {(half_t)1.f, (half_t)1.f, (half_t)1.f, (half_t)1.f,
                          (half_t)1.f, (half_t)1.f, (half_t)1.f, (half_t)1.f};

    const uint8_t* wrow = W + (long)row * (K >> 1);
    const half2_t* zrow = ZS + (long)row * groups;

    for (int c = wave; c < nchunks; c += nwaves) {
        const int kk = (c << 7) + 32 * lj;
        const bool kvalid = kk < K;
        const int kc = kvalid ? kk : 0;
        const u32x4_t wq = __builtin_nontemporal_load((const u32x4_t*)(wrow + (kc >> 1)));
        const half2_t zsv = zrow[kc >> gshift];
        u32x4_t xa[MT][4];
#pragma unroll
        for (int mt = 0; mt < MT; mt++) {
            const int m = imin(16 * mt + li, M - 1);
            const u32x4_t* xp = (const u32x4_t*)(X + (long)m * K + kc);
#pragma unroll
            for (int t = 0; t < 4; t++) {
                u32x4_t v = xp[t];
                xa[mt][t] = kvalid ? v : (u32x4_t){0u, 0u, 0u, 0u};
            }
        }
        if (!FIXUP) {
            const half2_t z64 = {zsv.x, zsv.x};
            const half2_t sc = {zsv.y, zsv.y};
#pragma unroll
            for (int t = 0; t < 4; t++) {
                const half8_t wv = dequant8(wq[t], z64, sc, nm);
#pragma unroll
                for (int mt = 0; mt < MT; mt++)
                    acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(bit_cast<half8_t>(xa[mt][t]), wv, acc[mt], 0,
                                                                      0, 0);
            }
        } else {
            float4_t tmp[MT], xs[MT];
#pragma unroll
            for (int mt = 0; mt < MT; mt++) {
                tmp[mt] = (float4_t){0.f, 0.f, 0.f, 0.f};
                xs[mt] = (float4_t){0.f, 0.f, 0.f, 0.f};
            }
#pragma unroll
            for (int t = 0; t < 4; t++) {
                const half8_t wv = unpack8_raw(wq[t], nm);
#pragma unroll
                for (int mt = 0; mt < MT; mt++) {
                    const half8_t xv = bit_cast<half8_t>(xa[mt][t]);
                    tmp[mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xv, wv, tmp[mt], 0, 0, 0);
                    xs[mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xv, ones, xs[mt], 0, 0, 0);
                }
            }
            const float zf = (float)zsv.x;
            const float sf = (float)zsv.y;
#pragma unroll
            for (int mt = 0; mt < MT; mt++)
#pragma unroll
                for (int v = 0; v < 4; v++) acc[mt][v] += sf * (tmp[mt][v] - zf * xs[mt][v]);
        }
    }

    // Sum the waves' partial 16x16 tiles through LDS: red[wave][mt][v][lane].
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int v = 0; v < 4; v++) red[((wave * MT + mt) * 4 + v) * 64 + lane] = acc[mt][v];
    __syncthreads();
    for (int t = threadIdx.x; t < MT * 4 * 64; t += blockDim.x) {
        float sum = 0.f;
        for (int p = 0; p < nwaves; p++) sum += red[p * (MT * 4 * 64) + t];
        const int l = t & 63;
        const int v = (t >> 6) & 3;
        const int mt = t >> 8;
        const int m = 16 * mt + 4 * (l >> 4) + v;
        const int n = row0 + (l & 15);
        if (m < M && n < N) Y[(long)m * N + n] = epilogue(sum, m, n, N, epi);
    }
}

template <int MT>
static hipError_t launch_mt(const void* x, const void* w, const void* zs, void* y, int M, int N, int K, int gshift,
                            bool fixup, int nwaves, Epilogue epi, hipStream_t st) {
    const dim3 grid((N + 15) / 16);
    const dim3 block(64 * nwaves);
    const size_t lds = (size_t)nwaves * MT * 4 * 64 * sizeof(float);
    if (fixup)
        hipLaunchKernelGGL((skinny_kernel<MT, true>), grid, block, lds, st, (const uint8_t*)w, (const half2_t*)zs,
                           (const half_t*)x, (half_t*)y, M, N, K, gshift, epi);
    else
        hipLaunchKernelGGL((skinny_kernel<MT, false>), grid, block, lds, st, (const uint8_t*)w, (const half2_t*)zs,
                           (const half_t*)x, (half_t*)y, M, N, K, gshift, epi);
    return hipGetLastError();
}

// tune = 0 for the heuristic, else waves | (mode << 8) with mode 1 = exact, 2 = fixup.
hipError_t launch_skinny_tuned(const void* x, const void* w, const void* zs, void* y, int M, int N, int K, int g,
                               int tune, Epilogue epi, hipStream_t st) {
    int gshift = 0;
    while ((1 << gshift) < g) gshift++;
    int nwaves = tune & 0xFF;
    const int mode = (tune >> 8) & 0xFF;
    const int nchunks = (K + 127) / 128;
    if (nwaves < 1 || nwaves > 8) nwaves = nchunks >= 8 ? 8 : nchunks;
    bool fixup = (g == 128);
    if (mode == 1) fixup = false;
    if (mode == 2 && g == 128) fixup = true;
    const int mt = (M + 15) / 16;
    switch (mt) {
        case 1: return launch_mt<1>(x, w, zs, y, M, N, K, gshift, fixup, nwaves, epi, st);
        case 2: return launch_mt<2>(x, w, zs, y, M, N, K, gshift, fixup, nwaves, epi, st);
        case 3: return launch_mt<3>(x, w, zs, y, M, N, K, gshift, fixup, nwaves, epi, st);
        default: return launch_mt<4>(x, w, zs, y, M, N, K, gshift, fixup, nwaves, epi, st);
    }
}


}  // namespace sq
