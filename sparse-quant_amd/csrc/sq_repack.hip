// One-time weight / zero-scale format converters (integer and byte shuffles).
// None of them is on the per-token path; each is a flat gather with one thread per
// destination element, so no atomics are needed.
#include "sq_common.h"
#include "sq_kernels.h"

namespace sq {

static dim3 flat_grid(long total, int block) {
    long b = (total + block - 1) / block;
    if (b < 1) b = 1;
    if (b > 65536) b = 65536;
    return dim3((unsigned)b);
}

// zeros, scales [N, K/g] -> zs half2 [K/g, N] = (zero + 64, scale).
// (reference: quantization/nvidia/kernel/gemm_s4_f16/format.cu:206-239)
__global__ void transpose_merge_kernel(const half_t* __restrict__ zeros, const half_t* __restrict__ scales,
                                       half2_t* __restrict__ zs, int groups, int N) {
    const long total = (long)groups * N;
    const long stride = (long)gridDim.x * blockDim.x;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        const int j = (int)(i / N);  // destination-major walk: coalesced stores
        const int n = (int)(i - (long)j * N);
        const long src = (long)n * groups + j;
        half2_t v = {(half_t)(zeros[src] + (half_t)64.0f), scales[src]};
        zs[i] = v;
    }
}

// "ours" uint8 [N, K/2] (even k in the high nibble) -> uint32 [K, N/8]; word (k,c)
// holds columns 8c + {0,2,4,6,1,3,5,7} from its least significant nibble.
// (reference: quantization/nvidia/kernel/gemm_s4_f16/format.cu:151-201)
__global__ void ours_to_awq_kernel(const uint8_t* __restrict__ src, uint32_t* __restrict__ dst, int K, int N) {
    const int words = N / 8;
    const long total = (long)K * words;
    const long stride = (long)gridDim.x * blockDim.x;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        const int k = (int)(i / words);
        const int c = (int)(i - (long)k * words);
        const int shift = (k & 1) ? 0 : 4;
        uint32_t out = 0;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const uint32_t v = (src[(long)(8 * c + j) * (K / 2) + (k >> 1)] >> shift) & 0xFu;
            const int pos = (j & 1) * 4 + (j >> 1);
            out |= v << (4 * pos);
        }
        dst[i] = out;
    }
}

// AWQ-order uint32 [K, N/8] -> layout-L2 storage.  The destination word index d
// decomposes as [tile][lane][word]; inverting the closed form gives, for nibble
// `nib` of that word,
//   k%32 = 16*(word/2) + 8*((nib/2)%2) + 2*(lane%4) + nib/4
//   n%32 = 16*(word%2) + 8*(nib%2) + lane/4.
// (reference: quantization/nvidia/kernel/gemm_s4_f16/format.cu:24-57,66-71)
__global__ void awq_to_lmdeploy_kernel(const uint32_t* __restrict__ src, uint32_t* __restrict__ dst, int K, int N) {
    const long total = (long)K * (N / 8);
    const int ntiles = N / 32;
    const long stride = (long)gridDim.x * blockDim.x;
    for (long d = (long)blockIdx.x * blockDim.x + threadIdx.x; d < total; d += stride) {
        const int word = (int)(d & 3);
        const int lane = (int)((d >> 2) & 31);
        const long tile = d >> 7;
        const int kt = (int)(tile / ntiles), nt = (int)(tile - (long)kt * ntiles);
        uint32_t out = 0;
#pragma unroll
        for (int nib = 0; nib < 8; nib++) {
            const int kk = 16 * (word >> 1) + 8 * ((nib >> 1) & 1) + 2 * (lane & 3) + (nib >> 2);
            const int nn = 16 * (word & 1) + 8 * (nib & 1) + (lane >> 2);
            const int k = kt * 32 + kk, n = nt * 32 + nn;
            const int j = n & 7;
            const int pos = (j & 1) * 4 + (j >> 1);
            const uint32_t v = (src[(long)k * (N / 8) + (n >> 3)] >> (4 * pos)) & 0xFu;
            out |= v << (4 * nib);
        }
        dst[d] = out;
    }
}

// Layout L2 -> layout L1: one thread per L1 word (row n, 8 consecutive k).
__global__ void l2_to_l1_weight_kernel(const uint32_t* __restrict__ w2, uint32_t* __restrict__ w1, int N, int K) {
    const int K8 = K / 8;
    const long total = (long)N * K8;
    const long stride = (long)gridDim.x * blockDim.x;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        const int n = (int)(i / K8);
        const int k0 = (int)(i - (long)n * K8) * 8;
        uint32_t out = 0;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int k = k0 + j;
            const int kk = k & 31, nn = n & 31;
            const int lane = (nn & 7) * 4 + ((kk & 7) >> 1);
            const int word = (kk >> 4) * 2 + (nn >> 4);
            const int nib = (kk & 1) * 4 + ((kk >> 3) & 1) * 2 + ((nn >> 3) & 1);
            const long tile = (long)(k >> 5) * (N >> 5) + (n >> 5);
            const uint32_t v = (w2[(tile * 32 + lane) * 4 + word] >> (4 * nib)) & 0xFu;
            const int pos = (j & 1) * 4 + (j >> 1);  // L1 nibble order k0,k2,k4,k6,k1,k3,k5,k7
            out |= v << (4 * pos);
        }
        w1[i] = out;
    }
}

// zs half2 [K/g, N] -> half2 [N, K/g].
__global__ void l2_to_l1_zs_kernel(const uint32_t* __restrict__ zs2, uint32_t* __restrict__ zs1, int groups, int N) {
    const long total = (long)groups * N;
    const long stride = (long)gridDim.x * blockDim.x;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        const int n = (int)(i / groups);
        const int j = (int)(i - (long)n * groups);
        zs1[i] = zs2[(long)j * N + n];
    }
}

// 2-bit packed byte b -> two 4-bit packed bytes
//   ((b & 0xC0) >> 2) + ((b & 0x30) >> 4)  and  ((b & 0x0C) << 2) + (b & 0x03).
// (reference: test/muxi/module/qlinear/qlinear.py:93-103)
__global__ void w2_to_w4_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst, long total) {
    const long stride = (long)gridDim.x * blockDim.x;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        const uint32_t b = src[i];
        dst[2 * i] = (uint8_t)(((b & 0xC0u) >> 2) + ((b & 0x30u) >> 4));
        dst[2 * i + 1] = (uint8_t)(((b & 0x0Cu) << 2) + (b & 0x03u));
    }
}

// Tensor-core layout, 2-bit storage, with the arithmetic the reference's Python performs
// (reference: test/nvidia/utils/quant_dequant_nvidia.py:34-54).  `<<` and `>>` bind tighter than `&`
// there, so the eight masks of each loop add up to one constant: a pair of 4-bit words (a, b) is
// stored as (a & 0xFFFF0000) + (b & 0x0000FFFF), and a stored word w expands to the pair
// (w & 0x33333333, w & 0x33333333).  Mirrored bit for bit; it is not an inverse pair.
__global__ void l2_w4_to_w2_kernel(const uint32_t* __restrict__ src, uint32_t* __restrict__ dst, long total) {
    const long stride = (long)gridDim.x * blockDim.x;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride)
        dst[i] = (src[2 * i] & 0xFFFF0000u) + (src[2 * i + 1] & 0x0000FFFFu);
}

__global__ void l2_w2_to_w4_kernel(const uint32_t* __restrict__ src, uint32_t* __restrict__ dst, long total) {
    const long stride = (long)gridDim.x * blockDim.x;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        const uint32_t w = src[i] & 0x33333333u;
        dst[2 * i] = w;
        dst[2 * i + 1] = w;
    }
}

hipError_t launch_transpose_merge_zeros_scales(const void* zeros, const void* scales, void* zs, int K, int N, int g,
                                               hipStream_t st) {
    const long total = (long)(K / g) * N;
    hipLaunchKernelGGL(transpose_merge_kernel, flat_grid(total, 256), dim3(256), 0, st, (const half_t*)zeros,
                       (const half_t*)scales, (half2_t*)zs, K / g, N);
    return hipGetLastError();
}

hipError_t launch_ours_to_awq(const void* src, void* dst, int K, int N, hipStream_t st) {
    hipLaunchKernelGGL(ours_to_awq_kernel, flat_grid((long)K * (N / 8), 256), dim3(256), 0, st,
                       (const uint8_t*)src, (uint32_t*)dst, K, N);
    return hipGetLastError();
}

hipError_t launch_awq_to_lmdeploy(const void* src, void* dst, int K, int N, hipStream_t st) {
    hipLaunchKernelGGL(awq_to_lmdeploy_kernel, flat_grid((long)K * (N / 8), 256), dim3(256), 0, st,
                       (const uint32_t*)src, (uint32_t*)dst, K, N);
    return hipGetLastError();
}

hipError_t launch_l2_to_l1(const void* w_l2, const void* zs_l2, void* w_l1, void* zs_l1, int N, int K, int g,
                           hipStream_t st) {
    hipLaunchKernelGGL(l2_to_l1_weight_kernel, flat_grid((long)N * (K / 8), 256), dim3(256), 0, st,
                       (const uint32_t*)w_l2, (uint32_t*)w_l1, N, K);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(l2_to_l1_zs_kernel, flat_grid((long)N * (K / g), 256), dim3(256), 0, st,
                       (const uint32_t*)zs_l2, (uint32_t*)zs_l1, K / g, N);
    return hipGetLastError();
}

hipError_t launch_2bit_to_4bit(const void* src, void* dst, int N, int K, hipStream_t st) {
    const long total = (long)N * (K / 4);
    hipLaunchKernelGGL(w2_to_w4_kernel, flat_grid(total, 256), dim3(256), 0, st, (const uint8_t*)src,
                       (uint8_t*)dst, total);
    return hipGetLastError();
}

hipError_t launch_l2_4bit_to_2bit(const void* src, void* dst, int K, int N, hipStream_t st) {
    const long total = (long)K * (N / 16);
    hipLaunchKernelGGL(l2_w4_to_w2_kernel, flat_grid(total, 256), dim3(256), 0, st, (const uint32_t*)src,
                       (uint32_t*)dst, total);
    return hipGetLastError();
}

hipError_t launch_l2_2bit_to_4bit(const void* src, void* dst, int K, int N, hipStream_t st) {
    const long total = (long)K * (N / 16);
    hipLaunchKernelGGL(l2_w2_to_w4_kernel, flat_grid(total, 256), dim3(256), 0, st, (const uint32_t*)src,
                       (uint32_t*)dst, total);
    return hipGetLastError();
}

}  // namespace sq
