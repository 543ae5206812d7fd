// Standalone dequantisation: packed int4 -> fp16 W_hat [N,K], natural k order.
// Replaces dequant_W_kernel (reference:
// quantization/tianshu/backend/w4a16_gemm.cuh:1060-1154).  Pure bandwidth:
// reads N*K/2 + (K/g)*N*4 bytes, writes 2*N*K bytes.
#include "sq_common.h"
#include "sq_kernels.h"

namespace sq {

// Layout L1.  One thread = one packed word = 8 outputs = one 16-byte store, so a
// wave reads 256 contiguous bytes and writes 1 KiB contiguous bytes.
__global__ __launch_bounds__(256) void dequant_l1_kernel(const uint32_t* __restrict__ w,
                                                         const half2_t* __restrict__ zs,
                                                         half8_t* __restrict__ out, int K8, int gshift8,
                                                         int groups, long total_words) {
    const NibbleMasks nm = nibble_masks();
    const long stride = (long)gridDim.x * blockDim.x;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total_words; i += stride) {
        const int n = (int)(i / K8);
        const int k8 = (int)(i - (long)n * K8);
        const uint32_t word = __builtin_nontemporal_load(w + i);
        const half2_t p = zs[(long)n * groups + (k8 >> gshift8)];
        const half2_t z64 = {p.x, p.x};
        const half2_t s = {p.y, p.y};
        __builtin_nontemporal_store(dequant8(word, z64, s, nm), out + i);
    }
}

// Closed-form position of element (n,k) inside the layout-L2 weight: the tile
// order is [K/32][N/32][32 lanes][4 words][8 nibbles] with
//   lane = (n%8)*4 + (k%8)/2, word = (k%32/16)*2 + (n%32/16),
//   nibble = (k%2)*4 + ((k/8)%2)*2 + ((n/8)%2).
// (derived from the 10-axis nibble permutation of
// quantization/nvidia/kernel/gemm_s4_f16/format.cu:66-71)
__device__ __forceinline__ uint32_t l2_nibble(const uint32_t* __restrict__ w, int n, int k, int N) {
    const int kk = k & 31, nn = n & 31;
    const int lane = (nn & 7) * 4 + ((kk & 7) >> 1);
    const int word = (kk >> 4) * 2 + (nn >> 4);
    const int nib = (kk & 1) * 4 + ((kk >> 3) & 1) * 2 + ((nn >> 3) & 1);
    const long tile = (long)(k >> 5) * (N >> 5) + (n >> 5);
    return (w[(tile * 32 + lane) * 4 + word] >> (4 * nib)) & 0xFu;
}

// Layout L2.  One thread = 8 consecutive k of one row; a one-time conversion, so
// the gather through the closed form is not tuned.
__global__ __launch_bounds__(256) void dequant_l2_kernel(const uint32_t* __restrict__ w,
                                                         const half2_t* __restrict__ zs,
                                                         half8_t* __restrict__ out, int N, int K, int g) {
    const long total = (long)N * (K / 8);
    const long stride = (long)gridDim.x * blockDim.x;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        const int n = (int)(i / (K / 8));
        const int k0 = (int)(i - (long)n * (K / 8)) * 8;
        const half2_t p = zs[(long)(k0 / g) * N + n];
        half8_t r;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const half_t h = (half_t)(float)(64u + l2_nibble(w, n, k0 + j, N));
            r[j] = (h - p.x) * p.y;
        }
        out[i] = r;
    }
}

static int log2i(int v) {
    int s = 0;
    while ((1 << s) < v) s++;
    return s;
}

hipError_t launch_dequant_l1(const void* w, const void* zs, void* out, int N, int K, int g, hipStream_t st) {
    const long total = (long)N * (K / 8);
    long blocks = (total + 255) / 256;
    if (blocks > 256 * 32) blocks = 256 * 32;
    hipLaunchKernelGGL(dequant_l1_kernel, dim3((unsigned)blocks), dim3(256), 0, st, (const uint32_t*)w,
                       (const half2_t*)zs, (half8_t*)out, K / 8, log2i(g) - 3, K / g, total);
    return hipGetLastError();
}

hipError_t launch_dequant_l2(const void* w, const void* zs, void* out, int N, int K, int g, hipStream_t st) {
    const long total = (long)N * (K / 8);
    long blocks = (total + 255) / 256;
    if (blocks > 256 * 32) blocks = 256 * 32;
    hipLaunchKernelGGL(dequant_l2_kernel, dim3((unsigned)blocks), dim3(256), 0, st, (const uint32_t*)w,
                       (const half2_t*)zs, (half8_t*)out, N, K, g);
    return hipGetLastError();
}

}  // namespace sq
