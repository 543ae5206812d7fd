// LayerNorm over the last dimension for fp16 activations, fp32 statistics:
//   y[r, :] = (x[r, :] - mean_r) * rsqrt(var_r + eps) * gamma + beta,  var = biased variance.
// The decode step of the OPT harness runs two of these per layer on a handful of rows
// (reference: test/nvidia/module/opt/modeling_opt_ours.py:500-507,561-562,603-604 -- torch's
// nn.LayerNorm there); at that size the work is one launch latency, so the kernel is a single
// pass: one workgroup per row, the row held in registers between the two reductions (mean
// first, then the variance around it, as torch computes it), one 128-bit load and store per
// eight elements, gamma and beta fetched before the reductions.
#include "sq_common.h"
#include "sq_kernels.h"

namespace sq {

namespace {

constexpr int LN_THREADS = 256;

__device__ __forceinline__ float block_sum(float v, float* red) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, 64);
    const int wave = threadIdx.x >> 6;
    __syncthreads();  // red may still be read from the previous reduction
    if ((threadIdx.x & 63) == 0) red[wave] = v;
    __syncthreads();
    return (red[0] + red[1]) + (red[2] + red[3]);
}

// VPT 128-bit vectors per thread: cols <= 8 * LN_THREADS * VPT
template <int VPT>
__global__ __launch_bounds__(LN_THREADS) void layernorm_kernel(const half_t* __restrict__ X,
                                                               const half_t* __restrict__ gamma,
                                                               const half_t* __restrict__ beta,
                                                               half_t* __restrict__ Y, int cols, float eps) {
    __shared__ float red[4];
    const long row = blockIdx.x;
    const int nvec = cols >> 3;
    half8_t v[VPT], g[VPT], b[VPT];
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < VPT; i++) {
        const int j = threadIdx.x + i * LN_THREADS;
        if (j < nvec) v[i] = *(const half8_t*)(X + row * cols + 8 * j);
    }
    // gamma and beta are requested now so that their latency hides behind the two reductions
#pragma unroll
    for (int i = 0; i < VPT; i++) {
        const int j = threadIdx.x + i * LN_THREADS;
        if (j < nvec) {
            if (gamma) g[i] = *(const half8_t*)(gamma + 8 * j);
            if (beta) b[i] = *(const half8_t*)(beta + 8 * j);
        }
    }
#pragma unroll
    for (int i = 0; i < VPT; i++) {
        const int j = threadIdx.x + i * LN_THREADS;
        if (j < nvec) {
#pragma unroll
            for (int e = 0; e < 8; e++) sum += (float)v[i][e];
        }
    }
    const float mean = block_sum(sum, red) / (float)cols;
    float sq = 0.f;
#pragma unroll
    for (int i = 0; i < VPT; i++) {
        const int j = threadIdx.x + i * LN_THREADS;
        if (j < nvec) {
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const float d = (float)v[i][e] - mean;
                sq += d * d;
            }
        }
    }
    const float rstd = rsqrtf(block_sum(sq, red) / (float)cols + eps);
#pragma unroll
    for (int i = 0; i < VPT; i++) {
        const int j = threadIdx.x + i * LN_THREADS;
        if (j < nvec) {
            half8_t o;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                float t = ((float)v[i][e] - mean) * rstd;
                if (gamma) t *= (float)g[i][e];
                if (beta) t += (float)b[i][e];
                o[e] = (half_t)t;
            }
            *(half8_t*)(Y + row * cols + 8 * j) = o;
        }
    }
}

}  // namespace

hipError_t launch_layernorm(const void* x, const void* gamma, const void* beta, void* y, int rows, int cols, float eps,
                            hipStream_t st) {
    const int nvec = cols / 8;
    const dim3 grid(rows), block(LN_THREADS);
#define SQ_LN(V)                                                                                                   \
    hipLaunchKernelGGL((layernorm_kernel<V>), grid, block, 0, st, (const half_t*)x, (const half_t*)gamma,          \
                       (const half_t*)beta, (half_t*)y, cols, eps)
    if (nvec <= LN_THREADS) SQ_LN(1);
    else if (nvec <= 2 * LN_THREADS) SQ_LN(2);
    else if (nvec <= 4 * LN_THREADS) SQ_LN(4);
    else SQ_LN(8);
#undef SQ_LN
    return hipGetLastError();
}

}  // namespace sq
