// Skinny GEMM for 5 <= M <= 32 with a caller-provided workspace (layout L1).
// Still HBM-bound on the weight stream; the point of this kernel is to keep the
// activation traffic (which a 16-row tile would re-read N/16 times) below the
// weight traffic and to have enough workgroups for any N.
//
// Mapping.  v_mfma_f32_16x16x32_f16 with the weights as the B operand straight
// from registers (lane l: row r + l%16, k = 128c + 32*(l/16) .. +31, one 128-bit
// load, one 32-bit word per MFMA) and the activations as the A operand (token
// l%16, the same k).  A workgroup owns 64 weight rows and one of `ksplit` K ranges;
// its waves take the 128-wide chunks of that range round-robin, and every wave
// reuses one set of activation registers for the four 16-row tiles of the 64 rows,
// so x is read once per 4 weight loads.  Partial 16x16 tiles are summed across the
// waves in LDS.  With ksplit > 1 each workgroup writes its fp32 partial tile to the
// workspace and bumps a per-row-block counter; the workgroup that arrives last adds
// the partials in a fixed order (bit-reproducible), writes Y and resets the counter.
//
// Arithmetic modes as in the GEMV kernel: exact (per-weight fp16 (q-z)*s, any group
// size) and, for g == 128 (one group per chunk), fixup: 64+q into the matrix core
// and s*(acc - (64+z)*sum_x) per chunk in fp32.
#include "sq_common.h"
#include "sq_kernels.h"

namespace sq {

constexpr int SK2_COUNTER_BYTES = 65536;  // start of the workspace: one uint32 per 64-row block

template <int MT, int NWV, bool FIXUP>
__global__ __launch_bounds__(64 * NWV) void skinny2_kernel(const uint8_t* __restrict__ W,
                                                           const half2_t* __restrict__ ZS,
                                                           const half_t* __restrict__ X, half_t* __restrict__ Y,
                                                           float* part, unsigned* counters, int M, int N, int K,
                                                           int gshift, int ksplit) {
    constexpr int TILE = 4 * MT * 4 * 64;  // floats a wave contributes: [rt][mt][v][lane]
    __shared__ float red[NWV * TILE];
    __shared__ unsigned last_flag;

    const NibbleMasks nm = nibble_masks();
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int li = lane & 15;
    const int lj = lane >> 4;
    const int rb = blockIdx.x;
    const int ks = blockIdx.y;
    const int groups = K >> gshift;
    const int nchunks = (K + 127) >> 7;
    const int cps = (nchunks + ksplit - 1) / ksplit;
    const int c_begin = ks * cps;
    const int c_end = imin(c_begin + cps, nchunks);

    float4_t acc[4][MT];
#pragma unroll
    for (int rt = 0; rt < 4; rt++)
#pragma unroll
        for (int mt = 0; mt < MT; mt++) acc[rt][mt] = (float4_t){0.f, 0.f, 0.f, 0.f};
    const half8_t ones = {(half_t)1.f, (half_t)1.f, (half_t)1.f, (half_t)1.f,
                          (half_t)1.f, (half_t)1.f, (half_t)1.f, (half_t)1.f};

    const uint8_t* wrow[4];
    const half2_t* zrow[4];
#pragma unroll
    for (int rt = 0; rt < 4; rt++) {
        const int row = imin(rb * 64 + 16 * rt + li, N - 1);
        wrow[rt] = W + (long)row * (K >> 1);
        zrow[rt] = ZS + (long)row * groups;
    }

    // Two chunks per trip: all eight weight loads are issued before the first use.
    for (int c0 = c_begin + 2 * wave; c0 < c_end; c0 += 2 * NWV) {
        u32x4_t wq[2][4];
        half2_t zq[2][4];
        int kcs[2];
        bool valid[2];
#pragma unroll
        for (int u = 0; u < 2; u++) {
            const int kk = ((c0 + u) << 7) + 32 * lj;
            valid[u] = (c0 + u < c_end) && (kk < K);
            kcs[u] = valid[u] ? kk : 0;
#pragma unroll
            for (int rt = 0; rt < 4; rt++) {
                wq[u][rt] = __builtin_nontemporal_load((const u32x4_t*)(wrow[rt] + (kcs[u] >> 1)));
                zq[u][rt] = zrow[rt][kcs[u] >> gshift];
            }
        }
#pragma unroll
        for (int u = 0; u < 2; u++) {
            u32x4_t xa[MT][4];
#pragma unroll
            for (int mt = 0; mt < MT; mt++) {
                const u32x4_t* xp = (const u32x4_t*)(X + (long)imin(16 * mt + li, M - 1) * K + kcs[u]);
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    const u32x4_t v = xp[t];
                    xa[mt][t] = valid[u] ? v : (u32x4_t){0u, 0u, 0u, 0u};
                }
            }
            float4_t xs[MT];
            if (FIXUP) {
#pragma unroll
                for (int mt = 0; mt < MT; mt++) {
                    xs[mt] = (float4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int t = 0; t < 4; t++)
                        xs[mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(bit_cast<half8_t>(xa[mt][t]), ones, xs[mt], 0, 0,
                                                                        0);
                }
            }
#pragma unroll
            for (int rt = 0; rt < 4; rt++) {
                if (!FIXUP) {
                    const half2_t z64 = {zq[u][rt].x, zq[u][rt].x};
                    const half2_t sc = {zq[u][rt].y, zq[u][rt].y};
#pragma unroll
                    for (int t = 0; t < 4; t++) {
                        const half8_t wv = dequant8(wq[u][rt][t], z64, sc, nm);
#pragma unroll
                        for (int mt = 0; mt < MT; mt++)
                            acc[rt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(bit_cast<half8_t>(xa[mt][t]), wv,
                                                                                 acc[rt][mt], 0, 0, 0);
                    }
                } else {
                    float4_t tmp[MT];
#pragma unroll
                    for (int mt = 0; mt < MT; mt++) tmp[mt] = (float4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int t = 0; t < 4; t++) {
                        const half8_t wv = unpack8_raw(wq[u][rt][t], nm);
#pragma unroll
                        for (int mt = 0; mt < MT; mt++)
                            tmp[mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(bit_cast<half8_t>(xa[mt][t]), wv, tmp[mt],
                                                                             0, 0, 0);
                    }
                    const float zf = (float)zq[u][rt].x;
                    const float sf = (float)zq[u][rt].y;
#pragma unroll
                    for (int mt = 0; mt < MT; mt++)
#pragma unroll
                        for (int v = 0; v < 4; v++) acc[rt][mt][v] += sf * (tmp[mt][v] - zf * xs[mt][v]);
                }
            }
        }
    }

    // Sum the waves' partial tiles: red[wave][rt][mt][v][lane].
#pragma unroll
    for (int rt = 0; rt < 4; rt++)
#pragma unroll
        for (int mt = 0; mt < MT; mt++)
#pragma unroll
            for (int v = 0; v < 4; v++) red[wave * TILE + ((rt * MT + mt) * 4 + v) * 64 + lane] = acc[rt][mt][v];
    __syncthreads();

    // Element t of the tile: lane l = t % 64, v, mt, rt -> token m = 16mt + 4(l/16) + v,
    // row n = 64 rb + 16 rt + l%16.
    if (ksplit == 1) {
        for (int t = tid; t < TILE; t += 64 * NWV) {
            float sum = 0.f;
#pragma unroll
            for (int p = 0; p < NWV; p++) sum += red[p * TILE + t];
            const int l = t & 63, v = (t >> 6) & 3, mt = (t >> 8) % MT, rt = (t >> 8) / MT;
            const int m = 16 * mt + 4 * (l >> 4) + v;
            const int n = rb * 64 + 16 * rt + (l & 15);
            if (m < M && n < N) Y[(long)m * N + n] = (half_t)sum;
        }
        return;
    }
    // Cross-workgroup exchange.  The partial tiles travel as agent-scope relaxed atomic
    // stores and loads, which go to the device-coherent level directly, so no device-wide
    // release/acquire fence (which would write back and invalidate the whole L2) is needed:
    // the wait for outstanding vector memory operations orders the partial stores before
    // the counter increment, and the last arriver reads the partials past its own caches.
    float* mine = part + ((long)ks * gridDim.x + rb) * TILE;
    for (int t = tid; t < TILE; t += 64 * NWV) {
        float sum = 0.f;
#pragma unroll
        for (int p = 0; p < NWV; p++) sum += red[p * TILE + t];
        __hip_atomic_store(mine + t, sum, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0) {
        const unsigned old = __hip_atomic_fetch_add(&counters[rb], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        last_flag = (old == (unsigned)(ksplit - 1)) ? 1u : 0u;
    }
    __syncthreads();
    if (!last_flag) return;
    for (int t = tid; t < TILE; t += 64 * NWV) {
        float sum = 0.f;
        for (int q = 0; q < ksplit; q++)
            sum += __hip_atomic_load(part + ((long)q * gridDim.x + rb) * TILE + t, __ATOMIC_RELAXED,
                                     __HIP_MEMORY_SCOPE_AGENT);
        const int l = t & 63, v = (t >> 6) & 3, mt = (t >> 8) % MT, rt = (t >> 8) / MT;
        const int m = 16 * mt + 4 * (l >> 4) + v;
        const int n = rb * 64 + 16 * rt + (l & 15);
        if (m < M && n < N) Y[(long)m * N + n] = (half_t)sum;
    }
    // leave the workspace ready for the next call
    if (tid == 0) __hip_atomic_store(&counters[rb], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

static int pick_ksplit(int N, int K, int nwv) {
    const int nchunks = (K + 127) / 128;
    const int row_blocks = (N + 63) / 64;
    int ks = 1;
    // enough workgroups for 256 CUs, but at least one chunk per wave and at most 8 partials
    while (ks < 8 && row_blocks * ks < 256 && nchunks / (ks * 2) >= nwv) ks *= 2;
    return ks;
}

size_t skinny2_workspace_bytes(int M, int N, int K) {
    const int mt = (M + 15) / 16;
    const int row_blocks = (N + 63) / 64;
    return (size_t)SK2_COUNTER_BYTES + (size_t)8 * row_blocks * (4 * mt * 4 * 64) * sizeof(float);
}

template <int MT, int NWV>
static hipError_t launch_cfg(const void* x, const void* w, const void* zs, void* y, void* ws, int M, int N, int K,
                             int gshift, bool fixup, int ksplit, hipStream_t st) {
    const dim3 grid((N + 63) / 64, ksplit);
    unsigned* counters = (unsigned*)ws;
    float* part = (float*)((char*)ws + SK2_COUNTER_BYTES);
    if (fixup)
        hipLaunchKernelGGL((skinny2_kernel<MT, NWV, true>), grid, dim3(64 * NWV), 0, st, (const uint8_t*)w,
                           (const half2_t*)zs, (const half_t*)x, (half_t*)y, part, counters, M, N, K, gshift, ksplit);
    else
        hipLaunchKernelGGL((skinny2_kernel<MT, NWV, false>), grid, dim3(64 * NWV), 0, st, (const uint8_t*)w,
                           (const half2_t*)zs, (const half_t*)x, (half_t*)y, part, counters, M, N, K, gshift, ksplit);
    return hipGetLastError();
}

// tune = 0 for the heuristic, else ksplit (1,2,4,8) | mode << 8 (1 = exact, 2 = fixup).
// The first 64 KiB of the workspace are counters and must be zero before the first call;
// every call leaves them zero.
hipError_t launch_skinny2_tuned(const void* x, const void* w, const void* zs, void* y, void* ws, int M, int N, int K,
                                int g, int tune, hipStream_t st) {
    int gshift = 0;
    while ((1 << gshift) < g) gshift++;
    const int mt = (M + 15) / 16;
    const int nwv = mt == 1 ? 8 : 4;
    int ksplit = tune & 0xFF;
    if (ksplit != 1 && ksplit != 2 && ksplit != 4 && ksplit != 8) ksplit = pick_ksplit(N, K, nwv);
    const int mode = (tune >> 8) & 0xFF;
    bool fixup = (g == 128);
    if (mode == 1) fixup = false;
    if (mt == 1) return launch_cfg<1, 8>(x, w, zs, y, ws, M, N, K, gshift, fixup, ksplit, st);
    return launch_cfg<2, 4>(x, w, zs, y, ws, M, N, K, gshift, fixup, ksplit, st);
}

}  // namespace sq
