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
//   * activations: the BM x 64 tile goes global -> registers (three K steps ahead) ->
//     LDS (double buffered, XOR-swizzled 16-byte chunks so that 128-bit reads are
//     bank-conflict free) and every wave reads its A operands with ds_read_b128; lane (l%32, l/32) reads
//     x[m0 + 32*mi + l%32][k0 + 32*(l/32) + 8*t .. +7], the same k the weight
//     operand of that lane holds.
// One barrier per K step.  D[m][n]: lane = n%32 + 32*((m/4)%2), register =
// m%4 + 4*(m/8).
// (replaces w4a16_gemm_wmma_kernel, reference:
// quantization/muxi/backend/w4a16_gemm.cuh:466-600, and the role of
// turbomind::GemmS4F16, quantization/nvidia/kernel/gemm_s4_f16/gemm_template.h:358-450)
#include "sq_common.h"
#include "sq_kernels.h"

#include <type_traits>

namespace sq {

constexpr int GEMM_BN = 256;
constexpr int GEMM_BK = 64;
constexpr int GEMM_STAGES = 3;  // register stages; loads run GEMM_STAGES - 1 steps ahead

__device__ __forceinline__ int swz(int row) { return (row & 7) ^ ((row >> 3) & 1); }

// What follows the K loop in both tiled kernels: with K split over gridDim.z workgroups the
// partial tiles meet in the workspace, then the epilogue and the fp16 stores (through `lds`, 32 KiB
// of shared memory that the main loop no longer needs).
template <int MI>
__device__ __forceinline__ void gemm_tail(float16_t (&acc)[MI][2], half_t* __restrict__ Y, int M, int N, int m0, int n0,
                                          const Epilogue& epi, float* part, unsigned* counters, float* lds) {
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int ln = lane & 31;
    const int lc = lane >> 5;
    const int ksplit = gridDim.z;
    if (ksplit > 1) {
        // Partial tiles meet in the workspace: 128-bit stores at the device-coherent cache level,
        // one counter per output tile; the workgroup that arrives last adds the partials in a
        // fixed order (bit-reproducible), stores the tile and resets the counter.
        __shared__ unsigned last_flag;
        constexpr int SLOTS = MI * 2 * 4;  // float4 per thread
        const long tile = (long)blockIdx.y * gridDim.x + blockIdx.x;
        const long ntile = (long)gridDim.x * gridDim.y;
        float* mine = part + ((long)blockIdx.z * ntile + tile) * (SLOTS * 256 * 4);
#pragma unroll
        for (int mi = 0; mi < MI; mi++)
#pragma unroll
            for (int ni = 0; ni < 2; ni++)
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const float4_t v4 = {acc[mi][ni][4 * q], acc[mi][ni][4 * q + 1], acc[mi][ni][4 * q + 2],
                                         acc[mi][ni][4 * q + 3]};
                    store_coherent_x4(mine + (((mi * 2 + ni) * 4 + q) * 256 + tid) * 4, v4);
                }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (tid == 0) {
            const unsigned old = __hip_atomic_fetch_add(&counters[tile], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            last_flag = (old == (unsigned)(ksplit - 1)) ? 1u : 0u;
        }
        __syncthreads();
        if (!last_flag) return;
        // The last arriver's loads are round trips to L2 that nothing hides: sixteen per thread in
        // flight, i.e. 16 / NZ of its SLOTS per trip, NZ = the number of partials rounded up to 2, 4
        // or 8 (sources past ksplit re-read the first partial and are not added).
        const float* first = part + tile * (SLOTS * 256 * 4) + tid * 4;
        const long zstride = ntile * (SLOTS * 256 * 4);
        auto reduce = [&](auto NZ_) {
            constexpr int NZ = decltype(NZ_)::value;
            constexpr int PAIRS = 8 / NZ;  // pairs of slots per trip
#pragma unroll
            for (int s0 = 0; s0 < SLOTS; s0 += 2 * PAIRS) {
                const float* src[8];
                float4_t pv[16];
#pragma unroll
                for (int pr = 0; pr < PAIRS; pr++)
#pragma unroll
                    for (int z = 0; z < NZ; z++)
                        src[pr * NZ + z] = first + (long)(z < ksplit ? z : 0) * zstride + (s0 + 2 * pr + 1) * 1024;
                load16_coherent_x4(src, pv);
#pragma unroll
                for (int pr = 0; pr < PAIRS; pr++)
#pragma unroll
                    for (int h = 0; h < 2; h++) {
                        float4_t sum = pv[2 * (pr * NZ) + h];
#pragma unroll
                        for (int z = 1; z < NZ; z++)
                            if (z < ksplit) sum += pv[2 * (pr * NZ + z) + h];
                        const int slot = s0 + 2 * pr + h;
#pragma unroll
                        for (int e = 0; e < 4; e++) acc[slot >> 3][(slot >> 2) & 1][4 * (slot & 3) + e] = sum[e];
                    }
            }
        };
        if (ksplit <= 2)
            reduce(std::integral_constant<int, 2>{});
        else if (ksplit <= 4)
            reduce(std::integral_constant<int, 4>{});
        else
            reduce(std::integral_constant<int, 8>{});
        if (tid == 0) __hip_atomic_store(&counters[tile], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }

    tile_store_via_lds<MI>(acc, Y, M, N, m0, n0 - 64 * (tid >> 6), epi, lds);
}

// Two waves per SIMD (two workgroups per CU): one wave alone cannot both issue the
// unpack / LDS / load instructions of a step and keep the matrix pipe full.
template <int MI>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void gemm_kernel(const uint8_t* __restrict__ W, const half2_t* __restrict__ ZS,
                                                   const half_t* __restrict__ X, half_t* __restrict__ Y, int M,
                                                   int N, int K, int gshift, Epilogue epi, float* part,
                                                   unsigned* counters) {
    constexpr int BM = 32 * MI;
    // Activation tile, two stages, row pitch 128 B (64 halves, no padding); the eight
    // 16-byte chunks of row R are stored at chunk position c ^ swz(R); 8 consecutive
    // rows then use 8 distinct positions and 16 consecutive rows 16 distinct 16-byte
    // slots of a 256-byte bank period, so the 128-bit operand reads are conflict free.
    // (at least 16 KiB per stage: the tail passes the tile through these 32 KiB)
    __shared__ __attribute__((aligned(1024))) uint8_t xs[2][BM * 128 < 16384 ? 16384 : BM * 128];

    const NibbleMasks nm = nibble_masks();
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int ln = lane & 31;
    const int lc = lane >> 5;
    const int m0 = blockIdx.y * BM;
    const int n0 = blockIdx.x * GEMM_BN + 64 * wave;
    const int groups = K >> gshift;
    const int nit = (K + GEMM_BK - 1) / GEMM_BK;
    // K split over gridDim.z workgroups (1 = no split): this one runs steps it0 .. it1-1.
    const int ksplit = gridDim.z;
    const int spz = (nit + ksplit - 1) / ksplit;
    const int it0 = blockIdx.z * spz;
    const int it1 = imin(it0 + spz, nit);

    // Global -> registers -> LDS staging of the activation tile.  Pass p of wave w moves
    // rows 32*p + 8*w .. +7; lane l = 8*r + c' fetches the chunk that belongs at
    // position c' of row R = 32*p + 8*w + r, so a wave writes 1 KiB of contiguous LDS.
    // Rows past M are clamped to row M-1: they only feed output rows that are never
    // stored.
    const half_t* xsrc[MI];
    int xchunk[MI];
#pragma unroll
    for (int p = 0; p < MI; p++) {
        const int R = 32 * p + 8 * wave + (lane >> 3);
        xchunk[p] = ((lane & 7) ^ swz(R)) * 8;
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

    // All loads are unconditional: a k past the end is clamped to the last valid 8
    // halves / 32 nibbles and the scale of those lanes is replaced by 0, which zeroes
    // their weight operand.
    struct WStage {
        u32x4_t q[2];
        half2_t zs[2];
    };
    WStage w[GEMM_STAGES];
    u32x4_t xr[GEMM_STAGES][MI];

    auto load_x = [&](int it, u32x4_t (&dst)[MI]) {
#pragma unroll
        for (int p = 0; p < MI; p++) {
            const int kx = imin(it * GEMM_BK + xchunk[p], K - 8);
            dst[p] = *(const u32x4_t*)(xsrc[p] + kx);
        }
    };
    auto store_x = [&](int buf, const u32x4_t (&src)[MI]) {
#pragma unroll
        for (int p = 0; p < MI; p++) *(u32x4_t*)(&xs[buf][(32 * p + 8 * wave) * 128 + lane * 16]) = src[p];
    };
    auto load_w = [&](int it, WStage& ws) {
        const int kc = imin(it * GEMM_BK + 32 * lc, K - 32);
#pragma unroll
        for (int ni = 0; ni < 2; ni++) {
            ws.q[ni] = *(const u32x4_t*)(wsrc[ni] + (kc >> 1));
            ws.zs[ni] = zsrc[ni][kc >> gshift];
        }
    };

    // Operand read offsets: lane (ln, lc) reads row 32*mi + ln, chunk 4*lc + t.
    int xoff[4];
#pragma unroll
    for (int t = 0; t < 4; t++) xoff[t] = ln * 128 + (((4 * lc + t) ^ swz(ln)) * 16);

    // One K step; C = it % GEMM_STAGES selects the register stage.  The loads of step
    // it + 2 are issued first and fenced off (the scheduler would otherwise sink them
    // below the matrix instructions); behind the fence the dequantisation of this
    // step's weight registers and the matrix instructions interleave freely.  At the
    // end the activations of step it + 1, fetched a step ago, go to the other LDS
    // buffer: loads complete in order, so that store waits for nothing recent.
    auto step = [&](int it, auto C, auto P) {
        constexpr int c = decltype(C)::value;
        constexpr int par = decltype(P)::value;  // LDS buffer of this step
        constexpr int cf = (c + GEMM_STAGES - 1) % GEMM_STAGES;  // stage receiving step it + 2
        constexpr int c1 = (c + 1) % GEMM_STAGES;                // stage holding step it + 1
        load_x(it + GEMM_STAGES - 1, xr[cf]);
        load_w(it + GEMM_STAGES - 1, w[cf]);
        __builtin_amdgcn_sched_barrier(0);
        half8_t bf[2][4];
        const bool kin = it < it1 && it * GEMM_BK + 32 * lc < K;  // false past the range: scale 0 -> W_hat 0
#pragma unroll
        for (int ni = 0; ni < 2; ni++) {
            const half_t sv = kin ? w[c].zs[ni].y : (half_t)0.f;
            const half2_t z64 = {w[c].zs[ni].x, w[c].zs[ni].x};
            const half2_t sc = {sv, sv};
#pragma unroll
            for (int t = 0; t < 4; t++) bf[ni][t] = dequant8(w[c].q[ni][t], z64, sc, nm);
        }
        const uint8_t* xp = &xs[par][0];
#pragma unroll
        for (int t = 0; t < 4; t++) {
#pragma unroll
            for (int mi = 0; mi < MI; mi++) {
                const half8_t a = *(const half8_t*)(xp + (32 * mi) * 128 + xoff[t]);
#pragma unroll
                for (int ni = 0; ni < 2; ni++)
                    acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, bf[ni][t], acc[mi][ni], 0, 0, 0);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        store_x(par ^ 1, xr[c1]);
        __syncthreads();
    };

#pragma unroll
    for (int s0 = 0; s0 < GEMM_STAGES - 1; s0++) {
        load_x(it0 + s0, xr[s0]);
        load_w(it0 + s0, w[s0]);
    }
    store_x(0, xr[0]);
    __syncthreads();
    // Six steps per trip (stage indices are compile-time); the step count is padded
    // with steps whose scale is 0 everywhere and whose loads are clamped.
    constexpr int TRIP = 2 * GEMM_STAGES;
    static_assert(GEMM_STAGES == 3, "the trip below is written for three register stages");
    const int nitp = (it1 - it0 + TRIP - 1) / TRIP * TRIP;
    for (int it = it0; it < it0 + nitp; it += TRIP) {
        // LDS buffer = step parity, register stage = step % GEMM_STAGES: unroll over
        // their common period.
        step(it, std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{});
        step(it + 1, std::integral_constant<int, 1>{}, std::integral_constant<int, 1>{});
        step(it + 2, std::integral_constant<int, 2>{}, std::integral_constant<int, 0>{});
        step(it + 3, std::integral_constant<int, 0>{}, std::integral_constant<int, 1>{});
        step(it + 4, std::integral_constant<int, 1>{}, std::integral_constant<int, 0>{});
        step(it + 5, std::integral_constant<int, 2>{}, std::integral_constant<int, 1>{});
    }

    gemm_tail<MI>(acc, Y, M, N, m0, n0, epi, part, counters, reinterpret_cast<float*>(&xs[0][0]));
}

// Both operands through LDS, for group sizes 32, 64 and 128 and K a multiple of 256.  The kernels above hand
// every lane its own 16 bytes of a weight row (32 rows per wave-wide load) and 4 bytes of
// zeros/scales, and the L1 takes lanes that are not neighbours in memory one at a time: about 1240
// cache accesses per workgroup and K step, three per four cycles, which is what bounds those
// kernels between decode and prefill.  Here every operand goes global -> LDS with direct loads
// (no registers in between):
//   * weights: a wave moves its own 64 rows x 32 bytes in two instructions whose neighbouring
//     lanes are neighbours in memory; lane l of instruction i fetches half
//     (l & 1) ^ ((row >> 3) & 1) of row 32 * i + l / 2, so that the operand reads (lane = row,
//     128 bits) are bank-conflict free;
//   * activations: the swizzled chunk order of the register-staged kernel, written by the load
//     instead of a store;
//   * zeros/scales: the two pairs of 2 g columns (four steps at group size 128, two at 64, one
//     at 32), one dword per lane, two neighbouring lanes on the two pairs of a row.
// Three stages (two for zeros/scales, three at group size 32), loads two steps ahead; one barrier per step, behind a
// counted wait for the loads of the next step (the loads just issued stay in flight).  Same
// operand mapping and arithmetic as gemm_kernel: bit-identical results.
template <int MI, int GS>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void gemm_lds_kernel(
    const uint8_t* __restrict__ W, const half2_t* __restrict__ ZS, const half_t* __restrict__ X, half_t* __restrict__ Y,
    int M, int N, int K, Epilogue epi, float* part, unsigned* counters) {
    constexpr int BM = 32 * MI;
    constexpr int XB = BM * 128;  // bytes of an activation stage
    constexpr int WB = 256 * 32;  // bytes of a weight stage
    constexpr int ZB = 256 * 8;   // bytes of a zeros/scales stage: 4 waves x 2 pairs x 64 rows
    // GS = log2 of the group size (5, 6, 7).  A zeros/scales stage always holds the two pairs of
    // 2 g columns, i.e. of P = g / 32 steps: it is refilled every P steps, and with P = 1 it rotates
    // with the operand stages (three of them) instead of alternating.
    constexpr int P = 1 << (GS - 5);
    constexpr int NZST = P == 1 ? 3 : 2;
    static_assert(GS >= 5 && GS <= 7, "group sizes 32, 64, 128");
    constexpr int W_OFF = 0, Z_OFF = 3 * WB, X_OFF = Z_OFF + NZST * ZB;
    __shared__ __attribute__((aligned(1024))) uint8_t lds[X_OFF + 3 * XB];
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)lds;

    const NibbleMasks nm = nibble_masks();
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int ln = lane & 31;
    const int lc = lane >> 5;
    const int m0 = blockIdx.y * BM;
    const int n0 = blockIdx.x * GEMM_BN + 64 * wave;
    const int groups = K >> GS;
    const int nit = K / GEMM_BK;
    // K split in whole four-step groups
    const int ksplit = gridDim.z;
    const int spz = ((nit + ksplit - 1) / ksplit + 3) & ~3;
    const int it0 = blockIdx.z * spz;
    const int it1 = imin(it0 + spz, nit);

    // Every address is a wave-uniform base that walks along K plus a byte offset per lane that never changes
    // (the launcher keeps operands whose offsets would not fit 32 bits away from this kernel).
    uint32_t xlane[MI];
#pragma unroll
    for (int p = 0; p < MI; p++) {
        const int R = 32 * p + 8 * wave + (lane >> 3);
        xlane[p] = (uint32_t)(((long)imin(m0 + R, M - 1) * K + ((lane & 7) ^ swz(R)) * 8) * 2);
    }
    uint32_t wlane[2];
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const int r = 32 * i + (lane >> 1);
        wlane[i] = (uint32_t)((long)imin(n0 + r, N - 1) * (K >> 1) + 16 * ((lane & 1) ^ ((r >> 3) & 1)));
    }
    // zeros/scales: instruction i moves the two pairs of rows 32 i .. 32 i + 31, two neighbouring lanes per row
    // (8 contiguous bytes), so that it touches 32 places in memory rather than 64
    uint32_t zlane[2];
#pragma unroll
    for (int i = 0; i < 2; i++)
        zlane[i] = (uint32_t)((long)imin(n0 + 32 * i + (lane >> 1), N - 1) * groups * 4 + (lane & 1) * 4);
    int woff[2], zoff[2];
#pragma unroll
    for (int ni = 0; ni < 2; ni++) {
        woff[ni] = W_OFF + wave * 2048 + ((32 * ni + ln) * 2 + (lc ^ ((ln >> 3) & 1))) * 16;
        zoff[ni] = Z_OFF + wave * 512 + ni * 256 + ln * 8 + (GS == 5 ? lc * 4 : 0);  // g = 32: the pair of the lane's half
    }
    int xoff[4];
#pragma unroll
    for (int t = 0; t < 4; t++) xoff[t] = X_OFF + ln * 128 + (((4 * lc + t) ^ swz(ln)) * 16);

    float16_t acc[MI][2];
#pragma unroll
    for (int mi = 0; mi < MI; mi++)
#pragma unroll
        for (int ni = 0; ni < 2; ni++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[mi][ni][v] = 0.f;

    // Loads of step `it` into stage c (both wave-uniform); a step past the end re-reads the last one, its scale
    // is zeroed at use.
    auto issue = [&](int it, int c) {
        const int itc = imin(it, nit - 1);
        const uint8_t* xb = (const uint8_t*)X + (long)itc * (GEMM_BK * 2);
        const uint8_t* wb = W + (long)itc * (GEMM_BK / 2);
#pragma unroll
        for (int p = 0; p < MI; p++) load_to_lds_x4(xb, xlane[p], lds0 + X_OFF + c * XB + (32 * p + 8 * wave) * 128);
#pragma unroll
        for (int i = 0; i < 2; i++) load_to_lds_x4(wb, wlane[i], lds0 + W_OFF + c * WB + wave * 2048 + i * 1024);
    };
    // The two zeros/scales pairs of the P steps that start at step `it`, into stage zc.
    auto issue_zs = [&](int it, int zc) {
        const half2_t* zb = ZS + imin((it * GEMM_BK) >> GS, groups - 2);
        load_to_lds_x1(zb, zlane[0], lds0 + Z_OFF + zc * ZB + wave * 512);
        load_to_lds_x1(zb, zlane[1], lds0 + Z_OFF + zc * ZB + wave * 512 + 256);
    };

    // One K step: J = step within its group of four, c = its stage, cf = the stage read in the step
    // before (free since that step's barrier), zc = the zeros/scales stage of steps 0 and 1 of the four.
    auto step = [&](int it, int c, int cf, int zc, auto J_) {
        constexpr int j = decltype(J_)::value;
        constexpr bool fill = (j + 2) % P == 0;  // step it + 2 starts a zeros/scales group
        const int zcur = P == 1 ? c : (P == 2 ? zc ^ (j >> 1) : zc);
        issue(it + 2, cf);
        if constexpr (fill) issue_zs(it + 2, P == 1 ? cf : zcur ^ 1);
        __builtin_amdgcn_sched_barrier(0);
        const bool kin = it < it1 && it * GEMM_BK + 32 * lc < K;  // false past the range: scale 0 -> W_hat 0
        u32x4_t q[2];
        half2_t z64[2], sc[2];
#pragma unroll
        for (int ni = 0; ni < 2; ni++) {
            q[ni] = *(const u32x4_t*)(lds + c * WB + woff[ni]);
            const half2_t zsv = *(const half2_t*)(lds + zcur * ZB + (P == 4 ? (j >> 1) : (P == 2 ? (j & 1) : 0)) * 4 + zoff[ni]);
            const half_t sv = kin ? zsv.y : (half_t)0.f;
            z64[ni] = (half2_t){zsv.x, zsv.x};
            sc[ni] = (half2_t){sv, sv};
        }
        const uint8_t* xp = lds + c * XB;
#pragma unroll
        for (int t = 0; t < 4; t++) {
            half8_t bf[2];
#pragma unroll
            for (int ni = 0; ni < 2; ni++) bf[ni] = dequant8(q[ni][t], z64[ni], sc[ni], nm);
#pragma unroll
            for (int mi = 0; mi < MI; mi++) {
                const half8_t a = *(const half8_t*)(xp + (32 * mi) * 128 + xoff[t]);
#pragma unroll
                for (int ni = 0; ni < 2; ni++)
                    acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, bf[ni], acc[mi][ni], 0, 0, 0);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        // the loads of step it + 1 (issued a step ago) have landed, this wave's operand reads are done:
        // behind the barrier stage c is free and the next stage is complete
        asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(MI + 2 + (fill ? 2 : 0)) : "memory");
    };

    issue_zs(it0, 0);
    issue(it0, 0);
    if constexpr (P == 1) issue_zs(it0 + 1, 1);
    issue(it0 + 1, 1);
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(MI + 2 + (P == 1 ? 2 : 0)) : "memory");
    const int end = it0 + (it1 - it0 + 3) / 4 * 4;  // padded with steps whose scale is 0 and whose loads are clamped
    int c = 0, cp = 2, zc = 0;
    auto advance = [&]() {
        cp = c;
        c = c == 2 ? 0 : c + 1;
    };
    for (int it = it0; it < end; it += 4) {
        step(it, c, cp, zc, std::integral_constant<int, 0>{});
        advance();
        step(it + 1, c, cp, zc, std::integral_constant<int, 1>{});
        advance();
        step(it + 2, c, cp, zc, std::integral_constant<int, 2>{});
        advance();
        step(it + 3, c, cp, zc, std::integral_constant<int, 3>{});
        advance();
        if constexpr (P == 4) zc ^= 1;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the last two steps' loads ran ahead of the range
    gemm_tail<MI>(acc, Y, M, N, m0, n0, epi, part, counters, reinterpret_cast<float*>(lds));
}

constexpr int GEMM_COUNTER_BYTES = 65536;  // start of the workspace: one uint32 per output tile

template <int MI>
static hipError_t launch_mi(const void* x, const void* w, const void* zs, void* y, int M, int N, int K, int gshift,
                            Epilogue epi, void* ws, int ksplit, bool lds, hipStream_t st) {
    const dim3 grid((N + GEMM_BN - 1) / GEMM_BN, (M + 32 * MI - 1) / (32 * MI), ksplit);
    unsigned* counters = (unsigned*)ws;
    float* part = ws ? (float*)((char*)ws + GEMM_COUNTER_BYTES) : nullptr;
    // the LDS kernel addresses its operands with 32-bit byte offsets per lane
    const bool fits32 = (long)M * K * 2 < (1L << 32) && (long)N * (K / 2) < (1L << 32);
    if (lds && gshift >= 5 && gshift <= 7 && K % 256 == 0 && fits32) {
        if (gshift == 7)
            hipLaunchKernelGGL((gemm_lds_kernel<MI, 7>), grid, dim3(256), 0, st, (const uint8_t*)w, (const half2_t*)zs,
                               (const half_t*)x, (half_t*)y, M, N, K, epi, part, counters);
        else if (gshift == 6)
            hipLaunchKernelGGL((gemm_lds_kernel<MI, 6>), grid, dim3(256), 0, st, (const uint8_t*)w, (const half2_t*)zs,
                               (const half_t*)x, (half_t*)y, M, N, K, epi, part, counters);
        else
            hipLaunchKernelGGL((gemm_lds_kernel<MI, 5>), grid, dim3(256), 0, st, (const uint8_t*)w, (const half2_t*)zs,
                               (const half_t*)x, (half_t*)y, M, N, K, epi, part, counters);
        return hipGetLastError();
    }
    hipLaunchKernelGGL((gemm_kernel<MI>), grid, dim3(256), 0, st, (const uint8_t*)w, (const half2_t*)zs,
                       (const half_t*)x, (half_t*)y, M, N, K, gshift, epi, part, counters);
    return hipGetLastError();
}

// Tile height and K split for a shape (shared by the launcher and the workspace query).
// Measured on MI355X: large M wants the tallest tile whose grid fills the 256 CUs (fewer
// unpack instructions per flop); when even 64-row tiles give fewer than 256 workgroups and a
// workspace is at hand, 64-row tiles (32-row when those are too few) with K split so that
// the grid reaches about 256 workgroups (4096 x 16384 at M = 128: 47 us against 163 us
// unsplit).  `pipe` receives the pipelined variant to use instead (-1 = none).
struct GemmPlan {
    int mi, ksplit, pipe;
    int lds = 0;  // 1: gemm_lds_kernel (group size 32, 64 or 128, K a multiple of 256)
};
// Group size 32, 64 or 128 with K a multiple of 256 and more than 16 tokens: gemm_lds_kernel; tile height and K
// split come from the cost model below.  Only a long K whose 256 x 256 tiles fill whole rounds stays with the
// pipelined kernel (4096 x 16384 at 4096 tokens: 497 against 530 us); at group size 32, where this kernel refills
// its zeros/scales every step, any K does (fc1 at 2048 tokens: 285 against 302 us).
static GemmPlan plan_gemm_lds(int M, long ncol, int nit, int g, bool have_ws) {
    GemmPlan p = {1, 1, -1};
    const long t256 = ncol * ((M + 255) / 256);
    const long rounds = (t256 + 255) / 256;
    if (M > 1024 && (nit >= 128 || g == 32) && t256 * 10 >= rounds * 256 * 9) {
        p.pipe = 2;
        return p;
    }
    p.lds = 1;
    // Tile height (32 mi rows) and K split by a cost model fitted to timings of all twelve combinations on 17 weights
    // x 7 token counts (48..2048 tokens; 768 x 3072 to 8192 x 28672): a workgroup alone on its CU takes
    // a1[mi] us per K step, one that shares its CU a2[mi] (two fit), plus b[mi] per workgroup; W workgroups run in
    // rounds of 512; a K split adds the exchange of the partial tiles.  The model's choice is within 1 % of the best
    // combination in the geometric mean over those 119 points (worst case 12 %); the rule it replaces (tile height by
    // token count, K split only below 128 tiles) was within 5 % (worst 81 %: 1024 x 1024 at 2048 tokens ran 64
    // workgroups).
    static const float a1[3] = {0.456f, 0.528f, 0.821f}, a2[3] = {0.965f, 1.275f, 1.992f}, b[3] = {3.49f, 4.53f, 5.77f};
    float best = 3.4e38f;
    for (int i = 0; i < 3; i++) {
        const int mi = 1 << i;
        const long t = ncol * ((M + 32 * mi - 1) / (32 * mi));
        for (int ks = 1; ks <= 8; ks *= 2) {
            if (ks > 1 && (!have_ws || t > 16384 || nit / ks < 4 || t * ks * (32 * mi) * 256 * 4 > (256L << 20))) break;
            const long W = t * ks;
            const int steps = ((nit + ks - 1) / ks + 3) & ~3;
            const float t1 = a1[i] * steps + b[i], t2 = a2[i] * steps + b[i];
            float cost;
            if (W <= 256) {
                cost = t1;
            } else if (W <= 512) {
                cost = t2;
            } else {
                const long full = W / 512, rem = W - full * 512;
                cost = full * t2 + (rem == 0 ? 0.f : (rem > 256 ? t2 : t1));
            }
            if (ks > 1) cost += 1.3f + 2.56f * mi;
            if (cost < best) {
                best = cost;
                p.mi = mi;
                p.ksplit = ks;
            }
        }
    }
    return p;
}

static GemmPlan plan_gemm(int M, int N, int K, int g, bool have_ws) {
    GemmPlan p = {1, 1, -1};
    const long ncol = (N + 255) / 256;
    auto ntiles = [&](int rows) { return ncol * ((M + rows - 1) / rows); };
    const long t256 = ntiles(256);
    const long rounds = (t256 + 255) / 256;
    const int nit = (K + GEMM_BK - 1) / GEMM_BK;
    if ((g == 128 || g == 64 || g == 32) && K % 256 == 0 && M > 16) return plan_gemm_lds(M, ncol, nit, g, have_ws);
    if (M > 64 && t256 * 10 >= rounds * 256 * 6) {
        p.pipe = 2;  // 256 x 256 tiles pay from about 60 % of the CUs (5120 x 13696 at M = 2048: 338 us against 390 us)
    } else if (M > 64 && ntiles(128) >= 160) {
        if (K >= 8192) p.pipe = 1;
        p.mi = 4;
    } else if (have_ws && M > 32 && ntiles(64) < 256 && ntiles(32) <= 16384) {
        p.mi = (ntiles(64) * 8 < 256 || (ntiles(64) * 8 == 256 && K <= 8192)) ? 1 : 2;
        const long t = ntiles(32 * p.mi);
        while (p.ksplit < 8 && t * p.ksplit * 2 <= 256 && nit / (p.ksplit * 2) >= 8) p.ksplit *= 2;
        if (p.ksplit == 1 && K >= 12288 && ntiles(128) * 4 <= 512) p = {4, 4, -1};
    } else if (have_ws && M > 64 && K >= 12288 && ntiles(128) * 4 <= 512) {
        // Long K with a grid between one and two rounds of 64-row tiles: 128-row tiles with K
        // split four ways even out the rounds (4096 x 16384 at M = 1024: 185 us against 207 us).
        p = {4, 4, -1};
    } else if (M > 32 && ntiles(64) >= 160) {
        p.mi = 2;
    } else {
        p.mi = 1;
    }
    return p;
}

static size_t plan_bytes(const GemmPlan& p, int M, int N) {
    if (p.ksplit == 1) return 0;
    const long tiles = (long)((N + 255) / 256) * ((M + 32 * p.mi - 1) / (32 * p.mi));
    return (size_t)GEMM_COUNTER_BYTES + (size_t)p.ksplit * tiles * (32 * p.mi) * 256 * sizeof(float);
}

// The query does not know the group size: the larger of what the two planners would use.
size_t gemm_workspace_bytes(int M, int N, int K) {
    const size_t a = plan_bytes(plan_gemm(M, N, K, 128, true), M, N);
    const size_t b = plan_bytes(plan_gemm(M, N, K, 0, true), M, N);
    return a > b ? a : b;
}

// tune = 0 for the heuristic, else the number of 32-row tiles per workgroup (1, 2 or 4) | ksplit << 8
// (needs ws) | 0x80 for the kernel with both operands through LDS (group size 32..128, K % 256 == 0), or 8 / 9 / 10 for the software-pipelined kernel (128 rows at two waves per SIMD, 128 rows
// at one, 256 rows at one).  ws = null or too small: K is never split.
hipError_t launch_gemm_tuned(const void* x, const void* w, const void* zs, void* y, void* ws, size_t ws_bytes, int M,
                             int N, int K, int g, int tune, Epilogue epi, hipStream_t st) {
    int gshift = 0;
    while ((1 << gshift) < g) gshift++;
    int mi = tune & 0x3F;
    int ksplit = (tune >> 8) & 0xFF;
    bool lds = (tune & 0x80) != 0;
    if (mi >= 8 && mi <= 10) return launch_gemm_pipe(x, w, zs, y, M, N, K, g, mi - 8, epi, st);
    if (mi != 1 && mi != 2 && mi != 4) {
        const bool have_ws = ws != nullptr && ws_bytes >= plan_bytes(plan_gemm(M, N, K, g, true), M, N);
        const GemmPlan p = plan_gemm(M, N, K, g, have_ws);
        if (p.pipe >= 0) return launch_gemm_pipe(x, w, zs, y, M, N, K, g, p.pipe, epi, st);
        mi = p.mi;
        ksplit = p.ksplit;
        lds = p.lds != 0;
    } else {
        if (ksplit != 2 && ksplit != 4 && ksplit != 8) ksplit = 1;
        const long tiles = (long)((N + 255) / 256) * ((M + 32 * mi - 1) / (32 * mi));
        const size_t need = (size_t)GEMM_COUNTER_BYTES + (size_t)ksplit * tiles * (32 * mi) * 256 * sizeof(float);
        if (ksplit > 1 && (!ws || ws_bytes < need || tiles > 16384)) ksplit = 1;
    }
    switch (mi) {
        case 1: return launch_mi<1>(x, w, zs, y, M, N, K, gshift, epi, ws, ksplit, lds, st);
        case 2: return launch_mi<2>(x, w, zs, y, M, N, K, gshift, epi, ws, ksplit, lds, st);
        default: return launch_mi<4>(x, w, zs, y, M, N, K, gshift, epi, ws, ksplit, lds, st);
    }
}

}  // namespace sq
