// Skinny GEMM for 5 <= M <= 32 with a caller-provided workspace (layout L1).
// HBM-bound on the weight stream; everything else is arranged so that the vector
// memory pipeline sees little besides that stream.
//
// Mapping.  v_mfma_f32_16x16x32_f16 with the weights as the B operand straight
// from registers (lane l: row r + l%16, k = 128c + 32*(l/16) .. +31, one 128-bit
// load, one 32-bit word per MFMA) and the activations as the A operand (token
// l%16, the same k).  A workgroup owns 64 weight rows and one of `ksplit` K ranges;
// its waves take pairs of 128-wide chunks of that range round-robin, and every wave
// reuses one set of activation registers for the four 16-row tiles of the 64 rows.
//
// Activations: a lane needs 64 contiguous bytes of one token per chunk, which as a
// direct load touches one cache line per lane.  Instead each wave loads its chunk
// row-contiguously (16 lanes x 16 bytes = the 256 bytes of one token) and turns it
// into operand order through a wave-private LDS buffer (pitch 272 bytes: both the
// row-contiguous writes and the operand-order reads are bank-conflict free).
// Zeros/scales of the workgroup's rows and K range are staged in LDS once, with
// row-contiguous loads, when they fit (32 groups per row); otherwise lanes fetch
// them per chunk.
//
// Partial 16x16 tiles are summed across the waves in LDS.  With ksplit > 1 each
// workgroup writes its fp32 partial tile to the workspace and bumps a per-row-block
// counter; the workgroup that arrives last adds the partials in a fixed order
// (bit-reproducible), writes Y and resets the counter.
//
// Arithmetic modes as in the GEMV kernel: exact (per-weight fp16 (q-z)*s, any group
// size) and, for g == 128 (one group per chunk), fixup: 64+q into the matrix core
// and s*(acc - (64+z)*sum_x) per chunk in fp32.
#include "sq_common.h"
#include "sq_kernels.h"

namespace sq {

constexpr int SK2_COUNTER_BYTES = 65536;  // start of the workspace: one uint32 per 64-row block
constexpr int SK2_XPITCH = 272;           // bytes per staged token row (256 + 16)
constexpr int SK2_ZCOLS = 32;             // groups per row held in LDS
constexpr int SK2_ZPITCH = 33;

__device__ __forceinline__ void wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// rb = row block inside this linear; slot = index of the row block in the workspace (counter and partial
// tiles), which differs from rb when several linears share a launch.
template <int MT, int NWV, int S, int RT, bool FIXUP>
__device__ __forceinline__ void skinny2_body(const uint8_t* __restrict__ W, const half2_t* __restrict__ ZS,
                                             const half_t* __restrict__ X, half_t* __restrict__ Y, float* part,
                                             unsigned* counters, int M, int N, int K, int gshift, int ksplit,
                                             const Epilogue& epi, int rb, int slot, int nslots) {
    constexpr int TILE = RT * MT * 4 * 64;  // floats a wave contributes: [rt][mt][v][lane]
    constexpr int ROWS = 16 * RT;           // weight rows per workgroup
    constexpr int XBUF = MT * 16 * SK2_XPITCH;
    constexpr int SH_BYTES = NWV * XBUF > NWV * TILE * 4 ? NWV * XBUF : NWV * TILE * 4;
    __shared__ __attribute__((aligned(16))) uint8_t sh[SH_BYTES];  // activation staging, later the wave partials
    __shared__ uint32_t zsl[ROWS * SK2_ZPITCH];
    __shared__ unsigned last_flag;
    float* red = (float*)sh;

    const NibbleMasks nm = nibble_masks();
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int li = lane & 15;
    const int lj = lane >> 4;
    const int ks = blockIdx.y;
    const int groups = K >> gshift;
    const int nchunks = (K + 127) >> 7;
    const int cps = (nchunks + ksplit - 1) / ksplit;
    const int c_begin = ks * cps;
    const int c_end = imin(c_begin + cps, nchunks);
    const int gpc_shift = 7 - gshift;  // groups per chunk = 1 << gpc_shift
    const int g_begin = c_begin << gpc_shift;
    const int ng = imin((c_end - c_begin) << gpc_shift, groups - g_begin);
    const bool zs_lds = ng > 0 && ng <= SK2_ZCOLS;

    // Zeros/scales of the row block: loaded now (row-contiguous), parked in LDS after the
    // first weight loads have been issued so that they do not delay the weight stream.
    constexpr int ZPT = (ROWS * SK2_ZCOLS) / (64 * NWV);
    uint32_t zreg[ZPT];
    if (zs_lds) {
#pragma unroll
        for (int p = 0; p < ZPT; p++) {
            const int idx = tid + p * 64 * NWV;
            const int r = idx >> 5, col = idx & 31;
            const int row = imin(rb * ROWS + r, N - 1);
            zreg[p] = ((const uint32_t*)ZS)[(long)row * groups + g_begin + (col < ng ? col : 0)];
        }
    }

    float4_t acc[RT][MT];
#pragma unroll
    for (int rt = 0; rt < RT; rt++)
#pragma unroll
        for (int mt = 0; mt < MT; mt++) acc[rt][mt] = (float4_t){0.f, 0.f, 0.f, 0.f};
    const half8_t ones = {(half_t)1.f, (half_t)1.f, (half_t)1.f, (half_t)1.f,
                          (half_t)1.f, (half_t)1.f, (half_t)1.f, (half_t)1.f};

    const uint8_t* wrow[RT];
    const uint32_t* zrow[RT];
#pragma unroll
    for (int rt = 0; rt < RT; rt++) {
        const int row = imin(rb * ROWS + 16 * rt + li, N - 1);
        wrow[rt] = W + (long)row * (K >> 1);
        zrow[rt] = (const uint32_t*)ZS + (long)row * groups;
    }
    uint8_t* xb = sh + wave * XBUF;
    uint8_t* xb_wr = xb + (lane >> 4) * SK2_XPITCH + (lane & 15) * 16;  // token lane/16 (+4j), 16-byte column lane%16
    const uint8_t* xb_rd = xb + li * SK2_XPITCH + lj * 64;              // token li (+16mt), k = 32 lj (+8t)

    // S chunks per wave and trip; every weight load of the trip is issued before the first
    // use, the activations run one chunk ahead.  The trip count is uniform over the waves
    // (the zeros/scales hand-over contains a barrier); a wave without chunks idles.
    bool first = true;
    for (int cb = c_begin; cb < c_end; cb += S * NWV) {
        const int c0 = cb + S * wave;
        const bool active = c0 < c_end;
        u32x4_t wq[S][RT];
        u32x4_t xr[2][4 * MT];
        uint32_t zq[S][RT];
        int zcol[S];
        auto load_x = [&](int c, u32x4_t* dst) {
            const int kx = (c << 7) + 8 * (lane & 15);
            const bool xvalid = (c < c_end) && (kx < K);
#pragma unroll
            for (int j = 0; j < 4 * MT; j++) {
                const int tok = imin(4 * j + (lane >> 4), M - 1);
                const u32x4_t v = *(const u32x4_t*)(X + (long)tok * K + (xvalid ? kx : 0));
                dst[j] = xvalid ? v : (u32x4_t){0u, 0u, 0u, 0u};
            }
        };
        if (active) {
            // (cache-allocating loads, the S chunks of a row back to back: consecutive chunks
            // share a 128-byte line, which is then requested from L2 once instead of per chunk)
            int kcs[S];
#pragma unroll
            for (int u = 0; u < S; u++) {
                const int kk = ((c0 + u) << 7) + 32 * lj;
                kcs[u] = ((c0 + u < c_end) && (kk < K)) ? kk : 0;
            }
#pragma unroll
            for (int rt = 0; rt < RT; rt++)
#pragma unroll
                for (int u = 0; u < S; u++) wq[u][rt] = *(const u32x4_t*)(wrow[rt] + (kcs[u] >> 1));
#pragma unroll
            for (int u = 0; u < S; u++) {
                const int c = c0 + u;
                const int kk = (c << 7) + 32 * lj;
                const bool valid = (c < c_end) && (kk < K);
                zcol[u] = valid ? (((c - c_begin) << gpc_shift) + ((32 * lj) >> gshift)) : 0;
                if (!zs_lds) {
#pragma unroll
                    for (int rt = 0; rt < RT; rt++) zq[u][rt] = zrow[rt][valid ? (kk >> gshift) : g_begin];
                }
            }
            load_x(c0, xr[0]);
        }
        if (first) {
            if (zs_lds) {
#pragma unroll
                for (int p = 0; p < ZPT; p++) {
                    const int idx = tid + p * 64 * NWV;
                    zsl[(idx >> 5) * SK2_ZPITCH + (idx & 31)] = zreg[p];
                }
            }
            __syncthreads();
            first = false;
        }
        if (active) {
#pragma unroll
            for (int u = 0; u < S; u++) {
                if (u + 1 < S) load_x(c0 + u + 1, xr[(u + 1) & 1]);
                wave_lds_sync();  // the previous chunk's operand reads are done
#pragma unroll
                for (int j = 0; j < 4 * MT; j++) *(u32x4_t*)(xb_wr + 4 * j * SK2_XPITCH) = xr[u & 1][j];
                wave_lds_sync();
                u32x4_t xa[MT][4];
#pragma unroll
                for (int mt = 0; mt < MT; mt++)
#pragma unroll
                    for (int t = 0; t < 4; t++) xa[mt][t] = *(const u32x4_t*)(xb_rd + 16 * mt * SK2_XPITCH + 16 * t);
                if (zs_lds) {
#pragma unroll
                    for (int rt = 0; rt < RT; rt++) zq[u][rt] = zsl[(16 * rt + li) * SK2_ZPITCH + zcol[u]];
                }
                float4_t xs[MT];
                if (FIXUP) {
#pragma unroll
                    for (int mt = 0; mt < MT; mt++) {
                        xs[mt] = (float4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
                        for (int t = 0; t < 4; t++)
                            xs[mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(bit_cast<half8_t>(xa[mt][t]), ones, xs[mt], 0,
                                                                            0, 0);
                    }
                }
#pragma unroll
                for (int rt = 0; rt < RT; rt++) {
                    const half2_t zsv = bit_cast<half2_t>(zq[u][rt]);
                    if (!FIXUP) {
                        const half2_t z64 = {zsv.x, zsv.x};
                        const half2_t sc = {zsv.y, zsv.y};
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
                                tmp[mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(bit_cast<half8_t>(xa[mt][t]), wv,
                                                                                 tmp[mt], 0, 0, 0);
                        }
                        const float zf = (float)zsv.x;
                        const float sf = (float)zsv.y;
#pragma unroll
                        for (int mt = 0; mt < MT; mt++)
#pragma unroll
                            for (int v = 0; v < 4; v++) acc[rt][mt][v] += sf * (tmp[mt][v] - zf * xs[mt][v]);
                    }
                }
            }
        }
    }
    __syncthreads();  // every wave is done with its staging buffer, which the partials now overwrite

    // Sum the waves' partial tiles: red[wave][rt][mt][v][lane].
#pragma unroll
    for (int rt = 0; rt < RT; rt++)
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
            const int n = rb * ROWS + 16 * rt + (l & 15);
            if (m < M && n < N) Y[(long)m * N + n] = epilogue(sum, m, n, N, epi);
        }
        return;
    }
    // Cross-workgroup exchange.  The partial tiles travel as agent-scope relaxed atomic
    // stores and loads, which go to the device-coherent level directly, so no device-wide
    // release/acquire fence (which would write back and invalidate the whole L2) is needed:
    // the wait for outstanding vector memory operations orders the partial stores before
    // the counter increment, and the last arriver reads the partials past its own caches.
    // (128-bit accesses with the same cache policy bit the compiler gives those atomics: the
    // exchange is bound by the number of requests, not by bytes.)
    float* mine = part + ((long)ks * nslots + slot) * TILE;
    for (int t4 = tid * 4; t4 < TILE; t4 += 4 * 64 * NWV) {
        float4_t sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int p = 0; p < NWV; p++) sum += *(const float4_t*)(&red[p * TILE + t4]);
        store_coherent_x4(mine + t4, sum);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0) {
        const unsigned old = __hip_atomic_fetch_add(&counters[slot], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        last_flag = (old == (unsigned)(ksplit - 1)) ? 1u : 0u;
    }
    __syncthreads();
    if (!last_flag) return;
    const bool fast_tail = tail4_applies(epi);
    for (int t4 = tid * 4; t4 < TILE; t4 += 4 * 64 * NWV) {
        // the four elements t4 .. t4 + 3 are one token and four consecutive rows of the weight; their bias and
        // residual are requested ahead of the partial tiles
        const int l4 = t4 & 63, v4 = (t4 >> 6) & 3, mt4 = (t4 >> 8) % MT, rt4 = (t4 >> 8) / MT;
        const int m4 = 16 * mt4 + 4 * (l4 >> 4) + v4;
        const int n4 = rb * ROWS + 16 * rt4 + (l4 & 15);
        const bool inside = m4 < M && n4 < N;
        Tail4 pre = {{0u, 0u}, {0u, 0u}};
        if (fast_tail) pre = tail4_request(epi, m4, n4, N, inside);
        // eight loads regardless of ksplit (absent partials re-read partial 0 and are dropped)
        const float* src[8];
#pragma unroll
        for (int q = 0; q < 8; q++) src[q] = part + ((long)(q < ksplit ? q : 0) * nslots + slot) * TILE + t4;
        float4_t pv[8];
        load8_coherent_x4(src, pv);
        float4_t sum = pv[0];
#pragma unroll
        for (int q = 1; q < 8; q++)
            if (q < ksplit) sum += pv[q];  // fixed order
        if (fast_tail) {
            if (inside) tail4_store(sum, pre, Y, m4, n4, N, epi);
            continue;
        }
#pragma unroll
        for (int e = 0; e < 4; e++)
            if (inside) Y[(long)m4 * N + n4 + e] = epilogue(sum[e], m4, n4 + e, N, epi);
    }
    // leave the workspace ready for the next call
    if (tid == 0) __hip_atomic_store(&counters[slot], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <int MT, int NWV, int S, int RT, bool FIXUP>
__global__ __launch_bounds__(64 * NWV) void skinny2_kernel(const uint8_t* __restrict__ W,
                                                           const half2_t* __restrict__ ZS,
                                                           const half_t* __restrict__ X, half_t* __restrict__ Y,
                                                           float* part, unsigned* counters, int M, int N, int K,
                                                           int gshift, int ksplit, Epilogue epi) {
    skinny2_body<MT, NWV, S, RT, FIXUP>(W, ZS, X, Y, part, counters, M, N, K, gshift, ksplit, epi, blockIdx.x, blockIdx.x,
                                        gridDim.x);
}

// Up to four linears that do not depend on each other and share M, K and the group size in one launch: the
// grid's x dimension is the concatenation of their 64-row blocks.
struct Skinny2Group {
    const uint8_t* W[GEMV_GROUP_MAX];
    const half2_t* ZS[GEMV_GROUP_MAX];
    const half_t* X[GEMV_GROUP_MAX];
    half_t* Y[GEMV_GROUP_MAX];
    const half_t* bias[GEMV_GROUP_MAX];
    const half_t* residual[GEMV_GROUP_MAX];
    int N[GEMV_GROUP_MAX];
    int act[GEMV_GROUP_MAX];
    int blk_end[GEMV_GROUP_MAX];  // first row block behind linear p
    int count;
};

template <int MT, int NWV, int S, int RT, bool FIXUP>
__global__ __launch_bounds__(64 * NWV) void skinny2_group_kernel(const Skinny2Group grp, float* part, unsigned* counters,
                                                                 int M, int K, int gshift, int ksplit) {
    int p = 0;
#pragma unroll
    for (int q = 0; q < GEMV_GROUP_MAX - 1; q++)
        if (q + 1 < grp.count && (int)blockIdx.x >= grp.blk_end[q]) p = q + 1;
    const int rb = blockIdx.x - (p > 0 ? grp.blk_end[p - 1] : 0);
    const Epilogue epi{grp.bias[p], grp.residual[p], grp.act[p]};
    skinny2_body<MT, NWV, S, RT, FIXUP>(grp.W[p], grp.ZS[p], grp.X[p], grp.Y[p], part, counters, M, grp.N[p], K, gshift,
                                        ksplit, epi, rb, blockIdx.x, gridDim.x);
}

size_t skinny2_workspace_bytes(int M, int N, int K) {
    const int mt = (M + 15) / 16;
    const int row_blocks = (N + 63) / 64;
    return (size_t)SK2_COUNTER_BYTES + (size_t)8 * row_blocks * (4 * mt * 4 * 64) * sizeof(float);
}

template <int MT, int NWV, int S, int RT>
static hipError_t launch_cfg(const void* x, const void* w, const void* zs, void* y, void* ws, int M, int N, int K,
                             int gshift, bool fixup, int ksplit, Epilogue epi, hipStream_t st) {
    const dim3 grid((N + 16 * RT - 1) / (16 * RT), ksplit);
    unsigned* counters = (unsigned*)ws;
    float* part = (float*)((char*)ws + SK2_COUNTER_BYTES);
    if (fixup)
        hipLaunchKernelGGL((skinny2_kernel<MT, NWV, S, RT, true>), grid, dim3(64 * NWV), 0, st, (const uint8_t*)w,
                           (const half2_t*)zs, (const half_t*)x, (half_t*)y, part, counters, M, N, K, gshift, ksplit, epi);
    else
        hipLaunchKernelGGL((skinny2_kernel<MT, NWV, S, RT, false>), grid, dim3(64 * NWV), 0, st, (const uint8_t*)w,
                           (const half2_t*)zs, (const half_t*)x, (half_t*)y, part, counters, M, N, K, gshift, ksplit, epi);
    return hipGetLastError();
}

// tune = 0 for the heuristic, else ksplit (1,2,4,8) | mode << 8 (1 = exact, 2 = fixup) |
// waves << 12 (4, 8).
// The first 64 KiB of the workspace are counters and must be zero before the first call;
// every call leaves them zero.
hipError_t launch_skinny2_tuned(const void* x, const void* w, const void* zs, void* y, void* ws, int M, int N, int K,
                                int g, int tune, Epilogue epi, hipStream_t st) {
    int gshift = 0;
    while ((1 << gshift) < g) gshift++;
    const int mt = (M + 15) / 16;
    const int nchunks = (K + 127) / 128;
    int ksplit = tune & 0xFF;
    int nwv = (tune >> 12) & 0xF;
    // Four 16-row tiles per wave (64 rows per workgroup); eight were measured and are slower:
    // the registers they need leave one wave per SIMD.
    const int row_blocks = (N + 63) / 64;
    if (ksplit != 1 && ksplit != 2 && ksplit != 4 && ksplit != 8) {
        // At most one workgroup per CU (a second round of workgroups costs more than idle CUs:
        // 12288 rows run 11.5 us as 192 workgroups, 16.5 us as 384), each K range at least 8
        // chunks long.
        ksplit = 1;
        while (ksplit < 8 && row_blocks * ksplit * 2 <= 256 && nchunks / (ksplit * 2) >= 8) ksplit *= 2;
    }
    const int cps = (nchunks + ksplit - 1) / ksplit;
    // Eight waves (two per SIMD, one computing while the other waits for memory) whenever a wave
    // still gets two chunks, and always with 17..32 tokens, where a single wave per SIMD ran
    // 16384 x 4096 in 19.6 us against 16.3 us.
    if (nwv != 4 && nwv != 8) nwv = (mt == 2 || cps >= 16) ? 8 : 4;
    const int mode = (tune >> 8) & 0xF;
    bool fixup = (g == 128);
    if (mode == 1) fixup = false;
    if (mt == 2 && nwv == 8) return launch_cfg<2, 8, 2, 4>(x, w, zs, y, ws, M, N, K, gshift, fixup, ksplit, epi, st);
    if (mt == 2) return launch_cfg<2, 4, 2, 4>(x, w, zs, y, ws, M, N, K, gshift, fixup, ksplit, epi, st);
    if (nwv == 8) return launch_cfg<1, 8, 2, 4>(x, w, zs, y, ws, M, N, K, gshift, fixup, ksplit, epi, st);
    return launch_cfg<1, 4, 2, 4>(x, w, zs, y, ws, M, N, K, gshift, fixup, ksplit, epi, st);
}

template <int MT, int NWV>
static hipError_t launch_group_cfg(const SeqProblem* probs, int count, void* ws, int M, int K, int gshift, int ksplit,
                                   hipStream_t st) {
    Skinny2Group g;
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
        if (p < count) blocks += (q.N + 63) / 64;
        g.blk_end[p] = blocks;
    }
    g.count = count;
    unsigned* counters = (unsigned*)ws;
    float* part = (float*)((char*)ws + SK2_COUNTER_BYTES);
    hipLaunchKernelGGL((skinny2_group_kernel<MT, NWV, 2, 4, true>), dim3(blocks, ksplit), dim3(64 * NWV), 0, st, g, part,
                       counters, M, K, gshift, ksplit);
    return hipGetLastError();
}

// Workspace for a grouped launch: as for one linear whose N is the sum of the group's (rounded up to 64 each).
size_t skinny2_group_workspace_bytes(const SeqProblem* probs, int count, int M) {
    int rows = 0;
    for (int p = 0; p < count; p++) rows += ((probs[p].N + 63) / 64) * 64;
    return skinny2_workspace_bytes(M, rows, probs[0].K);
}

// Grouped launch (fixup arithmetic, group size 128): count in 2..GEMV_GROUP_MAX linears with the same K and
// group size, 5 <= M <= 32.  hipErrorInvalidValue when the group does not qualify.
hipError_t launch_skinny2_group(const SeqProblem* probs, int count, int M, void* ws, size_t ws_bytes, hipStream_t st) {
    if (count < 2 || count > GEMV_GROUP_MAX || M < 5 || M > 32 || !ws) return hipErrorInvalidValue;
    const int K = probs[0].K;
    if (probs[0].group_size != 128) return hipErrorInvalidValue;
    for (int p = 1; p < count; p++)
        if (probs[p].K != K || probs[p].group_size != 128) return hipErrorInvalidValue;
    int row_blocks = 0;
    for (int p = 0; p < count; p++) row_blocks += (probs[p].N + 63) / 64;
    if (row_blocks > 16384 || ws_bytes < skinny2_group_workspace_bytes(probs, count, M)) return hipErrorInvalidValue;
    const int mt = (M + 15) / 16;
    const int nchunks = (K + 127) / 128;
    int ksplit = 1;  // same rule as for one linear with all the rows
    while (ksplit < 8 && row_blocks * ksplit * 2 <= 256 && nchunks / (ksplit * 2) >= 8) ksplit *= 2;
    const int cps = (nchunks + ksplit - 1) / ksplit;
    const int nwv = (mt == 2 || cps >= 16) ? 8 : 4;
    if (mt == 2 && nwv == 8) return launch_group_cfg<2, 8>(probs, count, ws, M, K, 7, ksplit, st);
    if (mt == 2) return launch_group_cfg<2, 4>(probs, count, ws, M, K, 7, ksplit, st);
    if (nwv == 8) return launch_group_cfg<1, 8>(probs, count, ws, M, K, 7, ksplit, st);
    return launch_group_cfg<1, 4>(probs, count, ws, M, K, 7, ksplit, st);
}

}  // namespace sq
