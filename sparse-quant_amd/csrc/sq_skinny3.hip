// Streaming skinny GEMM for up to 32 tokens, group size 128 (64 up to 16 tokens), layout L1: the decode kernel for
// small batches.
//
// The matrix instruction, the operand mapping and the per-chunk arithmetic are those of the split-K
// decode kernel in sq_skinny2.hip (v_mfma_f32_16x16x32_f16, weights as the B operand straight from
// registers, per 128-wide chunk s * (acc - (64 + z) * sum_x) in fp32), with the shift-free unpack of the
// GEMV (1024 + q on four of every eight positions; the chunk's accumulator starts at -960 * the sum of x
// over those positions, itself one more matrix instruction, so the extra bias costs no vector arithmetic).
// What differs is the order of memory operations, which is what bounds this regime.  Measured with time
// stamps inside the kernel (fc1 of OPT-6.7B, 8 tokens), the split-K kernel spends its time in two serial
// trips of "request, wait for everything, compute"; here:
//
//   * A workgroup (eight waves) owns 16 * RT weight rows and one K range of at most 8 * CH chunks.  Its
//     zeros/scales and ALL activations of that range are requested first; a bare s_barrier makes sure every
//     wave has done so before any wave requests weights (a CU serves its vector memory requests in order).
//   * The weights go out in units of four loads (two row tiles x the two 64-byte halves of a 128-byte line),
//     one unit ahead of the one being consumed.  A CU accepts only a few dozen such requests; a wave that
//     issues into a full queue stalls at that instruction, and a wave that has requested all its weights up
//     front reaches the parking of the activations only when most of the stream has arrived (first
//     arithmetic 5.3 us after launch instead of 1.9 us).
//   * The activations are parked in LDS (row-major per token, pitch = 16 mod 256 bytes: the operand-order
//     reads of 16 lanes fall into 16 different 16-byte slots).  The vector memory counter retires in order,
//     so waiting for them leaves the first weight unit in flight.
//   * Barriers are s_waitcnt lgkmcnt(0) + s_barrier, not __syncthreads(): the latter also waits for every
//     outstanding vector memory load.
//   * The main part is straight-line code (no loop, no branch), each request pinned in place by a
//     scheduling barrier; a chunk slot beyond the K range reads a valid address and meets zero activations.
//
// Partial tiles of the eight waves meet in LDS; with ksplit > 1 the workgroups of a row block exchange
// fp32 partial tiles through the workspace exactly as the split-K decode kernel does (same layout, same
// counters: a workspace sized for that kernel serves this one).
// (replaces w4a16_gemm_wmma_kernel for small batches, reference:
// quantization/muxi/backend/w4a16_gemm.cuh:466-600)
#include "sq_common.h"
#include "sq_kernels.h"

namespace sq {

namespace {

constexpr int SK3_COUNTER_BYTES = 65536;  // start of the workspace: one uint32 per row block
constexpr int SK3_NWV = 8;
constexpr int SK3_NT = 64 * SK3_NWV;
// Units of weight loads requested before the activations are parked, and ahead of the unit being consumed (two
// and three were measured: a wave that issues into a full memory queue stalls before it reaches the parking stores).
constexpr int SK3_DEPTH_PRE = 1;
constexpr int SK3_DEPTH = 1;

template <int MROWS, int RT, int CH, int GPC = 1>
struct Sk3Lds {
    static constexpr int ZPITCH = 32 * GPC + 1;          // (zero, scale) pairs per staged row: GPC per chunk slot
    static constexpr int CHUNKS = SK3_NWV * CH;          // chunk slots of a workgroup
    static constexpr int XPITCH = CHUNKS * 256 + 16;     // bytes per staged token row
    static constexpr int X_BYTES = MROWS * XPITCH;
    static constexpr int TILE = RT * 4 * 64;             // floats a wave contributes: [rt][v][lane]
    static constexpr int RED_BYTES = SK3_NWV * TILE * 4;
    static constexpr int Z_OFF = X_BYTES > RED_BYTES ? X_BYTES : RED_BYTES;  // the partials reuse the activations' space
    static constexpr int FLAG_OFF = Z_OFF + 16 * RT * ZPITCH * 4;
    static constexpr int LN_OFF = FLAG_OFF + 16;         // fused LayerNorm: mean and reciprocal deviation per token
    static constexpr int BYTES = LN_OFF + 2 * MROWS * 4;
};

__device__ __forceinline__ void sk3_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// rb = row block inside this linear; slot = index of the row block in the workspace, which differs from
// rb when several linears share a launch.
// GPC = groups per 128-wide chunk: 1 (group size 128: zero and scale applied per chunk in fp32) or 2 (group size 64:
// per-weight dequantisation in fp16, as the reference computes W_hat).
template <int MROWS, int RT, int CH, int DEPTH, bool LN, int GPC>
__device__ __forceinline__ void skinny3_body(const uint8_t* __restrict__ W, const uint32_t* __restrict__ ZS,
                                             const half_t* __restrict__ X, half_t* __restrict__ Y, float* part,
                                             unsigned* counters, int M, int N, int K, int ksplit, const Epilogue& epi,
                                             const LnPre& ln, int rb, int slot, int nslots) {
    using L = Sk3Lds<MROWS, RT, CH, GPC>;
    constexpr int ROWS = 16 * RT;
    constexpr int ZW = 32 * GPC;  // staged (zero, scale) pairs per row
    constexpr int TILE = L::TILE;
    constexpr int WPR = L::CHUNKS * 16;  // 128-bit words per staged token row
    constexpr int XPT = MROWS * WPR / SK3_NT;
    constexpr int ZPT = (ROWS * ZW + SK3_NT - 1) / SK3_NT;
    static_assert(CH == 1 || CH == 2 || CH == 4, "chunk slots per wave");
    static_assert(MROWS * WPR % SK3_NT == 0, "activation words divide over the threads");
    static_assert(!LN || WPR == SK3_NT, "fused LayerNorm: thread t holds columns 8t .. 8t+7 of every token");

    extern __shared__ __attribute__((aligned(16))) uint8_t sk3_lds[];
    uint8_t* xl = sk3_lds;
    uint32_t* zsl = (uint32_t*)(sk3_lds + L::Z_OFF);
    unsigned* last_flag = (unsigned*)(sk3_lds + L::FLAG_OFF);
    float* red = (float*)sk3_lds;

    const NibbleMasks nm = nibble_masks();
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int li = lane & 15;
    const int lj = lane >> 4;
    const int ks = blockIdx.y;
    const int chunks = K >> 7;
    const int groups = chunks * GPC;  // (z, s) pairs per row
    const int cps = (chunks + ksplit - 1) / ksplit;
    int c_begin = ks * cps;
    int nc = imin(c_begin + cps, chunks) - c_begin;
    if (nc <= 0) {  // an empty K range (the host does not create one) streams chunk 0 against zeros
        nc = 0;
        c_begin = 0;
    }

    // 1. zeros/scales of the row block and K range (row-contiguous)
    uint32_t zreg[ZPT];
#pragma unroll
    for (int p = 0; p < ZPT; p++) {
        const int idx = tid + p * SK3_NT;
        const int r = (idx / ZW) % ROWS, col = idx % ZW;
        const int row = imin(rb * ROWS + r, N - 1);
        zreg[p] = ZS[(long)row * groups + c_begin * GPC + (col < nc * GPC ? col : 0)];
    }
    // 2. every activation of the K range (tokens beyond M and chunk slots beyond the range: zeros)
    u32x4_t xr[XPT];
#pragma unroll
    for (int p = 0; p < XPT; p++) {
        const int idx = tid + p * SK3_NT;
        const int m = idx / WPR, col = idx % WPR;
        const bool ok = (m < M) && (col < nc * 16);
        // (masked with an AND, not selected: a select lets the compiler move the load under a branch, and its
        // wait counts around loads under branches are conservative)
        const uint32_t keep = ok ? 0xffffffffu : 0u;
        const u32x4_t v = *(const u32x4_t*)(X + (ok ? (long)m * K + c_begin * 128 + col * 8 : 0));
        xr[p] = (u32x4_t){v.x & keep, v.y & keep, v.z & keep, v.w & keep};
    }
    // (fused LayerNorm: its scale and shift for this thread's eight columns)
    u32x4_t lg = {0x3c003c00u, 0x3c003c00u, 0x3c003c00u, 0x3c003c00u}, lb = {0u, 0u, 0u, 0u};
    if (LN) {
        // unconditional loads (a missing scale or shift reads the activations' first bytes and is masked out)
        const bool ok = tid < nc * 16;
        const long off = ok ? c_begin * 128 + tid * 8 : 0;
        const uint32_t kg = ln.gamma ? 0xffffffffu : 0u, kb = ln.beta ? 0xffffffffu : 0u;
        const u32x4_t gv = *(const u32x4_t*)((ln.gamma ? ln.gamma : X) + off);
        const u32x4_t bv = *(const u32x4_t*)((ln.beta ? ln.beta : X) + off);
        lg = (u32x4_t){(gv.x & kg) | (lg.x & ~kg), (gv.y & kg) | (lg.y & ~kg), (gv.z & kg) | (lg.z & ~kg),
                       (gv.w & kg) | (lg.w & ~kg)};
        lb = (u32x4_t){bv.x & kb, bv.y & kb, bv.z & kb, bv.w & kb};
    }
    // Every wave has issued its activation loads before any wave issues a weight load: a CU serves its
    // vector memory requests in order, and activations queued behind another wave's sixteen weight loads
    // would reach the barrier below only when most of the stream has already arrived.
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_barrier" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);  // nothing that waits for a load moves above the weight requests
    // 3. the wave's weight loads, in units of four (two row tiles x the two 64-byte halves of a 128-byte
    //    line back to back, so that the line is requested from L2 once), DEPTH units ahead of the arithmetic
    constexpr int RTU = RT % 2 == 0 ? 2 : 1;    // row tiles per unit
    constexpr int RG = RT / RTU;                // units per chunk pair
    constexpr int HN = CH == 1 ? 1 : 2;         // chunk slots per unit
    constexpr int NU = (CH == 1 ? 1 : CH / 2) * RG;
    u32x4_t wq[CH][RT];
    int slot_of[CH];
#pragma unroll
    for (int u = 0; u < CH; u++) slot_of[u] = (CH == 1) ? wave : 2 * (wave + SK3_NWV * (u >> 1)) + (u & 1);
    const uint8_t* wrow[RT];
#pragma unroll
    for (int rt = 0; rt < RT; rt++) wrow[rt] = W + (long)imin(rb * ROWS + 16 * rt + li, N - 1) * (K >> 1) + lj * 16;
    auto issue_unit = [&](int un) {
        const int pr = un / RG, rg = un % RG;
#pragma unroll
        for (int r = 0; r < RTU; r++)
#pragma unroll
            for (int h = 0; h < HN; h++) {
                const int cl = slot_of[2 * pr + h];
                wq[2 * pr + h][RTU * rg + r] =
                    *(const u32x4_t*)(wrow[RTU * rg + r] + (long)(c_begin + (cl < nc ? cl : 0)) * 64);
            }
    };
    // (in front of a fused LayerNorm a 16-row workgroup, whose units are two loads, sends two of them: measured)
    constexpr int PRE = (LN && RT == 1) ? 2 : SK3_DEPTH_PRE;
    // (and 48-row workgroups one more once the activations have arrived, ahead of the LayerNorm arithmetic: the
    // memory system otherwise runs dry while every wave works on the activations.  Measured at 8 tokens:
    // 12288 x 4096 in 48-row workgroups 9.3 -> 8.8 us; 16384 x 4096 in 64-row workgroups 11.5 -> 12.0 us, so
    // those keep one unit.)
    constexpr int MID = (LN && RT == 3) ? 1 : 0;
    constexpr int STEADY = LN ? (DEPTH > PRE + MID ? DEPTH : PRE + MID) : DEPTH;
#pragma unroll
    for (int un = 0; un < NU; un++)
        if (un < PRE) issue_unit(un);
    __builtin_amdgcn_sched_barrier(0);
    // (fused LayerNorm, while the first weights are on their way: thread t holds columns 8t .. 8t+7 of every
    // token.  Per-thread partial sums go to LDS (the activations' space, not yet in use), wave w adds up the 512
    // partials of token w and leaves the statistic where every thread reads it; mean first, then the squared
    // deviations around it.  Every workgroup normalises all MROWS x K activations itself, so this is vector
    // arithmetic on the critical path of every CU: it runs on fp16 pairs.  Sums are two-wide dot products with
    // fp32 accumulation; the deviations are taken in fp16 around the fp16-rounded mean mh (the difference of two
    // fp16 numbers loses nothing that matters), the statistics correct for delta = mean - mh exactly
    // (var = E[(x - mh)^2] - delta^2, normalised value = (x - mh) * r - delta * r), and 1 / sigma enters as a
    // sum of two fp16 numbers so that its rounding does not scale the whole row.  The normalised row replaces
    // the raw one before it is parked.)
    if (LN) {
        float* scr = (float*)sk3_lds;                    // [MROWS][512] partials
        float* stat = (float*)(sk3_lds + L::LN_OFF);     // [2][MROWS]: mean, 1 / sqrt(var + eps)
        const bool cok = tid < nc * 16;
        const float inv_k = 1.f / (float)(nc * 128);
        auto token_sums = [&](const float (&part)[XPT], int which, bool finish_var) {
#pragma unroll
            for (int p = 0; p < XPT; p++) scr[p * SK3_NT + tid] = part[p];
            sk3_barrier();
            if (wave < MROWS) {
                float a = 0.f;
#pragma unroll
                for (int j = 0; j < SK3_NT / 64; j++) a += scr[wave * SK3_NT + lane + 64 * j];
                a = row_sum_stride4(quad_sum(a));  // every lane: the sum of its 16-lane row
                const float tot = (bit_cast<float>(__builtin_amdgcn_readlane(bit_cast<int>(a), 0)) +
                                   bit_cast<float>(__builtin_amdgcn_readlane(bit_cast<int>(a), 16))) +
                                  (bit_cast<float>(__builtin_amdgcn_readlane(bit_cast<int>(a), 32)) +
                                   bit_cast<float>(__builtin_amdgcn_readlane(bit_cast<int>(a), 48)));
                if (lane == 0) {
                    if (finish_var) {
                        const float mean_w = stat[wave];
                        const float dl = mean_w - (float)(half_t)mean_w;
                        stat[MROWS + wave] = rsqrtf(fmaxf(tot * inv_k - dl * dl, 0.f) + ln.eps);
                    } else {
                        stat[wave] = tot * inv_k;
                    }
                }
            }
            sk3_barrier();
        };
        const half2_t one2 = {(half_t)1.f, (half_t)1.f};
        float part[XPT], delta[XPT];
#pragma unroll
        for (int p = 0; p < XPT; p++) {
            float a = 0.f;
#pragma unroll
            for (int e = 0; e < 4; e++) a = __builtin_amdgcn_fdot2(bit_cast<half2_t>(xr[p][e]), one2, a, false);
            part[p] = a;  // zero where the token or the column does not exist
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int un = PRE; un < NU; un++)
            if (un < PRE + MID) issue_unit(un);
        __builtin_amdgcn_sched_barrier(0);
        token_sums(part, 0, false);
#pragma unroll
        for (int p = 0; p < XPT; p++) {
            const float mean = stat[p];
            const half_t mh = (half_t)mean;
            delta[p] = mean - (float)mh;
            const half2_t mh2 = {mh, mh};
            float q = 0.f;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const half2_t d = bit_cast<half2_t>(xr[p][e]) - mh2;
                xr[p][e] = bit_cast<uint32_t>(d);
                q = __builtin_amdgcn_fdot2(d, d, q, false);
            }
            part[p] = cok ? q : 0.f;
        }
        token_sums(part, 1, true);
#pragma unroll
        for (int p = 0; p < XPT; p++) {
            const float rstd = stat[MROWS + p];
            const half_t rh = (half_t)rstd;
            const half_t rl = (half_t)(rstd - (float)rh);
            const half_t ch = (half_t)(-delta[p] * rstd);
            const half2_t rh2 = {rh, rh}, rl2 = {rl, rl}, c2 = {ch, ch};
            u32x4_t o;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const half2_t d = bit_cast<half2_t>(xr[p][e]);
                const half2_t t = d * rh2 + (d * rl2 + c2);
                o[e] = bit_cast<uint32_t>(t * bit_cast<half2_t>(lg[e]) + bit_cast<half2_t>(lb[e]));
            }
            xr[p] = (cok && p < M) ? o : (u32x4_t){0u, 0u, 0u, 0u};
        }
        sk3_barrier();  // the partials' space becomes the activations' space
    }
    // 4. park zeros/scales and activations (waits for 1 and 2 only: the weight loads stay in flight)
#pragma unroll
    for (int p = 0; p < ZPT; p++) {
        const int idx = tid + p * SK3_NT;
        if (idx < ROWS * ZW) zsl[(idx / ZW) * L::ZPITCH + idx % ZW] = zreg[p];
    }
#pragma unroll
    for (int p = 0; p < XPT; p++) {
        const int idx = tid + p * SK3_NT;
        *(u32x4_t*)(xl + (idx / WPR) * L::XPITCH + (idx % WPR) * 16) = xr[p];
    }
    sk3_barrier();

    // 5. the wave's units in issue order, the next request going out before each unit's arithmetic
    float4_t acc[RT];
#pragma unroll
    for (int rt = 0; rt < RT; rt++) acc[rt] = (float4_t){0.f, 0.f, 0.f, 0.f};
    const half8_t ones = {(half_t)1.f, (half_t)1.f, (half_t)1.f, (half_t)1.f,
                          (half_t)1.f, (half_t)1.f, (half_t)1.f, (half_t)1.f};
    const uint8_t* xrd = xl + (li & (MROWS - 1)) * L::XPITCH + lj * 64;  // token li (a token >= MROWS repeats one: ignored)
    float4_t xsum[CH], x960[CH];
    const half8_t m960 = {(half_t)-960.f, (half_t)-960.f, (half_t)0.f, (half_t)0.f,
                          (half_t)-960.f, (half_t)-960.f, (half_t)0.f, (half_t)0.f};
#pragma unroll
    for (int un = PRE + MID; un < NU; un++)
        if (un < STEADY) issue_unit(un);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int un = 0; un < NU; un++) {
        if (un + STEADY < NU) {
            issue_unit(un + STEADY);
            __builtin_amdgcn_sched_barrier(0);  // the request goes out here, not wherever the scheduler finds room
        }
        const int pr = un / RG, rg = un % RG;
#pragma unroll
        for (int h = 0; h < HN; h++) {
            const int u = 2 * pr + h;
            const int cl = slot_of[u];
            const int zcol = cl < nc ? cl : 0;
            half8_t xa[4];
#pragma unroll
            for (int t = 0; t < 4; t++) xa[t] = *(const half8_t*)(xrd + cl * 256 + 16 * t);
            if (GPC == 1) {
                if (rg == 0) {
                    xsum[u] = (float4_t){0.f, 0.f, 0.f, 0.f};
                    x960[u] = (float4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int t = 0; t < 4; t++) {
                        xsum[u] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[t], ones, xsum[u], 0, 0, 0);
                        x960[u] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[t], m960, x960[u], 0, 0, 0);
                    }
                }
#pragma unroll
                for (int r = 0; r < RTU; r++) {
                    const int rt = RTU * rg + r;
                    const half2_t zsv = bit_cast<half2_t>(zsl[(16 * rt + li) * L::ZPITCH + zcol]);
                    // shift-free unpack (1024 + q on four of every eight positions); the accumulator starts at
                    // -960 * (sum of x over those positions), which takes the extra bias out again
                    float4_t tmp = x960[u];
#pragma unroll
                    for (int t = 0; t < 4; t++)
                        tmp = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[t], unpack8_mixed(wq[u][rt][t], nm), tmp, 0, 0, 0);
                    const float zf = (float)zsv.x;
                    const float sf = (float)zsv.y;
#pragma unroll
                    for (int v = 0; v < 4; v++) acc[rt][v] += sf * (tmp[v] - zf * xsum[u][v]);
                }
            } else {
                // Group size 64: a matrix instruction spans both groups of the chunk (lanes lj = 0, 1 hold the
                // first 64 columns, lj = 2, 3 the second), so zero and scale cannot be applied to its result;
                // each lane dequantises its own weights instead (its row and its group are its own), bit-identical
                // to the reference's fp16 (q - z) * s.
#pragma unroll
                for (int r = 0; r < RTU; r++) {
                    const int rt = RTU * rg + r;
                    const half2_t zsv = bit_cast<half2_t>(zsl[(16 * rt + li) * L::ZPITCH + zcol * GPC + (lj >> 1)]);
                    const half2_t z64 = {zsv.x, zsv.x}, sc = {zsv.y, zsv.y};
#pragma unroll
                    for (int t = 0; t < 4; t++)
                        acc[rt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[t], dequant8(wq[u][rt][t], z64, sc, nm), acc[rt], 0, 0, 0);
                }
            }
        }
    }
    sk3_barrier();  // every wave is done with the activations, which the partials now overwrite

    // Sum the waves' partial tiles: red[wave][rt][v][lane].
#pragma unroll
    for (int rt = 0; rt < RT; rt++)
#pragma unroll
        for (int v = 0; v < 4; v++) red[wave * TILE + (rt * 4 + v) * 64 + lane] = acc[rt][v];
    sk3_barrier();

    // Element t of the tile: lane l = t % 64, v, rt -> token m = 4 (l / 16) + v, row n = ROWS rb + 16 rt + l % 16.
    if (ksplit == 1 && RT == 1) {
        // a 16-row workgroup has 256 elements: one per thread is faster than four for a quarter of the threads
        // (4096 x 4096 at 8 tokens: 5.0 against 5.4 us)
        for (int t = tid; t < TILE; t += SK3_NT) {
            float sum = 0.f;
#pragma unroll
            for (int p = 0; p < SK3_NWV; p++) sum += red[p * TILE + t];
            const int l = t & 63, v = (t >> 6) & 3, rt = t >> 8;
            const int m = 4 * (l >> 4) + v;
            const int n = rb * ROWS + 16 * rt + (l & 15);
            if (m < M && n < N) Y[(long)m * N + n] = epilogue(sum, m, n, N, epi);
        }
        return;
    }
    if (ksplit == 1) {
        // four consecutive elements per thread: one token, four consecutive rows of the weight, so that bias,
        // residual and result travel as 64-bit accesses
        const bool fast_tail = tail4_applies(epi);
        for (int t4 = tid * 4; t4 < TILE; t4 += 4 * SK3_NT) {
            const int l4 = t4 & 63, v4 = (t4 >> 6) & 3, rt4 = t4 >> 8;
            const int m4 = 4 * (l4 >> 4) + v4;
            const int n4 = rb * ROWS + 16 * rt4 + (l4 & 15);
            const bool inside = m4 < M && n4 < N;
            Tail4 pre = {{0u, 0u}, {0u, 0u}};
            if (fast_tail) pre = tail4_request(epi, m4, n4, N, inside);
            float4_t sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int p = 0; p < SK3_NWV; p++) sum += *(const float4_t*)(&red[p * TILE + t4]);
            if (fast_tail) {
                if (inside) tail4_store(sum, pre, Y, m4, n4, N, epi);
                continue;
            }
#pragma unroll
            for (int e = 0; e < 4; e++)
                if (inside) Y[(long)m4 * N + n4 + e] = epilogue(sum[e], m4, n4 + e, N, epi);
        }
        return;
    }
    // Cross-workgroup exchange as in the split-K decode kernel: partial tiles as stores at the
    // agent-coherent level, a wait for them, one relaxed counter per row block; the last arriver adds
    // the partials in a fixed order, writes Y and resets the counter.
    float* mine = part + ((long)ks * nslots + slot) * TILE;
    for (int t4 = tid * 4; t4 < TILE; t4 += 4 * SK3_NT) {
        float4_t sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int p = 0; p < SK3_NWV; p++) sum += *(const float4_t*)(&red[p * TILE + t4]);
        store_coherent_x4(mine + t4, sum);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    sk3_barrier();
    if (tid == 0) {
        const unsigned old = __hip_atomic_fetch_add(&counters[slot], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        *last_flag = (old == (unsigned)(ksplit - 1)) ? 1u : 0u;
    }
    sk3_barrier();
    if (!*last_flag) return;
    const bool fast_tail = tail4_applies(epi);
    for (int t4 = tid * 4; t4 < TILE; t4 += 4 * SK3_NT) {
        // the four elements t4 .. t4 + 3 are one token and four consecutive rows of the weight
        const int l4 = t4 & 63, v4 = (t4 >> 6) & 3, rt4 = t4 >> 8;
        const int m4 = 4 * (l4 >> 4) + v4;
        const int n4 = rb * ROWS + 16 * rt4 + (l4 & 15);
        const bool inside = m4 < M && n4 < N;
        Tail4 pre = {{0u, 0u}, {0u, 0u}};
        if (fast_tail) pre = tail4_request(epi, m4, n4, N, inside);
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
    if (tid == 0) __hip_atomic_store(&counters[slot], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// 17..32 tokens: two token tiles per operand (every unpacked weight word meets both), 64-row workgroups, a wave owns
// the same four chunk slots as above.  A wave needs the activations of ITS chunks only (32 tokens x 256 bytes per
// chunk), so nothing about them is shared: each wave moves them global -> LDS itself with direct loads (no
// registers, no workgroup barrier) through a private ring of two chunks, the third and fourth chunk requested as
// soon as the first and second are consumed.  The row of a token is stored with its sixteen 16-byte pieces XORed by
// the token index, which makes the 128-bit operand reads (lane = token) conflict-free.  All sixteen weight words of
// the wave are requested at the start, in the order of use and interleaved with the activation chunks, and every
// wait names the number of younger requests that may stay in flight (the vector memory counter retires in order).
// The loads are inline assembly: the compiler then inserts no waits of its own, which could only be conservative
// here (it cannot see the direct loads).  A timeline of the previous form (activations staged by the whole
// workgroup in two halves through registers) showed 12 of its 15.5 us waiting: 1.9 us to issue the first half's
// requests (a CU takes a few dozen wave-wide requests at a time), 4 us from the first barrier to the end of the first
// unit (the second half's requests had to be issued before its arithmetic could start), 1.5 us for the swap.
//
// RT row tiles per workgroup and CH chunk slots per wave (a workgroup covers 8 CH chunks of K); launched with 4 and 4.
template <int RT, int CH>
struct Sk3WideLds {
    static constexpr int XSLOT = 32 * 256;               // one chunk of 32 tokens
    static constexpr int XWAVE = 2 * XSLOT;              // a wave's ring
    static constexpr int TILE = RT * 2 * 4 * 64;         // floats a wave contributes: [rt][mt][v][lane]; they overwrite its ring
    static constexpr int ZCOLS = 8 * CH;                 // chunk slots of a workgroup
    static constexpr int Z_OFF = SK3_NWV * XWAVE;        // zeros/scales of the row block: 16 RT rows x ZCOLS
    static constexpr int FLAG_OFF = Z_OFF + 16 * RT * ZCOLS * 4;
    static constexpr int BYTES = FLAG_OFF + 16;
};

// Wait until at most N younger requests are outstanding.  Names a chunk's weight words, so that no use of them can be
// scheduled ahead of the wait (they are loaded by inline assembly: the compiler does not know they arrive later).
template <int N, int RT>
__device__ __forceinline__ void sk3_wait_words(u32x4_t (&w)[RT]) {
    static_assert(RT == 4 || RT == 8, "row tiles per workgroup");
    if constexpr (RT == 4)
        asm volatile("s_waitcnt vmcnt(%4)" : "+v"(w[0]), "+v"(w[1]), "+v"(w[2]), "+v"(w[3]) : "n"(N) : "memory");
    else
        asm volatile("s_waitcnt vmcnt(%8)"
                     : "+v"(w[0]), "+v"(w[1]), "+v"(w[2]), "+v"(w[3]), "+v"(w[4]), "+v"(w[5]), "+v"(w[6]), "+v"(w[7])
                     : "n"(N)
                     : "memory");
}

template <int RT, int CH>
__device__ __forceinline__ void skinny3_wide_body(const uint8_t* __restrict__ W, const uint32_t* __restrict__ ZS,
                                                  const half_t* __restrict__ X, half_t* __restrict__ Y, float* part,
                                                  unsigned* counters, int M, int N, int K, int ksplit,
                                                  const Epilogue& epi, int rb, int slot, int nslots) {
    using L = Sk3WideLds<RT, CH>;
    constexpr int MT = 2, ROWS = 16 * RT, TILE = L::TILE, ZC = L::ZCOLS;
    static_assert(CH == 4, "the request schedule below is written for four chunk slots per wave");
    static_assert(L::XWAVE >= TILE * 4, "a wave's partial tile fits its ring");

    extern __shared__ __attribute__((aligned(16))) uint8_t sk3_lds[];
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)sk3_lds;
    const uint32_t* zsl = (const uint32_t*)(sk3_lds + L::Z_OFF);
    unsigned* last_flag = (unsigned*)(sk3_lds + L::FLAG_OFF);

    const NibbleMasks nm = nibble_masks();
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 15;
    const int lj = lane >> 4;
    const int ks = blockIdx.y;
    const int chunks = K >> 7;
    const int cps = (chunks + ksplit - 1) / ksplit;
    int c_begin = ks * cps;
    int nc = imin(c_begin + cps, chunks) - c_begin;
    if (nc <= 0) {
        nc = 0;
        c_begin = 0;
    }
    uint8_t* xw = sk3_lds + wave * L::XWAVE;
    const uint32_t xw0 = lds0 + wave * L::XWAVE;

    // chunk slots of this wave; one past the range reads chunk c_begin and gets scale 0
    int cl[CH], cg[CH];
#pragma unroll
    for (int u = 0; u < CH; u++) {
        cl[u] = 2 * (wave + SK3_NWV * (u >> 1)) + (u & 1);
        cg[u] = c_begin + (cl[u] < nc ? cl[u] : 0);
    }
    // Instruction i of a chunk moves tokens 4 i .. 4 i + 3: lane l fetches, for ring position l % 16 of token
    // 4 i + l / 16, the piece (l % 16) ^ (token % 16).  Tokens past M re-read the last one (never stored).
    const half_t* xrow[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const int t = 4 * i + lj;
        xrow[i] = X + (long)imin(t, M - 1) * K + ((li ^ (t & 15)) * 8);
    }
    auto dma_x = [&](int u) {
#pragma unroll
        for (int i = 0; i < 8; i++) load_to_lds_x4(xrow[i] + (long)cg[u] * 128, xw0 + (u & 1) * L::XSLOT + i * 1024);
    };
    const uint8_t* wrow[RT];
#pragma unroll
    for (int rt = 0; rt < RT; rt++) wrow[rt] = W + (long)imin(rb * ROWS + 16 * rt + li, N - 1) * (K >> 1) + lj * 16;
    u32x4_t wq[CH][RT];
    auto load_w = [&](int u) {
#pragma unroll
        for (int rt = 0; rt < RT; rt++)
            asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(wq[u][rt]) : "v"(wrow[rt] + (long)cg[u] * 64) : "memory");
    };
    // zeros/scales of the row block, by the whole workgroup: ZQ instructions per wave, 64 consecutive (row, chunk
    // slot) pairs each
    constexpr int ZQ = RT * CH / 4;
#pragma unroll
    for (int q = 0; q < ZQ; q++) {
        const int idx = (wave * ZQ + q) * 64 + lane;
        const int r = idx / ZC, col = idx % ZC;
        const int row = imin(rb * ROWS + r, N - 1);
        load_to_lds_x1(ZS + (long)row * chunks + c_begin + (col < nc ? col : 0), lds0 + L::Z_OFF + (wave * ZQ + q) * 256);
    }
    dma_x(0);
    load_w(0);
    // The one thing the waves share are the zeros/scales: meet as soon as they have landed (the twelve requests
    // behind them stay in flight), before the bulk of the requests is issued.  Issuing takes a wave 2..8 us here
    // (a CU takes a few dozen wave-wide requests at a time); with the barrier behind all of it every wave would
    // start its arithmetic when the slowest has finished issuing.
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(8 + RT) : "memory");
    dma_x(1);
    load_w(1);
    load_w(2);
    load_w(3);

    float4_t acc[RT][MT];
#pragma unroll
    for (int rt = 0; rt < RT; rt++)
#pragma unroll
        for (int mt = 0; mt < MT; mt++) acc[rt][mt] = (float4_t){0.f, 0.f, 0.f, 0.f};
    const half8_t ones = {(half_t)1.f, (half_t)1.f, (half_t)1.f, (half_t)1.f,
                          (half_t)1.f, (half_t)1.f, (half_t)1.f, (half_t)1.f};
    const half8_t m960 = {(half_t)-960.f, (half_t)-960.f, (half_t)0.f, (half_t)0.f,
                          (half_t)-960.f, (half_t)-960.f, (half_t)0.f, (half_t)0.f};

    auto consume = [&](int u) {
        const uint8_t* xs = xw + (u & 1) * L::XSLOT + li * 256;
        const bool valid = cl[u] < nc;
        const int zcol = valid ? cl[u] : 0;
        half8_t xa[MT][4];
        float4_t xsum[MT], x960[MT];
#pragma unroll
        for (int mt = 0; mt < MT; mt++) {
#pragma unroll
            for (int t = 0; t < 4; t++) xa[mt][t] = *(const half8_t*)(xs + 16 * mt * 256 + (((4 * lj + t) ^ li) * 16));
            xsum[mt] = (float4_t){0.f, 0.f, 0.f, 0.f};
            x960[mt] = (float4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int t = 0; t < 4; t++) {
                xsum[mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[mt][t], ones, xsum[mt], 0, 0, 0);
                x960[mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[mt][t], m960, x960[mt], 0, 0, 0);
            }
        }
#pragma unroll
        for (int rt = 0; rt < RT; rt++) {
            const half2_t zsv = bit_cast<half2_t>(zsl[(16 * rt + li) * ZC + zcol]);
            const float zf = (float)zsv.x;
            const float sf = valid ? (float)zsv.y : 0.f;
            half8_t wv[4];
#pragma unroll
            for (int t = 0; t < 4; t++) wv[t] = unpack8_mixed(wq[u][rt][t], nm);
#pragma unroll
            for (int mt = 0; mt < MT; mt++) {
                float4_t tmp = x960[mt];
#pragma unroll
                for (int t = 0; t < 4; t++) tmp = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[mt][t], wv[t], tmp, 0, 0, 0);
#pragma unroll
                for (int v = 0; v < 4; v++) acc[rt][mt][v] += sf * (tmp[v] - zf * xsum[mt][v]);
            }
        }
    };

    // requests so far, oldest first: zeros/scales, x0 8, w0 RT, x1 8, w1 RT, w2 RT, w3 RT
    sk3_wait_words<8 + 3 * RT>(wq[0]);  // x0, w0 are there
    consume(0);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // ring position 0 has been read
    dma_x(2);
    sk3_wait_words<8 + 2 * RT>(wq[1]);  // x1, w1 (w2, w3, x2 may be outstanding)
    consume(1);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    dma_x(3);
    sk3_wait_words<8>(wq[2]);  // w2, w3, x2 (x3 may be outstanding)
    consume(2);
    sk3_wait_words<0>(wq[3]);
    consume(3);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // this wave's ring is free: its partial tile goes there

    float* mine_lds = (float*)xw;
#pragma unroll
    for (int rt = 0; rt < RT; rt++)
#pragma unroll
        for (int mt = 0; mt < MT; mt++)
#pragma unroll
            for (int v = 0; v < 4; v++) mine_lds[((rt * MT + mt) * 4 + v) * 64 + lane] = acc[rt][mt][v];
    sk3_barrier();
    auto red = [&](int p, int t) -> const float* { return (const float*)(sk3_lds + p * L::XWAVE) + t; };

    // Element t of the tile: lane l = t % 64, v, mt, rt -> token m = 16 mt + 4 (l / 16) + v, row n = 64 rb + 16 rt + l % 16.
    if (ksplit == 1) {
        // four consecutive elements per thread: one token, four consecutive rows of the weight, so that bias,
        // residual and result travel as 64-bit accesses
        const bool fast_tail = tail4_applies(epi);
        for (int t4 = tid * 4; t4 < TILE; t4 += 4 * SK3_NT) {
            const int l4 = t4 & 63, v4 = (t4 >> 6) & 3, mt4 = (t4 >> 8) % MT, rt4 = (t4 >> 8) / MT;
            const int m4 = 16 * mt4 + 4 * (l4 >> 4) + v4;
            const int n4 = rb * ROWS + 16 * rt4 + (l4 & 15);
            const bool inside = m4 < M && n4 < N;
            Tail4 pre = {{0u, 0u}, {0u, 0u}};
            if (fast_tail) pre = tail4_request(epi, m4, n4, N, inside);
            float4_t sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int p = 0; p < SK3_NWV; p++) sum += *(const float4_t*)red(p, t4);
            if (fast_tail) {
                if (inside) tail4_store(sum, pre, Y, m4, n4, N, epi);
                continue;
            }
#pragma unroll
            for (int e = 0; e < 4; e++)
                if (inside) Y[(long)m4 * N + n4 + e] = epilogue(sum[e], m4, n4 + e, N, epi);
        }
        return;
    }
    float* mine = part + ((long)ks * nslots + slot) * TILE;
    for (int t4 = tid * 4; t4 < TILE; t4 += 4 * SK3_NT) {
        float4_t sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int p = 0; p < SK3_NWV; p++) sum += *(const float4_t*)red(p, t4);
        store_coherent_x4(mine + t4, sum);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    sk3_barrier();
    if (tid == 0) {
        const unsigned old = __hip_atomic_fetch_add(&counters[slot], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        *last_flag = (old == (unsigned)(ksplit - 1)) ? 1u : 0u;
    }
    sk3_barrier();
    if (!*last_flag) return;
    const bool fast_tail = tail4_applies(epi);
    for (int t4 = tid * 4; t4 < TILE; t4 += 4 * SK3_NT) {
        // the four elements t4 .. t4 + 3 are one token and four consecutive rows of the weight
        const int l4 = t4 & 63, v4 = (t4 >> 6) & 3, mt4 = (t4 >> 8) % MT, rt4 = (t4 >> 8) / MT;
        const int m4 = 16 * mt4 + 4 * (l4 >> 4) + v4;
        const int n4 = rb * ROWS + 16 * rt4 + (l4 & 15);
        const bool inside = m4 < M && n4 < N;
        Tail4 pre = {{0u, 0u}, {0u, 0u}};
        if (fast_tail) pre = tail4_request(epi, m4, n4, N, inside);
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
    if (tid == 0) __hip_atomic_store(&counters[slot], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <int RT, int CH>
__global__ __launch_bounds__(SK3_NT) void skinny3_wide_kernel(const uint8_t* __restrict__ W, const uint32_t* __restrict__ ZS,
                                                              const half_t* __restrict__ X, half_t* __restrict__ Y,
                                                              float* part, unsigned* counters, int M, int N, int K,
                                                              int ksplit, Epilogue epi) {
    skinny3_wide_body<RT, CH>(W, ZS, X, Y, part, counters, M, N, K, ksplit, epi, blockIdx.x, blockIdx.x, gridDim.x);
}

template <int MROWS, int RT, int CH, bool LN, int GPC>
__global__ __launch_bounds__(SK3_NT) void skinny3_kernel(const uint8_t* __restrict__ W, const uint32_t* __restrict__ ZS,
                                                         const half_t* __restrict__ X, half_t* __restrict__ Y,
                                                         float* part, unsigned* counters, int M, int N, int K,
                                                         int ksplit, Epilogue epi, LnPre ln) {
    skinny3_body<MROWS, RT, CH, SK3_DEPTH, LN, GPC>(W, ZS, X, Y, part, counters, M, N, K, ksplit, epi, ln, blockIdx.x, blockIdx.x,
                                               gridDim.x);
}

struct Skinny3Group {
    const uint8_t* W[GEMV_GROUP_MAX];
    const uint32_t* ZS[GEMV_GROUP_MAX];
    const half_t* X[GEMV_GROUP_MAX];
    half_t* Y[GEMV_GROUP_MAX];
    const half_t* bias[GEMV_GROUP_MAX];
    const half_t* residual[GEMV_GROUP_MAX];
    int N[GEMV_GROUP_MAX];
    int act[GEMV_GROUP_MAX];
    int blk_end[GEMV_GROUP_MAX];  // first row block behind linear p
    int count;
};

template <int MROWS, int RT, int CH>
__global__ __launch_bounds__(SK3_NT) void skinny3_group_kernel(const Skinny3Group grp, float* part, unsigned* counters,
                                                               int M, int K, int ksplit) {
    int p = 0;
#pragma unroll
    for (int q = 0; q < GEMV_GROUP_MAX - 1; q++)
        if (q + 1 < grp.count && (int)blockIdx.x >= grp.blk_end[q]) p = q + 1;
    const int rb = blockIdx.x - (p > 0 ? grp.blk_end[p - 1] : 0);
    const Epilogue epi{grp.bias[p], grp.residual[p], grp.act[p]};
    skinny3_body<MROWS, RT, CH, SK3_DEPTH, false, 1>(grp.W[p], grp.ZS[p], grp.X[p], grp.Y[p], part, counters, M, grp.N[p], K,
                                                  ksplit, epi, LnPre{nullptr, nullptr, 0.f}, rb, blockIdx.x, gridDim.x);
}

template <int RT, int CH>
__global__ __launch_bounds__(SK3_NT) void skinny3_wide_group_kernel(const Skinny3Group grp, float* part,
                                                                    unsigned* counters, int M, int K, int ksplit) {
    int p = 0;
#pragma unroll
    for (int q = 0; q < GEMV_GROUP_MAX - 1; q++)
        if (q + 1 < grp.count && (int)blockIdx.x >= grp.blk_end[q]) p = q + 1;
    const int rb = blockIdx.x - (p > 0 ? grp.blk_end[p - 1] : 0);
    const Epilogue epi{grp.bias[p], grp.residual[p], grp.act[p]};
    skinny3_wide_body<RT, CH>(grp.W[p], grp.ZS[p], grp.X[p], grp.Y[p], part, counters, M, grp.N[p], K, ksplit, epi, rb,
                              blockIdx.x, gridDim.x);
}

template <typename Kern>
hipError_t allow_lds(Kern kern, int bytes, bool* done) {
    if (bytes <= 64 * 1024) return hipSuccess;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return hipErrorInvalidDevice;
    if (!done[dev]) {
        const hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
        if (e != hipSuccess) return e;
        done[dev] = true;
    }
    return hipSuccess;
}

template <int MROWS, int RT, int CH, bool LN, int GPC = 1>
hipError_t launch_cfg(const void* x, const void* w, const void* zs, void* y, void* ws, int M, int N, int K, int ksplit,
                      Epilogue epi, LnPre ln, hipStream_t st) {
    static bool allowed[64];
    constexpr int lds = Sk3Lds<MROWS, RT, CH, GPC>::BYTES;
    const hipError_t e = allow_lds(skinny3_kernel<MROWS, RT, CH, LN, GPC>, lds, allowed);
    if (e != hipSuccess) return e;
    const dim3 grid((N + 16 * RT - 1) / (16 * RT), ksplit);
    hipLaunchKernelGGL((skinny3_kernel<MROWS, RT, CH, LN, GPC>), grid, dim3(SK3_NT), lds, st, (const uint8_t*)w,
                       (const uint32_t*)zs, (const half_t*)x, (half_t*)y,
                       ws ? (float*)((char*)ws + SK3_COUNTER_BYTES) : nullptr, (unsigned*)ws, M, N, K, ksplit, epi, ln);
    return hipGetLastError();
}

template <int MROWS, int RT, int CH>
hipError_t launch_group_cfg(const SeqProblem* probs, int count, void* ws, int M, int K, int ksplit, hipStream_t st) {
    static bool allowed[64];
    constexpr int lds = Sk3Lds<MROWS, RT, CH>::BYTES;
    const hipError_t e = allow_lds(skinny3_group_kernel<MROWS, RT, CH>, lds, allowed);
    if (e != hipSuccess) return e;
    Skinny3Group g;
    int blocks = 0;
    for (int p = 0; p < GEMV_GROUP_MAX; p++) {
        const SeqProblem& q = probs[p < count ? p : 0];
        g.W[p] = (const uint8_t*)q.w;
        g.ZS[p] = (const uint32_t*)q.zs;
        g.X[p] = (const half_t*)q.x;
        g.Y[p] = (half_t*)q.y;
        g.bias[p] = (const half_t*)q.bias;
        g.residual[p] = (const half_t*)q.residual;
        g.N[p] = q.N;
        g.act[p] = q.act;
        if (p < count) blocks += (q.N + 16 * RT - 1) / (16 * RT);
        g.blk_end[p] = blocks;
    }
    g.count = count;
    hipLaunchKernelGGL((skinny3_group_kernel<MROWS, RT, CH>), dim3(blocks, ksplit), dim3(SK3_NT), lds, st, g,
                       ws ? (float*)((char*)ws + SK3_COUNTER_BYTES) : nullptr, (unsigned*)ws, M, K, ksplit);
    return hipGetLastError();
}

// Shape of a launch: rows per workgroup (16 RT), chunk slots per wave (CH) and the K split.  `blocks64` = 64-row
// blocks of all linears of the launch together.
struct Sk3Plan {
    int rt, ch, ksplit;
};

Sk3Plan plan(const int* rows, int count, int K, bool have_ws, int tune, int M) {
    const int groups = K / 128;
    const int ks0 = (groups + 31) / 32;  // the least split: a workgroup covers at most 32 chunks
    Sk3Plan none{4, 4, 0};
    auto shape = [&](int ks, Sk3Plan* p) {
        p->ksplit = ks;
        const int cps = (groups + ks - 1) / ks;
        p->ch = cps <= 8 ? 1 : cps <= 16 ? 2 : 4;
        return !(cps > 32 || (ks > 1 && !have_ws) || ks > 8 || (ks - 1) * cps >= groups);
    };
    if ((tune >> 4) & 0xF) {
        Sk3Plan p{4, 4, 0};
        if (!shape((tune >> 4) & 0xF, &p)) return none;
        p.rt = (tune & 0xF) == 1 ? 1 : ((tune & 0xF) == 3 && p.ksplit == 1 && p.ch == 4) ? 3 : 4;
        if ((tune & 0xF) == 0) {
            // rows per workgroup by the count below, at the given split
            int best = 1 << 30;
            for (int rt : {4, 3, 1}) {
                if (rt == 3 && (p.ksplit != 1 || p.ch != 4)) continue;
                long blocks = 0;
                for (int l = 0; l < count; l++) blocks += (rows[l] + 16 * rt - 1) / (16 * rt);
                const long cost = (blocks * p.ksplit + 255) / 256 * (rt + 2);
                if (cost < best) best = (int)cost, p.rt = rt;
            }
        }
        return p;
    }
    // Rows per workgroup (64, 48 or 16) and K split (the least one, or two or four times as fine) by a count of
    // time calibrated on timed launches at 8 and 16 tokens, in units of 1.75 us (what a CU needs to stream one
    // 16-row tile over a full range of 32 chunks): rounds of 256 workgroups (one per CU; 512 below) x ((row tiles + M / 24 for
    // the activations, which come from L2 at a sixth of the price per byte) x the part of a full range a workgroup
    // covers + 1 for a workgroup's start: its activations must be there before its first matrix instruction),
    // + 1.54 (2.7 us) where partial tiles are exchanged.  OPT-6.7B: 4096 rows -> 16 (256 workgroups), 12288 and
    // 11008 -> 48 (256 and 230), 16384 -> 64 (256), 4096 x 16384 -> 64 rows x 4 ranges.  A finer split pays where
    // the least one leaves rounds half empty: 5120 x 13824 at 16 tokens 80 x 4 = 320 workgroups (18.7 us) -> 80 x 8
    // (15.7); 1024 x 8192 64 x 2 -> 64 x 4 with 16 rows (7.3 -> 6.4).  48-row workgroups only without a K split
    // (their partial tiles do not fit the workspace layout) and with full-length K ranges.
    Sk3Plan bestp = none;
    float best = 3.4e38f;
    for (int ks = ks0; ks <= 8 && ks <= 4 * ks0; ks *= 2) {
        Sk3Plan p{4, 4, 0};
        if (!shape(ks, &p)) continue;
        const int cps = (groups + ks - 1) / ks;
        for (int rt : {4, 3, 1}) {
            if (rt == 3 && (ks != 1 || p.ch != 4)) continue;
            long blocks = 0;
            for (int l = 0; l < count; l++) blocks += (rows[l] + 16 * rt - 1) / (16 * rt);
            // (an unsplit K of at most 2048 leaves room for two workgroups per CU: 6144 x 2048 at 8 tokens in
            // 16-row workgroups 4.6 against 5.8 us in 64-row ones, 8192 x 1024 3.4 against 3.8)
            const int per_round = (ks == 1 && p.ch <= 2) ? 512 : 256;
            const long rounds = (blocks * ks + per_round - 1) / per_round;
            const float cost = rounds * ((rt + M / 24.f) * (cps / 32.f) + 1.f) + (ks > 1 ? 1.54f : 0.f);
            if (cost < best - 1e-3f) {
                best = cost;
                bestp = p;
                bestp.rt = rt;
            }
        }
    }
    if ((tune & 0xF) && bestp.ksplit)
        bestp.rt = (tune & 0xF) == 1 ? 1 : ((tune & 0xF) == 3 && bestp.ksplit == 1 && bestp.ch == 4) ? 3 : 4;
    return bestp;
}

}  // namespace

// M <= 16, group size 128 or 64, K % 128 == 0.  tune = rows per workgroup (1: 16, 3: 48, 4: 64) | ksplit << 4, 0 = heuristic.
// ln (may be null): LayerNorm of the activations inside the kernel; possible when a workgroup holds whole rows
// (2048 < K <= 4096, no K split) of at most 8 tokens.  hipErrorInvalidValue when the shape does not fit (K range per workgroup beyond
// 4096, a K split without a workspace, or a LayerNorm over rows the workgroup does not hold whole).
hipError_t launch_skinny3_tuned(const void* x, const void* w, const void* zs, void* y, void* ws, int M, int N, int K,
                                int g, int tune, Epilogue epi, const LnPre* ln, hipStream_t st) {
    if (M < 1 || M > 16 || K % 128 != 0 || (g != 128 && g != 64)) return hipErrorInvalidValue;
    Sk3Plan p = plan(&N, 1, K, ws != nullptr, tune, M);
    if (p.ksplit == 0) return hipErrorInvalidValue;
    if (g == 64 && p.rt == 3) p.rt = 4;  // group size 64: 16- and 64-row workgroups only
    if (p.ksplit > 1 && (N + 16 * p.rt - 1) / (16 * p.rt) > 16384) return hipErrorInvalidValue;
    const LnPre none{nullptr, nullptr, 0.f};
    if (g == 64) {
        if (ln) return hipErrorInvalidValue;
#define SQ_SK3_G64(MR, RT)                                                                                   \
    do {                                                                                                     \
        if (p.ch == 1) return launch_cfg<MR, RT, 1, false, 2>(x, w, zs, y, ws, M, N, K, p.ksplit, epi, none, st); \
        if (p.ch == 2) return launch_cfg<MR, RT, 2, false, 2>(x, w, zs, y, ws, M, N, K, p.ksplit, epi, none, st); \
        return launch_cfg<MR, RT, 4, false, 2>(x, w, zs, y, ws, M, N, K, p.ksplit, epi, none, st);                \
    } while (0)
        if (M <= 8) {
            if (p.rt == 1) SQ_SK3_G64(8, 1);
            SQ_SK3_G64(8, 4);
        }
        if (p.rt == 1) SQ_SK3_G64(16, 1);
        SQ_SK3_G64(16, 4);
#undef SQ_SK3_G64
    }
    if (ln) {
        if (p.ksplit != 1 || p.ch != 4) return hipErrorInvalidValue;
#define SQ_SK3_LN(MR, RT) return launch_cfg<MR, RT, 4, true>(x, w, zs, y, ws, M, N, K, 1, epi, *ln, st)
        if (M <= 4) {
            if (p.rt == 1) SQ_SK3_LN(4, 1);
            if (p.rt == 3) SQ_SK3_LN(4, 3);
            SQ_SK3_LN(4, 4);
        }
        if (M > 8) return hipErrorInvalidValue;  // sixteen rows of statistics per thread do not fit the registers
        if (p.rt == 1) SQ_SK3_LN(8, 1);
        if (p.rt == 3) SQ_SK3_LN(8, 3);
        SQ_SK3_LN(8, 4);
#undef SQ_SK3_LN
    }
#define SQ_SK3(MR, RT, CH) return launch_cfg<MR, RT, CH, false>(x, w, zs, y, ws, M, N, K, p.ksplit, epi, none, st)
#define SQ_SK3_CH(MR, RT)            \
    do {                             \
        if (p.ch == 1) SQ_SK3(MR, RT, 1); \
        if (p.ch == 2) SQ_SK3(MR, RT, 2); \
        SQ_SK3(MR, RT, 4);           \
    } while (0)
    if (M <= 4) {
        if (p.rt == 1) SQ_SK3_CH(4, 1);
        if (p.rt == 3) SQ_SK3(4, 3, 4);
        SQ_SK3_CH(4, 4);
    }
    if (M <= 8) {
        if (p.rt == 1) SQ_SK3_CH(8, 1);
        if (p.rt == 3) SQ_SK3(8, 3, 4);
        SQ_SK3_CH(8, 4);
    }
    if (p.rt == 1) SQ_SK3_CH(16, 1);
    if (p.rt == 3) SQ_SK3(16, 3, 4);
    SQ_SK3_CH(16, 4);
#undef SQ_SK3_CH
#undef SQ_SK3
}

// 17..32 tokens (any M <= 32 works), group size 128, K % 128 == 0, 64-row workgroups.  hipErrorInvalidValue when the
// shape does not fit: a K split without a workspace, or so few row blocks that most CUs would idle (the caller then
// takes the split-K kernel, which splits K further).
// The two-tile kernel runs 64 rows x 4096 columns per workgroup (RT 4, CH 4); a longer K is split over workgroups
// through the workspace.  Measured and dropped at 32 tokens: 128 rows x 2048 columns (a third fewer requests per
// unit of work, but every K is then split: fc1 19.0 against 16.5 us, q/k/v-sized weights 16.8 against 14.3) and
// 64 rows x 2048 columns (4096 x 4096, where the 4096-column shape has too few workgroups: 10.2 us, the split-K
// kernel's 10.1).  blocks64 = 64-row blocks of all linears of the launch together.
static bool wide_fits(long blocks64, int K, bool have_ws, int* ksplit) {
    if (K <= 0 || K % 128 != 0) return false;
    const int chunks = K / 128, ks = (chunks + 31) / 32;
    const int cps = (chunks + ks - 1) / ks;
    *ksplit = ks;
    return ks <= 8 && (ks == 1 || have_ws) && (ks - 1) * cps < chunks && blocks64 <= 16384 && blocks64 * ks >= 128;
}

bool skinny3_wide_applies(int N, int K, bool have_ws) {
    int ks;
    return wide_fits((N + 63) / 64, K, have_ws, &ks);
}

// The same with the grid it would run: workgroups, and how many of a workgroup's 32 chunk slots its K range fills.
bool skinny3_wide_shape(int N, int K, bool have_ws, long* workgroups, int* slots_in_use) {
    int ks;
    const long blocks64 = (N + 63) / 64;
    if (!wide_fits(blocks64, K, have_ws, &ks)) return false;
    *workgroups = blocks64 * ks;
    *slots_in_use = (K / 128 + ks - 1) / ks;
    return true;
}

// ws = the caller's workspace or null (then K is never split); it must hold skinny2_workspace_bytes(M, N, K).
hipError_t launch_skinny3_wide(const void* x, const void* w, const void* zs, void* y, void* ws, int M, int N, int K,
                               Epilogue epi, hipStream_t st) {
    int ksplit;
    if (M < 1 || M > 32 || !wide_fits((N + 63) / 64, K, ws != nullptr, &ksplit)) return hipErrorInvalidValue;
    static bool allowed[64];
    constexpr int lds = Sk3WideLds<4, 4>::BYTES;
    const hipError_t e = allow_lds(skinny3_wide_kernel<4, 4>, lds, allowed);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((skinny3_wide_kernel<4, 4>), dim3((N + 63) / 64, ksplit), dim3(SK3_NT), lds, st, (const uint8_t*)w,
                       (const uint32_t*)zs, (const half_t*)x, (half_t*)y,
                       ws ? (float*)((char*)ws + SK3_COUNTER_BYTES) : nullptr, (unsigned*)ws, M, N, K, ksplit, epi);
    return hipGetLastError();
}

hipError_t launch_skinny3_wide_group(const SeqProblem* probs, int count, int M, void* ws, size_t ws_bytes,
                                     hipStream_t st) {
    if (count < 2 || count > GEMV_GROUP_MAX || M < 1 || M > 32) return hipErrorInvalidValue;
    const int K = probs[0].K;
    Skinny3Group g;
    int blocks = 0;
    for (int p = 0; p < GEMV_GROUP_MAX; p++) {
        const SeqProblem& q = probs[p < count ? p : 0];
        if (q.K != K || q.group_size != 128) return hipErrorInvalidValue;
        g.W[p] = (const uint8_t*)q.w;
        g.ZS[p] = (const uint32_t*)q.zs;
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
    const bool have_ws = ws && ws_bytes >= skinny2_group_workspace_bytes(probs, count, M);
    int ksplit;
    if (!wide_fits(blocks, K, have_ws, &ksplit)) return hipErrorInvalidValue;
    static bool allowed[64];
    constexpr int lds = Sk3WideLds<4, 4>::BYTES;
    const hipError_t e = allow_lds(skinny3_wide_group_kernel<4, 4>, lds, allowed);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((skinny3_wide_group_kernel<4, 4>), dim3(blocks, ksplit), dim3(SK3_NT), lds, st, g,
                       ws ? (float*)((char*)ws + SK3_COUNTER_BYTES) : nullptr, (unsigned*)ws, M, K, ksplit);
    return hipGetLastError();
}

// Grouped launch: count in 2..GEMV_GROUP_MAX linears with the same K, group size 128, 5 <= M <= 16.
hipError_t launch_skinny3_group(const SeqProblem* probs, int count, int M, void* ws, size_t ws_bytes, hipStream_t st) {
    if (count < 2 || count > GEMV_GROUP_MAX || M < 1 || M > 16) return hipErrorInvalidValue;
    const int K = probs[0].K;
    if (K % 128 != 0) return hipErrorInvalidValue;
    int rows[GEMV_GROUP_MAX];
    int blocks64 = 0;
    for (int p = 0; p < count; p++) {
        if (probs[p].K != K || probs[p].group_size != 128) return hipErrorInvalidValue;
        rows[p] = probs[p].N;
        blocks64 += (probs[p].N + 63) / 64;
    }
    const Sk3Plan pl = plan(rows, count, K, ws != nullptr, 0, M);
    if (pl.ksplit == 0) return hipErrorInvalidValue;
    if (pl.ksplit > 1 && (blocks64 * (4 / pl.rt) > 16384 || ws_bytes < skinny2_group_workspace_bytes(probs, count, M)))
        return hipErrorInvalidValue;
#define SQ_SK3(MR, RT, CH) return launch_group_cfg<MR, RT, CH>(probs, count, ws, M, K, pl.ksplit, st)
#define SQ_SK3_CH(MR, RT)             \
    do {                              \
        if (pl.ch == 1) SQ_SK3(MR, RT, 1); \
        if (pl.ch == 2) SQ_SK3(MR, RT, 2); \
        SQ_SK3(MR, RT, 4);            \
    } while (0)
    if (M <= 4) {
        if (pl.rt == 1) SQ_SK3_CH(4, 1);
        if (pl.rt == 3) SQ_SK3(4, 3, 4);
        SQ_SK3_CH(4, 4);
    }
    if (M <= 8) {
        if (pl.rt == 1) SQ_SK3_CH(8, 1);
        if (pl.rt == 3) SQ_SK3(8, 3, 4);
        SQ_SK3_CH(8, 4);
    }
    if (pl.rt == 1) SQ_SK3_CH(16, 1);
    if (pl.rt == 3) SQ_SK3(16, 3, 4);
    SQ_SK3_CH(16, 4);
#undef SQ_SK3_CH
#undef SQ_SK3
}

}  // namespace sq
