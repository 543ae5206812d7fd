// A sequence of decode linears (M <= 4 tokens) in ONE persistent launch, layout L1.
// HBM-bandwidth bound: algorithmic bytes = sum over the linears of
// N*K/2 + (K/g)*N*4 + M*K*2 + M*N*2.
//
// Why.  A decode linear of 9..36 MB takes 1..4.5 us of HBM time, but every kernel launch
// costs about 2 us before its first byte arrives (dispatch, wave start, first-miss latency)
// and drains its tail with the memory system idle.  With one launch per linear those gaps
// are half of a decoder layer's time.  Weight addresses, however, do not depend on the
// previous linear's output: only the activations do.  This kernel keeps one workgroup
// resident per CU for the whole sequence and lets every streaming wave run a single,
// never-draining stream of weight loads across all linears; only the consumption of a
// linear's weights waits (at a grid barrier) for the activations the previous linear wrote.
//
// Roles.  A workgroup has 8 streaming waves and 4 control waves.
//   Streaming waves do nothing but: request weights, multiply, leave partial sums in LDS.
//   They never wait for anything but their own oldest weight load, so their loads stay in
//   flight across the ends of linears (vector memory operations retire in order: a wave that
//   waited for a store or for freshly written activations would drain its whole queue).
//   Control waves own everything that needs such a wait: they sum the partial sums, apply the
//   epilogue, store Y, run the grid barrier and stage the next linear's activations in LDS.
//
// Mapping (arithmetic as in the single-linear GEMV).  v_mfma_f32_4x4x4_16B_f16 multiplies
// 16 independent 4x4x4 blocks; in block b lane 4b+i supplies row i of A (tokens) and column i
// of B (weights of output row i) and receives D[0..3][i].  A wave-wide 128-bit load covers
// 4 rows x 256 contiguous bytes = 4 rows x 512 k (a "k-step").  Workgroup g owns the rows
// [g*R, (g+1)*R) of every linear (R = ceil(N / workgroups) rounded up to 4).  Its work on one
// linear is cut into sub-units of 4 rows x 2048 k (four k-steps = four loads per lane);
// sub-unit u goes to streaming wave u % 8.  Every wave walks the same list of entries (linear,
// turn); the loads of entry t + NBUF - 1 are issued before entry t is consumed, into a ring of
// NBUF register buffers, and the ring does not care where one linear ends and the next begins.
// A wave without a sub-unit in some turn loads a dummy line that stays in cache, so that the
// instruction stream (and with it the compiler's wait counts) is the same for every wave.
//
// Activations: the whole [M, K] input of the current linear is staged in LDS (K <= 16384:
// 32 KiB per token) with the per-32-k sums the zero-point fixup needs; row pitch K*2 + 16
// bytes keeps the 64 lanes of a 128-bit read on distinct slots.
//
// Grid barrier between dependent linears: Y is stored at the device-coherent level (sc1),
// the stores are waited for, one thread adds 1 to the linear's counter (relaxed, agent scope)
// and polls it until all workgroups have arrived; the next activations are read with sc1
// loads.  At the end every workgroup arrives at an exit counter and the last one clears all
// counters, so they are zero between launches.  The poll is bounded: if it runs out (a
// workgroup that never became resident), a sticky error word is set in the workspace and the
// kernel finishes with wrong results instead of hanging.
// (replaces back-to-back launches of w4a16_bs1_kernel / w4a16_bs2_kernel, reference:
// quantization/muxi/backend/w4a16_gemm.cuh:14-151,153-326, for the linears of one decoder
// layer, test/nvidia/module/opt/modeling_opt_ours.py:158-164,598-611)
#include "sq_common.h"
#include "sq_kernels.h"

namespace sq {

namespace {

constexpr int SEQ_SW = 8;                         // streaming waves
constexpr int SEQ_CW = 4;                         // control waves
constexpr int SEQ_NT = 64 * (SEQ_SW + SEQ_CW);
constexpr int SEQ_CT = 64 * SEQ_CW;
constexpr int SEQ_S = 4;                          // k-steps (128-bit loads per lane) per sub-unit
constexpr int SEQ_KSUB = 512 * SEQ_S;
constexpr int SEQ_NBUF = 2;
constexpr int SEQ_ERR_WORD = SEQ_MAX_LINEARS + 1;  // index of the sticky error word among the counters

struct SeqLinear {
    const uint8_t* w;
    const half2_t* zs;
    const half_t* x;
    half_t* y;
    const half_t* bias;
    const half_t* residual;
    int N, K, gshift, act;
    int rows;     // rows per workgroup (multiple of 4)
    int nch;      // sub-units per row group = ceil(K / 2048)
    int units;    // sub-units per workgroup = rows / 4 * nch
    int turns;    // entries per wave = max(1, ceil(units / 8))
    int barrier;  // 1: a grid barrier separates this linear from the previous one
    int restage;  // 1: the activations must be staged (0: same buffer as the previous linear)
    int kpad;     // K rounded up to 2048
    int pad_;
};

struct SeqArgs {
    SeqLinear p[SEQ_MAX_LINEARS];
    int count;
    int M;
    unsigned* counters;   // [count] barrier counters, [count] = exit counter, [SEQ_ERR_WORD] = sticky error word
    unsigned spin_limit;
    int xsum_off;         // byte offsets of the LDS regions behind the activations
    int red_off;
    int red_half;         // floats per half of the partial-sum buffer
    unsigned long long* trace;  // diagnostic instantiation only: 64 time stamps (100 MHz counter) per workgroup
};

// Slots of a workgroup's trace: 0 start, 1 first activations staged, then per linear l at 2 + 4l:
// streaming wave 0 done with its weights | control waves done storing Y | grid barrier passed (if any) |
// next activations staged (if they had to be); 60 = streaming wave 0 leaves, 61 = control waves leave.
template <bool TRACE>
__device__ __forceinline__ void stamp(const SeqArgs& a, int slot, bool who) {
    if (TRACE) {
        if (who) a.trace[(long)blockIdx.x * 64 + slot] = wall_clock64();
    }
}

// Workgroup barrier without the vector-memory drain of __syncthreads(): LDS operations are
// complete (lgkmcnt), vector loads of the streaming waves stay in flight.
__device__ __forceinline__ void wg_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// Eight device-coherent 128-bit loads, a workgroup barrier, then the wait for the loads: the other waves
// are released as soon as these requests are on their way, so that what they request next queues up
// behind them and not in front of them.
__device__ __forceinline__ void load8_coherent_x4_then_barrier(const float* const (&p)[8], float4_t (&v)[8]) {
    asm volatile(
        "global_load_dwordx4 %0, %8, off sc1\n\t"
        "global_load_dwordx4 %1, %9, off sc1\n\t"
        "global_load_dwordx4 %2, %10, off sc1\n\t"
        "global_load_dwordx4 %3, %11, off sc1\n\t"
        "global_load_dwordx4 %4, %12, off sc1\n\t"
        "global_load_dwordx4 %5, %13, off sc1\n\t"
        "global_load_dwordx4 %6, %14, off sc1\n\t"
        "global_load_dwordx4 %7, %15, off sc1\n\t"
        "s_barrier\n\t"
        "s_waitcnt vmcnt(0)"
        : "=&v"(v[0]), "=&v"(v[1]), "=&v"(v[2]), "=&v"(v[3]), "=&v"(v[4]), "=&v"(v[5]), "=&v"(v[6]), "=&v"(v[7])
        : "v"(p[0]), "v"(p[1]), "v"(p[2]), "v"(p[3]), "v"(p[4]), "v"(p[5]), "v"(p[6]), "v"(p[7])
        : "memory");
}

// `first`: this is the staging at the start of the kernel; its first batch of loads carries the barrier that
// releases the streaming waves.
template <int MROWS>
__device__ __forceinline__ void stage_activations(const SeqLinear& L, int M, uint8_t* xbuf, float* xsum, int ct,
                                                  bool first = false) {
    const int pitch = L.kpad * 2 + 16;
    const int words_per_row = L.kpad >> 3;  // 128-bit words
    const int words = MROWS * words_per_row;
    for (int base = 0; base < words; base += 8 * SEQ_CT) {
        const float* ptr[8];
        float4_t v[8];
        int mm[8], ww[8];
        bool ok[8], in[8];
#pragma unroll
        for (int q = 0; q < 8; q++) {
            const int idx = base + q * SEQ_CT + ct;
            mm[q] = idx / words_per_row;
            ww[q] = idx - mm[q] * words_per_row;
            in[q] = idx < words;
            ok[q] = in[q] && mm[q] < M && ww[q] * 8 < L.K;
            ptr[q] = (const float*)(L.x + (ok[q] ? (long)mm[q] * L.K + ww[q] * 8 : 0));
        }
        if (first && base == 0)
            load8_coherent_x4_then_barrier(ptr, v);
        else
            load8_coherent_x4(ptr, v);
#pragma unroll
        for (int q = 0; q < 8; q++) {
            if (!ok[q]) v[q] = (float4_t){0.f, 0.f, 0.f, 0.f};
            const half8_t h = bit_cast<half8_t>(v[q]);
            float lo = ((float)h[0] + (float)h[1]) + ((float)h[4] + (float)h[5]);
            float sum = lo + (((float)h[2] + (float)h[3]) + ((float)h[6] + (float)h[7]));
            sum = quad_sum(sum);
            lo = quad_sum(lo);
            if (in[q]) {
                *(float4_t*)(xbuf + mm[q] * pitch + ww[q] * 16) = v[q];
                if ((ct & 3) == 0) {
                    float* xs = xsum + ((ww[q] >> 2) * MROWS + mm[q]) * 2;
                    xs[0] = sum;
                    xs[1] = 960.f * lo;
                }
            }
        }
    }
}

template <int MROWS, bool TRACE>
__global__ __launch_bounds__(SEQ_NT) void gemv_seq_kernel(const SeqArgs a) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    uint8_t* xbuf = lds;                                   // [MROWS][pitch]
    float* xsum = (float*)(lds + a.xsum_off);              // [kpad / 32][MROWS][2]
    float* red0 = (float*)(lds + a.red_off);               // [2][units_max][MROWS][4]: partial sums, one half per linear parity

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wg = blockIdx.x;
    const int nwg = gridDim.x;
    const int M = a.M;
    const int count = a.count;

    if (wave >= SEQ_SW) {
        // ------------------------------------------------------------------ control waves
        const int ct = tid - 64 * SEQ_SW;
        stamp<TRACE>(a, 0, ct == 0);
        stage_activations<MROWS>(a.p[0], M, xbuf, xsum, ct, true);  // contains the barrier that starts the weight stream
        wg_barrier();  // activations of linear 0 are staged
        stamp<TRACE>(a, 1, ct == 0);
        for (int cl = 0; cl < count; cl++) {
            const SeqLinear& L = a.p[cl];
            const bool last = (cl == count - 1);
            const bool sync_next = !last && a.p[cl + 1].barrier;
            wg_barrier();  // A: every partial sum of this linear is in LDS
            const float* red = red0 + (cl & 1) * a.red_half;
            for (int t = ct; t < L.rows * MROWS; t += SEQ_CT) {
                const int m = t / L.rows;
                const int r = t - m * L.rows;
                const int n = wg * L.rows + r;
                if (n < L.N && m < M) {
                    const float* pr = red + ((r >> 2) * L.nch * MROWS + m) * 4 + (r & 3);
                    float v = 0.f;
                    for (int c = 0; c < L.nch; c++) v += pr[c * MROWS * 4];  // fixed order: bit-reproducible
                    if (L.bias) v += (float)L.bias[n];
                    if (L.act == 1) v = fmaxf(v, 0.f);
                    if (L.residual) {
                        const unsigned short rb = __hip_atomic_load((const unsigned short*)(L.residual + (long)m * L.N + n),
                                                                    __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        v += (float)bit_cast<half_t>(rb);
                    }
                    __hip_atomic_store((unsigned short*)(L.y + (long)m * L.N + n), bit_cast<unsigned short>((half_t)v),
                                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            }
            stamp<TRACE>(a, 2 + 4 * cl + 1, ct == 0);
            if (sync_next) {
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this workgroup's rows of Y have left the CU
                wg_barrier();                                      // A2
                if (ct == 0) {
                    __hip_atomic_fetch_add(&a.counters[cl], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    unsigned polls = 0;
                    while (__hip_atomic_load(&a.counters[cl], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < (unsigned)nwg) {
                        if (++polls > a.spin_limit) {
                            __hip_atomic_store(&a.counters[SEQ_ERR_WORD], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                            break;
                        }
                        __builtin_amdgcn_s_sleep(1);
                    }
                }
                wg_barrier();  // B1: every workgroup has stored its rows
            }
            stamp<TRACE>(a, 2 + 4 * cl + 2, ct == 0);
            if (!last && a.p[cl + 1].restage) {
                stage_activations<MROWS>(a.p[cl + 1], M, xbuf, xsum, ct);
                wg_barrier();  // B2: the next activations are staged
            }
            stamp<TRACE>(a, 2 + 4 * cl + 3, ct == 0);
        }
        // Exit: the last workgroup to get here clears every counter (all polls are over by then).
        if (ct == 0) {
            const unsigned old = __hip_atomic_fetch_add(&a.counters[count], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (old == (unsigned)(nwg - 1))
                for (int c = 0; c <= count; c++)
                    __hip_atomic_store(&a.counters[c], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        stamp<TRACE>(a, 61, ct == 0);
        return;
    }

    // ---------------------------------------------------------------------- streaming waves
    const NibbleMasks nm = nibble_masks();
    const int lane = tid & 63;
    const int i = lane & 3;
    const int b = lane >> 2;
    int total = 0;
    for (int l = 0; l < count; l++) total += a.p[l].turns;

    // Issue side of the ring: entry (il, ie) is the next one whose loads are requested.
    int il = 0, ie = 0, issued = 0;
    u32x4_t wq[SEQ_NBUF][SEQ_S];
    half2_t zq[SEQ_NBUF][SEQ_S];

    auto issue = [&](u32x4_t (&wb)[SEQ_S], half2_t (&zb)[SEQ_S]) {
        // This lane's first k-step of the entry, or a dummy line (all lanes the same 16 bytes).
        const uint8_t* wrow = a.p[0].w;
        const half2_t* zrow = a.p[0].zs;
        int k0 = 0, K = 0, gshift = 5;
        if (issued < total) {
            const SeqLinear& L = a.p[il];
            const int u = ie * SEQ_SW + wave;
            if (u < L.units) {
                const int rg = u / L.nch;
                const int c = u - rg * L.nch;
                const int row = imin(wg * L.rows + 4 * rg + i, L.N - 1);
                wrow = L.w + (long)row * (L.K >> 1);
                zrow = L.zs + (long)row * (L.K >> L.gshift);
                k0 = c * SEQ_KSUB;
                K = L.K;
                gshift = L.gshift;
            }
            if (++ie == L.turns) {
                ie = 0;
                il++;
            }
        }
        issued++;
#pragma unroll
        for (int s = 0; s < SEQ_S; s++) {
            const int kk = k0 + 512 * s + 32 * b;
            const int kc = kk < K ? kk : 0;
            wb[s] = __builtin_nontemporal_load((const u32x4_t*)(wrow + (kc >> 1)));
            zb[s] = zrow[kc >> gshift];
        }
        asm volatile("" ::: "memory");
    };

    asm volatile("s_barrier" ::: "memory");  // the control waves' first activation loads are on their way
#pragma unroll
    for (int j = 0; j < SEQ_NBUF - 1; j++) issue(wq[j], zq[j]);
    wg_barrier();  // activations of linear 0 are staged

    int cl = 0, ce = 0;  // consume side: entry (cl, ce)
    // The loads are issued unconditionally, once per ring slot and turn of the loop (past the last entry
    // they fetch the dummy line), so that the number of loads between a request and its use is the same on
    // every path and the wait counts the compiler derives keep the whole ring in flight.
    for (int t0 = 0; t0 < total; t0 += SEQ_NBUF) {
#pragma unroll
        for (int j = 0; j < SEQ_NBUF; j++) {
            issue(wq[(j + SEQ_NBUF - 1) % SEQ_NBUF], zq[(j + SEQ_NBUF - 1) % SEQ_NBUF]);
            if (t0 + j < total) {
                const SeqLinear& L = a.p[cl];
                const int u = ce * SEQ_SW + wave;
                float* red = red0 + (cl & 1) * a.red_half;
                if (u < L.units) {
                    const int rg = u / L.nch;
                    const int c = u - rg * L.nch;
                    const int pitch = L.kpad * 2 + 16;
                    float4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int s = 0; s < SEQ_S; s++) {
                        const int kb = c * SEQ_KSUB + 512 * s + 32 * b;
                        const uint8_t* xp = xbuf + (i & (MROWS - 1)) * pitch + kb * 2;
                        half8_t xa[4];
#pragma unroll
                        for (int q = 0; q < 4; q++) xa[q] = *(const half8_t*)(xp + 16 * q);
                        float4_t tmp = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                        for (int q = 0; q < 4; q++) {
                            const half8_t wv = unpack8_mixed(wq[j][s][q], nm);
                            tmp = __builtin_amdgcn_mfma_f32_4x4x4f16(xa[q].lo, wv.lo, tmp, 0, 0, 0);
                            tmp = __builtin_amdgcn_mfma_f32_4x4x4f16(xa[q].hi, wv.hi, tmp, 0, 0, 0);
                        }
                        const float zf = (float)zq[j][s].x;
                        const float sf = (float)zq[j][s].y;
                        const float* xs = xsum + (kb >> 5) * MROWS * 2;
#pragma unroll
                        for (int m = 0; m < MROWS; m++) acc[m] += sf * ((tmp[m] - xs[2 * m + 1]) - zf * xs[2 * m]);
                    }
                    // fold the 16 blocks of the wave; lanes 0..3 hold rows 4*rg + 0..3
#pragma unroll
                    for (int m = 0; m < MROWS; m++) {
                        float v = row_sum_stride4(acc[m]);
                        v += __shfl_xor(v, 16);
                        v += __shfl_xor(v, 32);
                        if (lane < 4) red[(u * MROWS + m) * 4 + i] = v;
                    }
                }
                if (ce == L.turns - 1) {
                    const bool last = (cl == count - 1);
                    const bool sync_next = !last && a.p[cl + 1].barrier;
                    stamp<TRACE>(a, 2 + 4 * cl, tid == 0);
                    wg_barrier();  // A
                    if (sync_next) {
                        wg_barrier();  // A2
                        wg_barrier();  // B1
                    }
                    if (!last && a.p[cl + 1].restage) wg_barrier();  // B2
                    cl++;
                    ce = 0;
                } else {
                    ce++;
                }
            }
        }
    }
    stamp<TRACE>(a, 60, tid == 0);
}

int g_cus[64] = {};

int cu_count() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
    if (g_cus[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
        g_cus[dev] = n;
    }
    return g_cus[dev];
}

template <int MROWS, bool TRACE>
hipError_t launch_m(const SeqArgs& a, int grid, size_t lds_bytes, hipStream_t st) {
    static bool attr_set[64] = {};
    int dev = 0;
    (void)hipGetDevice(&dev);
    auto kern = gemv_seq_kernel<MROWS, TRACE>;
    if (dev >= 0 && dev < 64 && !attr_set[dev]) {
        const hipError_t e =
            hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, SEQ_LDS_LIMIT);
        if (e != hipSuccess) return e;
        attr_set[dev] = true;
    }
    hipLaunchKernelGGL(kern, dim3(grid), dim3(SEQ_NT), lds_bytes, st, a);
    return hipGetLastError();
}

}  // namespace

size_t gemv_seq_workspace_bytes() { return 256; }

int launch_gemv_seq(const SeqProblem* probs, int count, int M, void* workspace, unsigned spin_limit, hipStream_t st,
                    unsigned long long* trace) {
    if (count < 1 || count > SEQ_MAX_LINEARS || M < 1 || M > 4) return 1;
    const int grid = cu_count();
    if (grid <= 0) return 2;
    const int mrows = M <= 1 ? 1 : (M <= 2 ? 2 : 4);
    SeqArgs a;
    a.count = count;
    a.M = M;
    a.counters = (unsigned*)workspace;
    a.spin_limit = spin_limit;
    a.trace = trace;
    int kpad_max = 0, units_max = 0;
    for (int l = 0; l < count; l++) {
        const SeqProblem& q = probs[l];
        SeqLinear& L = a.p[l];
        L.w = (const uint8_t*)q.w;
        L.zs = (const half2_t*)q.zs;
        L.x = (const half_t*)q.x;
        L.y = (half_t*)q.y;
        L.bias = (const half_t*)q.bias;
        L.residual = (const half_t*)q.residual;
        L.N = q.N;
        L.K = q.K;
        L.gshift = 0;
        while ((1 << L.gshift) < q.group_size) L.gshift++;
        L.act = q.act;
        L.rows = (((q.N + grid - 1) / grid) + 3) & ~3;
        L.kpad = ((q.K + SEQ_KSUB - 1) / SEQ_KSUB) * SEQ_KSUB;
        L.nch = L.kpad / SEQ_KSUB;
        L.units = (L.rows / 4) * L.nch;
        L.turns = (L.units + SEQ_SW - 1) / SEQ_SW;
        if (L.turns < 1) L.turns = 1;
        L.barrier = (l > 0 && q.depends) ? 1 : 0;
        L.restage = (l == 0 || q.depends || q.x != probs[l - 1].x || q.K != probs[l - 1].K) ? 1 : 0;
        L.pad_ = 0;
        if (L.kpad > kpad_max) kpad_max = L.kpad;
        if (L.units > units_max) units_max = L.units;
    }
    for (int l = count; l < SEQ_MAX_LINEARS; l++) a.p[l] = a.p[0];
    const size_t xbuf_bytes = (size_t)mrows * ((size_t)kpad_max * 2 + 16);
    const size_t xsum_bytes = (size_t)(kpad_max / 32) * mrows * 2 * sizeof(float);
    a.red_half = units_max * mrows * 4;
    const size_t red_bytes = 2 * (size_t)a.red_half * sizeof(float);
    a.xsum_off = (int)((xbuf_bytes + 15) & ~(size_t)15);
    a.red_off = (int)((a.xsum_off + xsum_bytes + 15) & ~(size_t)15);
    const size_t lds_bytes = a.red_off + red_bytes;
    if (lds_bytes > SEQ_LDS_LIMIT) return 1;
    hipError_t e;
    if (trace)
        e = mrows == 1 ? launch_m<1, true>(a, grid, lds_bytes, st)
                       : (mrows == 2 ? launch_m<2, true>(a, grid, lds_bytes, st) : launch_m<4, true>(a, grid, lds_bytes, st));
    else if (mrows == 1)
        e = launch_m<1, false>(a, grid, lds_bytes, st);
    else if (mrows == 2)
        e = launch_m<2, false>(a, grid, lds_bytes, st);
    else
        e = launch_m<4, false>(a, grid, lds_bytes, st);
    return e == hipSuccess ? 0 : 2;
}

}  // namespace sq
